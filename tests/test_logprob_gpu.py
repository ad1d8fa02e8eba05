"""Parity of the HIP logprob kernel (through the C ABI) with the CPU oracle.  Needs an MI355X.

Tolerance: 1e-4 absolute on the fp32 output against the fp32 torch CPU path, as the operator's
specification states; the fp64 evaluation is checked at 2e-5.  Determinism checks are bit-exact.
"""
import math

import pytest
import torch

from benchmarks.workloads import cfg1_logits, spike_block, spike_logits
from oracle import logprob_ref as O

pytestmark = pytest.mark.gpu
TOL = 1e-4
TOL64 = 2e-5


def _check(sampler, logits_cpu, ids_cpu, **kw):
    got = sampler.compute_logp(logits_cpu.cuda(), ids_cpu.cuda(), **kw).cpu()
    want = O.logprob_ref(logits_cpu, ids_cpu)
    truth = O.logprob_f64(logits_cpu, ids_cpu)
    assert got.dtype == torch.float32 and got.shape == want.shape
    assert (got - want).abs().max().item() <= TOL
    assert (got.double() - truth).abs().max().item() <= TOL64
    return got


def test_cfg1_parity(sampler):
    logits, ids = cfg1_logits()
    got = _check(sampler, logits, ids)
    assert got.shape == (4, 128)


def test_llama_vocab_spike_rows(sampler):
    logits, ids = spike_block(1024, 128256, seed=0, block=0, device="cpu", spike_frac=0.05)
    _check(sampler, logits, ids)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_other_dtypes(sampler, dtype):
    g = torch.Generator().manual_seed(11)
    logits = (torch.randn(64, 32000, generator=g) * 2.0).to(dtype)
    ids = torch.randint(0, 32000, (64,), generator=g)
    _check(sampler, logits, ids)


@pytest.mark.parametrize("vocab", [1, 2, 7, 8, 9, 63, 64, 255, 2047, 2049, 32003, 151936])
def test_ragged_vocab(sampler, vocab):
    g = torch.Generator().manual_seed(vocab)
    logits = (torch.randn(5, vocab, generator=g) * 3.0).bfloat16()
    ids = torch.randint(0, vocab, (5,), generator=g)
    _check(sampler, logits, ids)


def test_unaligned_and_strided_rows(sampler):
    g = torch.Generator().manual_seed(12)
    big = (torch.randn(16, 4104, generator=g) * 3.0).bfloat16().cuda()
    ids = torch.randint(0, 4001, (16,), generator=g)
    for view in (big[:, 3:4004], big[:, 8:4009], big[:, :4096]):  # odd offset, aligned offset + ragged, strided
        got = sampler.compute_logp(view, ids.cuda()).cpu()
        want = O.logprob_ref(view.cpu().contiguous(), ids)
        assert (got - want).abs().max().item() <= TOL


def test_empty_and_single_row(sampler):
    out = sampler.compute_logp(torch.empty(0, 7, 128, dtype=torch.bfloat16, device="cuda"),
                               torch.empty(0, 7, dtype=torch.int64, device="cuda"))
    assert out.shape == (0, 7)
    logits = torch.randn(1, 1, 640).bfloat16()
    _check(sampler, logits, torch.tensor([[639]]))


def test_closed_forms(sampler):
    v = 128256
    x = torch.zeros(3, v, dtype=torch.bfloat16)
    x[0, 777] = 25.0
    x[1, 777] = 25.0
    ids = torch.tensor([777, 5, 9])
    got = sampler.compute_logp(x.cuda(), ids.cuda()).cpu().double()
    l = math.log1p((v - 1) * math.exp(-25.0))
    assert abs(got[0].item() + l) < 1e-5
    assert abs(got[1].item() + 25.0 + l) < 1e-5
    assert abs(got[2].item() + math.log(v)) < 1e-5


def test_masked_vocab_and_degenerate_rows(sampler):
    g = torch.Generator().manual_seed(13)
    x = (torch.randn(6, 4096, generator=g) * 3).bfloat16()
    x[:, 1000:] = -math.inf          # whole lanes see only -inf
    x[4, :] = -math.inf              # all -inf row -> NaN, as torch
    x[5, 17] = math.inf              # +inf -> NaN, as torch
    ids = torch.tensor([0, 999, 5, 2000, 1, 17])
    got = sampler.compute_logp(x.cuda(), ids.cuda()).cpu()
    want = O.logprob_ref(x, ids)
    assert (got[:3] - want[:3]).abs().max().item() <= TOL
    assert got[3].item() == -math.inf and want[3].item() == -math.inf
    assert math.isnan(got[4].item()) and math.isnan(want[4].item())
    assert math.isnan(got[5].item()) and math.isnan(want[5].item())


def test_out_of_range_id_gives_nan(sampler):
    x = torch.zeros(2, 64, dtype=torch.bfloat16, device="cuda")
    got = sampler.compute_logp(x, torch.tensor([64, -1], device="cuda")).cpu()
    assert torch.isnan(got).all()


def test_probabilities_sum_to_one(sampler):
    g = torch.Generator().manual_seed(14)
    row = (torch.randn(1, 2048, generator=g) * 3).bfloat16()
    got = sampler.compute_logp(row.expand(2048, 2048).contiguous().cuda(), torch.arange(2048).cuda()).cpu()
    assert abs(got.double().exp().sum().item() - 1.0) < 1e-5


def test_reference_output_dtype_option(sampler):
    logits, ids = cfg1_logits()
    got = sampler.compute_logp(logits.cuda(), ids.cuda(), out_dtype=torch.bfloat16)
    assert got.dtype == torch.bfloat16 and got.shape == (4, 128)
    assert torch.equal(got.cpu(), sampler.compute_logp(logits.cuda(), ids.cuda()).cpu().bfloat16())


def test_bit_identical_across_runs_splits_and_chunks(sampler):
    logits, ids = spike_logits(4096, 128256, seed=1, device="cuda")
    base = sampler.compute_logp(logits, ids)
    for _ in range(3):
        assert torch.equal(base, sampler.compute_logp(logits, ids))
    for chunk in (1, 7, 1024, 4096, 1 << 20):
        assert torch.equal(base, sampler.compute_logp(logits, ids, chunk_tokens=chunk))
    for split in (1, 64, 1000):
        parts = [sampler.compute_logp(logits[s:s + split], ids[s:s + split]) for s in range(0, 4096, split)][:8]
        assert torch.equal(base[:sum(p.numel() for p in parts)], torch.cat(parts))
    view3d = sampler.compute_logp(logits.view(8, 512, -1), ids.view(8, 512))
    assert torch.equal(view3d.view(-1), base)


def test_entropy_variant(sampler):
    logits, ids = spike_block(512, 128256, seed=2, block=0, device="cpu", spike_frac=0.05)
    lp, ent = sampler.compute_logp_entropy(logits.cuda(), ids.cuda())
    assert torch.equal(lp, sampler.compute_logp(logits.cuda(), ids.cuda()))
    assert (ent.cpu().double() - O.entropy_f64(logits)).abs().max().item() <= TOL
    masked = logits.clone()
    masked[:, 5000:] = -math.inf
    _, ent2 = sampler.compute_logp_entropy(masked.cuda(), ids.cuda() % 5000)
    assert (ent2.cpu().double() - O.entropy_f64(masked)).abs().max().item() <= TOL


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_entropy_variant_other_dtypes(sampler, dtype):
    """fp16 and fp32 logits through the same pass (aligned rows, and an unaligned view that takes the scalar loads)."""
    g = torch.Generator().manual_seed(17)
    logits = (torch.randn(96, 40003, generator=g) * 3).to(dtype)
    logits[::7, 11] = 20.0
    logits[5, 2000:] = -math.inf
    ids = torch.randint(0, 2000, (96,), generator=g)
    aligned = logits[:, :40000].contiguous()
    for x in (aligned, logits[:, 3:40003]):
        lp, ent = sampler.compute_logp_entropy(x.cuda(), ids.cuda())
        assert torch.equal(lp, sampler.compute_logp(x.cuda(), ids.cuda()))
        assert (lp.cpu().double() - O.logprob_f64(x, ids)).abs().max().item() <= 2e-5
        assert (ent.cpu().double() - O.entropy_f64(x)).abs().max().item() <= TOL
    with pytest.raises(ValueError, match="chunk_tokens"):
        sampler.compute_logp_entropy(aligned.cuda(), ids.cuda(), chunk_tokens=-4)


def test_full_size_grpo_group(sampler):
    """[256, 512, 128256] bf16 (33.6 GB): parity on sampled blocks, invariance on everything."""
    n_rows, vocab, blk = 256 * 512, 128256, 2048
    free, _ = torch.cuda.mem_get_info()
    if free < 40 << 30:
        pytest.skip("needs 40 GB of free HBM")
    logits, ids = spike_logits(n_rows, vocab, seed=0, device="cuda", rows_per_block=blk)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    whole = sampler.compute_logp(logits.view(256, 512, vocab), ids.view(256, 512))
    torch.cuda.synchronize()
    extra = torch.cuda.max_memory_allocated() - before
    assert extra <= 512 << 20, f"extra device memory {extra} B"
    assert whole.shape == (256, 512)
    flat = whole.view(-1)
    # batch invariance: four G=64 groups, and other launch granularities, give the same bits
    groups = torch.cat([sampler.compute_logp(logits[s:s + 64 * 512].view(64, 512, vocab),
                                             ids[s:s + 64 * 512].view(64, 512)).view(-1)
                        for s in range(0, n_rows, 64 * 512)])
    assert torch.equal(flat, groups)
    assert torch.equal(flat, sampler.compute_logp(logits, ids, chunk_tokens=n_rows))
    assert torch.equal(flat, sampler.compute_logp(logits, ids, chunk_tokens=5000))
    # oracle parity on three whole blocks (first, middle, last) and on every spike row of the tensor (found on the
    # device: a spike is +25, N(0, 3^2) stays below 16): both branches of the spike closed form are hit, since every
    # fourth spike row targets its spike
    for b in (0, 31, 63):
        s = b * blk
        lc, ic = logits[s:s + blk].cpu(), ids[s:s + blk].cpu()
        assert (flat[s:s + blk].cpu() - O.logprob_ref(lc, ic)).abs().max().item() <= TOL
    spike_rows = torch.cat([(logits[s:s + blk].max(dim=-1).values.float() >= 24.0).nonzero().squeeze(-1) + s
                            for s in range(0, n_rows, blk)])
    assert 1000 <= spike_rows.numel() <= 1700                          # Bernoulli(0.01) of 131,072 rows
    ls, isp = logits[spike_rows].cpu(), ids[spike_rows].cpu()
    got_spike = flat[spike_rows].cpu()
    assert (got_spike - O.logprob_ref(ls, isp)).abs().max().item() <= TOL
    on_spike = ls.float().argmax(dim=-1) == isp
    assert 200 <= int(on_spike.sum()) <= 500
    lse_minus_c = math.log1p((vocab - 1) * math.exp(-25.0 + 4.5))      # crude bound: the rest of the row is exp(N(0, 9))
    assert (got_spike[on_spike] > -lse_minus_c - 0.5).all() and (got_spike[on_spike] <= 0).all()
    # every row is a proper log-probability; spike rows that target their spike are ~0
    assert torch.isfinite(flat).all() and (flat <= 0).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rows_that_start_with_masked_entries(sampler, dtype):
    """A masked prefix (the first entries of the row are -inf) leaves lanes whose first groups hold nothing but -inf:
    their running maximum stays at its floor for a while, and the rescale factor between two equal floors must be
    exactly 1 (an FMA contraction there would return the rounding residue of a 1e30-sized product).  Compared with
    the oracle, for logprob, entropy and the gradient."""
    g = torch.Generator().manual_seed(29)
    logits = (torch.randn(12, 128256, generator=g) * 3).to(dtype)
    logits[0, :70000] = -math.inf
    logits[1, :1000] = -math.inf
    logits[2, 1::2] = -math.inf                      # every other entry
    logits[3, :] = -math.inf
    logits[3, 128255] = 1.0                          # a single finite entry at the very end
    ids = torch.randint(70000, 128256, (12,), generator=g)
    ids[2] = 2 * (ids[2] // 2)
    ids[3] = 128255
    got = sampler.compute_logp(logits.cuda(), ids.cuda()).cpu()
    assert torch.isfinite(got).all()
    assert (got.double() - O.logprob_f64(logits, ids)).abs().max().item() <= 2e-5
    assert abs(got[3].item()) <= 1e-6                # a single finite entry: probability 1
    lp, ent = sampler.compute_logp_entropy(logits.cuda(), ids.cuda())
    assert torch.equal(lp.cpu(), got) and (ent.cpu().double() - O.entropy_f64(logits)).abs().max().item() <= TOL
    grad = torch.randn(12, generator=g)
    d = sampler.compute_logp_backward(logits.cuda(), ids.cuda(), lp, grad.cuda()).cpu().double()
    want = O.logprob_backward_closed_form(logits, ids, grad)
    rel = 2.0 ** -8 if dtype == torch.bfloat16 else 1e-5
    assert ((d - want).abs() <= rel * want.abs() + 1e-6).all()
