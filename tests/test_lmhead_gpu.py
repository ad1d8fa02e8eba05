"""Parity of the fused lm_head -> logprob kernel (bf16 MFMA, fp32 accumulate) with the CPU oracle.

Tolerance 1e-4 absolute on the fp32 output against the fp32/fp64 CPU evaluation of
logprob(hidden @ W^T); determinism checks are bit-exact.  Needs an MI355X.
"""
import math

import pytest
import torch

from oracle import logprob_ref as O

pytestmark = pytest.mark.gpu
TOL = 1e-4


def make(n, h, v, seed, w_scale=0.02):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, h, generator=g).bfloat16()
    weight = (torch.randn(v, h, generator=g) * w_scale).bfloat16()
    ids = torch.randint(0, v, (n,), generator=g)
    return hidden, weight, ids


@pytest.mark.parametrize("n,h,v", [(1, 64, 1), (5, 64, 7), (300, 256, 1000), (256, 128, 256), (257, 192, 16129),
                                   (64, 4096, 2048), (700, 512, 16385)])
def test_small_shapes_against_fp64(sampler, n, h, v):
    hidden, weight, ids = make(n, h, v, seed=n + h + v, w_scale=0.2)
    got = sampler.fused_linear_logp(hidden.cuda(), weight.cuda(), ids.cuda()).cpu()
    want = O.lmhead_logprob_ref(hidden, weight, ids, dtype=torch.float64)
    assert got.shape == (n,) and got.dtype == torch.float32
    assert (got.double() - want).abs().max().item() <= TOL


@pytest.mark.parametrize("n,h,v", [(9000, 64, 5000),      # 36 token blocks: eight groups walked XCD-resident + one left over;
                                                            # one hidden slab per tile, so the copy cursor crosses items at once
                                   (8300, 128, 70000),     # 274 vocabulary tiles = 40 splits (5 split groups), two slabs per tile
                                   (16640, 64, 300)])      # 65 token blocks, two tiles = two one-tile splits
def test_many_token_blocks_walk_several_items_per_workgroup(sampler, n, h, v):
    """More (token block, split) items than CUs: every workgroup walks several items and its copy pipeline runs
    across their boundaries.  Checked against the CPU oracle, and bit for bit against a short call on the
    first rows (the split plan depends on the vocabulary only)."""
    hidden, weight, ids = make(n, h, v, seed=n + v, w_scale=0.2)
    hg, wg, ig = hidden.cuda(), weight.cuda(), ids.cuda()
    got = sampler.fused_linear_logp(hg, wg, ig)
    want = O.lmhead_logprob_ref(hidden, weight, ids, dtype=torch.float32 if v > 10000 else torch.float64)
    assert (got.cpu().double() - want.double()).abs().max().item() <= TOL
    assert torch.equal(got[:300], sampler.fused_linear_logp(hg[:300], wg, ig[:300]))
    assert torch.equal(got[-517:], sampler.fused_linear_logp(hg[-517:], wg, ig[-517:]))


@pytest.mark.parametrize("seed", range(4))
def test_randomised_shapes(sampler, seed):
    """Random row counts (1 .. 40 token blocks and a ragged last one), hidden sizes and vocabularies (1 .. 160
    tiles with a ragged last one): every (token block, split) item order and split plan against the oracle."""
    rng = torch.Generator().manual_seed(1000 + seed)
    for _ in range(5):
        h = int(torch.randint(1, 5, (1,), generator=rng)) * 64
        v = int(torch.randint(1, 40000, (1,), generator=rng))
        n = int(torch.randint(1, 10000, (1,), generator=rng))
        while n * v * h > 2.5e10:                              # keep the CPU oracle within a second or two
            n = n // 2 + 1
        hidden, weight, ids = make(n, h, v, seed=n + v + h, w_scale=0.15)
        got = sampler.fused_linear_logp(hidden.cuda(), weight.cuda(), ids.cuda()).cpu()
        want = O.lmhead_logprob_ref(hidden, weight, ids, dtype=torch.float32)
        assert (got - want).abs().max().item() <= TOL, (n, h, v)


def test_llama_shape_slice(sampler):
    hidden, weight, ids = make(384, 4096, 128256, seed=0)
    got = sampler.fused_linear_logp(hidden.cuda(), weight.cuda(), ids.cuda()).cpu()
    want = O.lmhead_logprob_ref(hidden, weight, ids, dtype=torch.float32)
    assert (got - want).abs().max().item() <= TOL
    # and it agrees with the unfused path on an fp32 linear layer computed by torch on the GPU
    logits = torch.nn.functional.linear(hidden.cuda().float(), weight.cuda().float())
    unfused = sampler.compute_logp(logits, ids.cuda()).cpu()
    assert (got - unfused).abs().max().item() <= TOL


def test_full_baseline_shape(sampler):
    """hidden [32768, 4096] x W [128256, 4096] (generated on the device): 64 scattered rows against the fp32 CPU
    oracle, and two row ranges bit for bit against calls of their own."""
    g = torch.Generator(device="cuda").manual_seed(0)
    hidden = torch.randn(32768, 4096, generator=g, device="cuda").bfloat16()
    weight = (torch.randn(128256, 4096, generator=g, device="cuda") * 0.02).bfloat16()
    ids = torch.randint(0, 128256, (32768,), generator=g, device="cuda")
    got = sampler.fused_linear_logp(hidden, weight, ids)
    assert torch.isfinite(got).all()
    pick = torch.randperm(32768, generator=torch.Generator().manual_seed(1))[:64].sort().values
    want = O.lmhead_logprob_ref(hidden[pick.cuda()].cpu(), weight.cpu(), ids[pick.cuda()].cpu(), dtype=torch.float32)
    assert (got[pick.cuda()].cpu() - want).abs().max().item() <= TOL
    # calls of few rows run every split as four work items and fold them in the second kernel: same bits
    for lo, hi in ((0, 64), (0, 256), (20000, 20600), (20000, 20777), (31000, 32768)):
        assert torch.equal(got[lo:hi], sampler.fused_linear_logp(hidden[lo:hi], weight, ids[lo:hi]))
    lp, ent = sampler.fused_linear_logp(hidden[:8192], weight, ids[:8192], return_entropy=True)
    lp64, ent64 = sampler.fused_linear_logp(hidden[100:164], weight, ids[100:164], return_entropy=True)
    assert torch.equal(lp, got[:8192]) and torch.equal(lp64, got[100:164]) and torch.equal(ent64, ent[100:164])


def test_weight_matrix_above_4_gib(sampler):
    """W [300000, 8192] bf16 is 4.9 GB: row offsets beyond 32 bits.  Rows with targets in the last part of the
    vocabulary against the fp32 CPU oracle, all rows against the unfused path on the GPU."""
    g = torch.Generator(device="cuda").manual_seed(5)
    vocab, hdim, n = 300000, 8192, 320
    weight = torch.empty(vocab, hdim, dtype=torch.bfloat16, device="cuda")
    for lo in range(0, vocab, 50000):                                    # generated in pieces: no 9.8 GB fp32 temporary
        weight[lo:lo + 50000] = (torch.randn(50000, hdim, generator=g, device="cuda") * 0.02).bfloat16()
    hidden = torch.randn(n, hdim, generator=g, device="cuda").bfloat16()
    ids = torch.randint(0, vocab, (n,), generator=g, device="cuda")
    ids[:8] = torch.tensor([vocab - 1, vocab - 2, 262144, 262143, 280000, 299999 - 256, 0, 131072], device="cuda")
    got = sampler.fused_linear_logp(hidden, weight, ids)
    logits = torch.cat([torch.nn.functional.linear(hidden.float(), weight[lo:lo + 50000].float())
                        for lo in range(0, vocab, 50000)], dim=1)
    unfused = sampler.compute_logp(logits, ids)
    assert (got - unfused).abs().max().item() <= TOL
    want = O.lmhead_logprob_ref(hidden[:8].cpu(), weight.cpu(), ids[:8].cpu(), dtype=torch.float32)
    assert (got[:8].cpu() - want).abs().max().item() <= TOL
    # the backward's gradient matrix from the same (wide-addressing) kernel against the unfused logits on the GPU
    got2, lse = sampler.fused_linear_logp(hidden, weight, ids, return_lse=True)
    assert torch.equal(got2, got)
    assert (lse - torch.logsumexp(logits, -1)).abs().max().item() <= TOL
    grad = torch.randn(n, generator=g, device="cuda")
    dl = torch.empty(n, vocab, dtype=torch.bfloat16, device="cuda")
    from rl_engine.kernels import _hip
    _hip.check(sampler._lib.ka_lmhead_dlogits_bf16(hidden.data_ptr(), weight.data_ptr(), ids.data_ptr(), lse.data_ptr(),
                                                   grad.data_ptr(), dl.data_ptr(), vocab, n, hdim, vocab,
                                                   torch.cuda.current_stream().cuda_stream), "ka_lmhead_dlogits_bf16")
    want_dl = -torch.softmax(logits, -1) * grad[:, None]
    want_dl[torch.arange(n, device="cuda"), ids] += grad
    assert ((dl.float() - want_dl).abs() <= 2.0 ** -7 * want_dl.abs() + 1e-6).all()


def test_leading_dims_and_invalid_ids(sampler):
    hidden, weight, ids = make(96, 128, 3000, seed=3, w_scale=0.2)
    ids[5], ids[6] = 3000, -2
    got = sampler.fused_linear_logp(hidden.view(8, 12, 128).cuda(), weight.cuda(), ids.view(8, 12).cuda()).cpu()
    assert got.shape == (8, 12)
    flat = got.view(-1)
    assert math.isnan(flat[5].item()) and math.isnan(flat[6].item())
    keep = torch.ones(96, dtype=torch.bool)
    keep[5] = keep[6] = False
    want = O.lmhead_logprob_ref(hidden[keep], weight, ids[keep], dtype=torch.float64)
    assert (flat[keep].double() - want).abs().max().item() <= TOL
    with pytest.raises(ValueError):
        sampler.fused_linear_logp(hidden[:, :80].contiguous().cuda(), weight[:, :80].contiguous().cuda(), ids.cuda())


def test_bit_identical_across_runs_and_row_counts(sampler):
    hidden, weight, ids = make(1500, 1024, 40000, seed=4)
    h, w, i = hidden.cuda(), weight.cuda(), ids.cuda()
    base = sampler.fused_linear_logp(h, w, i)
    assert torch.equal(base, sampler.fused_linear_logp(h, w, i))
    # 1 .. 64 rows: the 64-token kernel; 65 .. 128: the 128-token kernel; above: the 256-token kernel (with units as work
    # items while token blocks x splits < 256: every call here; the test at the benchmark shape crosses into whole splits)
    for n in (1, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 1024, 1281):
        assert torch.equal(base[:n], sampler.fused_linear_logp(h[:n], w, i[:n])), n
    lp, ent = sampler.fused_linear_logp(h, w, i, return_entropy=True)
    for n in (63, 65, 128, 300):
        lp_n, ent_n = sampler.fused_linear_logp(h[100:100 + n], w, i[100:100 + n], return_entropy=True)
        assert torch.equal(lp_n, base[100:100 + n]) and torch.equal(ent_n, ent[100:100 + n]), n
    assert torch.equal(base[600:900], sampler.fused_linear_logp(h[600:900], w, i[600:900]))


def test_rows_are_sliced_to_fit_a_small_workspace_pool(sampler):
    """With a pool too small for all rows the wrapper feeds the kernel 256-row multiples; the result is
    bit-identical to the single call (every row's reduction order is fixed)."""
    from rl_engine.kernels.pool import PoolExhausted
    from rl_engine.kernels.sampling import SamplerBackend

    hidden, weight, ids = make(1000, 128, 40000, seed=9)
    per_row = sampler._lib.ka_lmhead_workspace_bytes(1 << 20, 128, 40000) >> 20   # 16 B per vocabulary split
    assert per_row % 16 == 0 and per_row >= 48
    base = sampler.fused_linear_logp(hidden.cuda(), weight.cuda(), ids.cuda())
    # (calls of so few rows keep one partial per unit of a split: four times per_row)
    small = SamplerBackend(pool_bytes=4 * 300 * per_row).cuda()          # room for 300 rows -> slices of 256
    assert torch.equal(small.fused_linear_logp(hidden.cuda(), weight.cuda(), ids.cuda()), base)
    tiny = SamplerBackend(pool_bytes=4 * 100 * per_row).cuda()                # less than one tile of a long input
    with pytest.raises(PoolExhausted):
        tiny.fused_linear_logp(hidden.cuda(), weight.cuda(), ids.cuda())
    assert torch.equal(tiny.fused_linear_logp(hidden[:64].cuda(), weight.cuda(), ids[:64].cuda()), base[:64])


def test_one_backend_shared_by_two_streams_and_two_threads(sampler):
    """Calls on different streams (and from different host threads) share the backend's one workspace arena: the
    pool orders them, so each result equals the sequential call's bit for bit.  Two inputs whose partials
    overlap in the arena; were the kernels of the two streams to run in it at once, one would fold the other's
    partials."""
    import threading

    a = tuple(t.cuda() for t in make(2048, 512, 30000, seed=31))
    b = tuple(t.cuda() for t in make(1792, 512, 30000, seed=32))
    want_a, want_b = sampler.fused_linear_logp(*a), sampler.fused_linear_logp(*b)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for _ in range(3):
        with torch.cuda.stream(s1):
            got_a = sampler.fused_linear_logp(*a)
        with torch.cuda.stream(s2):
            got_b = sampler.fused_linear_logp(*b)
        with torch.cuda.stream(s1):
            got_a2 = sampler.fused_linear_logp(*a)
        torch.cuda.synchronize()
        assert torch.equal(got_a, want_a) and torch.equal(got_b, want_b) and torch.equal(got_a2, want_a)

    results, errors = {}, []

    def worker(name, args, stream):
        try:
            with torch.cuda.stream(stream):
                outs = [sampler.fused_linear_logp(*args) for _ in range(4)]
            stream.synchronize()
            results[name] = outs
        except Exception as exc:  # noqa: BLE001
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=("a", a, s1)), threading.Thread(target=worker, args=("b", b, s2))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert all(torch.equal(o, want_a) for o in results["a"]) and all(torch.equal(o, want_b) for o in results["b"])


@pytest.mark.parametrize("n,h,v", [(5, 64, 7), (300, 256, 1000), (257, 192, 16129), (700, 512, 16385), (384, 4096, 128256)])
def test_entropy_from_the_same_pass(sampler, n, h, v):
    """fused_linear_logp(..., return_entropy=True): the log-probabilities are those of the plain call bit for bit
    (the entropy accumulator does not touch the max / sum arithmetic), and the entropy matches the fp64 entropy of
    softmax(hidden @ W^T) - ragged last tile and last token block included."""
    hidden, weight, ids = make(n, h, v, seed=3 * n + v, w_scale=0.2 if v < 100000 else 0.02)
    hg, wg, ig = hidden.cuda(), weight.cuda(), ids.cuda()
    lp, ent = sampler.fused_linear_logp(hg, wg, ig, return_entropy=True)
    assert torch.equal(lp, sampler.fused_linear_logp(hg, wg, ig))
    assert ent.shape == (n,) and ent.dtype == torch.float32
    if v > 100000:
        logits = torch.nn.functional.linear(hidden[:64].double(), weight.double())
        want = O.entropy_f64(logits)
        assert (ent[:64].cpu().double() - want).abs().max().item() <= TOL
        # and the unfused route on the device agrees on every row
        lp2, ent2 = sampler.compute_logp_entropy(torch.nn.functional.linear(hg.float(), wg.float()), ig)
        assert (ent - ent2).abs().max().item() <= TOL
    else:
        want = O.entropy_f64(torch.nn.functional.linear(hidden.double(), weight.double()))
        assert (ent.cpu().double() - want).abs().max().item() <= TOL
    assert (ent > 0).all() and (ent.cpu() <= math.log(v) + 1e-4).all()
