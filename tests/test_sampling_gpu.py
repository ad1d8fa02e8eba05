"""Parity of the HIP sampling kernel (through the C ABI) with the CPU oracles.  Needs an MI355X.

Token ids must be bit-exact against oracle/ka_oracle.c (the exactly specified definition) on
every row, and against the torch restatement of the reference's native_sampling on every row
whose threshold decisions are not within fp32 rounding noise of a tie (on the benchmark
configuration that is every row).
"""
import math

import pytest
import torch

from benchmarks.workloads import cfg5_sampling
from oracle import exact, sampling_ref
from rl_engine.kernels import _hip

pytestmark = pytest.mark.gpu
DTYPES = [torch.bfloat16, torch.float16, torch.float32]


def run(sampler, logits, u, k, p, temp, route_flags=0):
    return sampler.sample(logits.cuda(), top_k=k, top_p=p, temperature=temp, uniforms=u.cuda(),
                          route_flags=route_flags).cpu()


# shortest, block-wide top-k, radix; the short top-k route on 512 and on 1024 threads per row (where the row qualifies)
ROUTES = (0, _hip.SAMPLE_FLAG_BLOCK_WIDE_TOPK, _hip.SAMPLE_FLAG_GENERAL_PATH, _hip.SAMPLE_FLAG_TWO_ROWS_PER_CU,
          _hip.SAMPLE_FLAG_ONE_ROW_PER_CU)


def check_exact(sampler, logits, u, k, p, temp):
    got = run(sampler, logits, u, k, p, temp)
    want = exact.sample(logits, temp, k, p, u)
    assert got.dtype == torch.int64 and got.shape == want.shape
    bad = (got != want).nonzero().flatten().tolist()
    assert not bad, f"rows {bad[:8]}: got {got[bad[:8]].tolist()} want {want[bad[:8]].tolist()}"
    return got


@pytest.mark.parametrize("batch", [64, 128, 256])
def test_baseline_config_bit_exact(sampler, batch):
    logits, u = cfg5_sampling(batch)
    got = check_exact(sampler, logits, u, 50, 0.9, 0.7)
    ref, margin = sampling_ref.sample(logits, 50, 0.9, 0.7, u)
    assert margin.min().item() > 1e-6
    assert torch.equal(got, ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k,p,temp", [(50, 0.9, 0.7), (50, None, 1.0), (None, 0.9, 1.0), (None, None, 1.0),
                                      (None, None, 0.7), (1, None, 1.0), (1, 0.5, 1.3), (5000, 0.99, 0.5),
                                      (50, 1e-6, 1.0), (2, 1.0, 1.0)])
def test_modes_and_dtypes(sampler, dtype, k, p, temp):
    g = torch.Generator().manual_seed(21)
    logits = (torch.randn(48, 32000, generator=g) * 3).to(dtype)
    u = torch.rand(48, generator=g)
    got = check_exact(sampler, logits, u, k, p, temp)
    ref, margin = sampling_ref.sample(logits, k, p, temp, u)
    differ = got != ref
    assert (margin[differ] < 1e-6).all() and differ.sum().item() <= 1


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k,p,temp", [(5, 0.9, 0.7), (5, None, 1.0), (None, 0.8, 1.0), (17, 0.05, 1.0),
                                      (200, 0.95, 0.5), (3, 1.0, 2.0)])
def test_heavy_ties_and_degenerate_rows(sampler, dtype, k, p, temp):
    g = torch.Generator().manual_seed(22)
    logits = ((torch.randn(40, 3000, generator=g) * 12).round() / 4).to(dtype)
    u = torch.rand(40, generator=g)
    logits[0, :] = 1.5                       # all equal: every entry ties at the k-th value and at the cut
    logits[1, :] = -math.inf                 # only -inf
    logits[2, 7] = math.inf                  # +inf wins outright
    logits[3, :2500] = -math.inf             # masked prefix
    logits[4, :] = 0.0
    logits[4, 100:200] = -0.0                # signed zeros are one value
    logits[5, 5] = 30.0                      # one dominant entry: everything else has mass ~0
    logits[6, :] = -2.0                      # all equal and negative: the cut key is a negative value
    logits[7] = -logits[7].abs() - 1.0       # only negative values, coarse grid: negative ties at k-th value and cut
    logits[8, :] = -math.inf
    logits[8, 10:40] = -7.5                  # few finite negative entries over a -inf background
    check_exact(sampler, logits, u, k, p, temp)


@pytest.mark.parametrize("value", [0.0, -3.0, 2.5])
def test_all_equal_llama_row_cut_inside_tie_group(sampler, value):
    logits = torch.full((4, 128256), value, dtype=torch.bfloat16)
    u = torch.tensor([0.0, 0.25, 0.5, 0.999])
    got = check_exact(sampler, logits, u, 50, 0.3, 0.7)
    kept = math.floor(float(torch.tensor(0.3, dtype=torch.float32)) * 128256) + 1
    assert got.tolist() == [math.floor(float(x) * kept) for x in u]


@pytest.mark.parametrize("vocab", [1, 2, 7, 8, 9, 63, 1000, 2047, 8193, 32003, 151936])
def test_ragged_vocab(sampler, vocab):
    g = torch.Generator().manual_seed(vocab)
    logits = (torch.randn(6, vocab, generator=g) * 3).bfloat16()
    u = torch.rand(6, generator=g)
    check_exact(sampler, logits, u, 50, 0.9, 0.7)
    check_exact(sampler, logits, u, None, 0.9, 1.0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("vocab", [131080, 151936, 262144 + 1032])
def test_rows_longer_than_the_register_file(sampler, dtype, vocab):
    """Rows above 131,072 entries stay on the histogram path (a wavefront's share of the row is searched in
    rounds of sixteen steps); every filter combination against the exact oracle, draws spread over the row."""
    g = torch.Generator().manual_seed(vocab)
    logits = (torch.randn(8, vocab, generator=g) * (3 if dtype == torch.bfloat16 else 1.5)).to(dtype)
    logits[3, vocab // 2:] = float("-inf")                    # masked second half
    logits[4] = logits[4, 0]                                   # one value: the draw is uniform over the row
    u = torch.tensor([0.0, 0.03, 0.31, 0.5, 0.77, 0.93, 0.999, 0.9999999])
    for k, p, t in [(None, None, 1.0), (None, 0.9, 0.7), (None, 0.999, 1.3), (2000, 0.9, 0.7), (50, 0.9, 0.7)]:
        check_exact(sampler, logits, u, k, p, t)


@pytest.mark.parametrize("dtype,vocab", [(torch.float32, 151936), (torch.float32, 300004), (torch.bfloat16, 600008),
                                         (torch.float16, 262144)])
def test_top_k_on_rows_longer_than_the_tracked_maxima(sampler, dtype, vocab):
    """The top-k fast path keeps 32 maxima per lane; above 32,768 vectors a maximum covers several vectors."""
    g = torch.Generator().manual_seed(vocab + 1)
    logits = (torch.randn(8, vocab, generator=g) * 2.5).to(dtype)
    logits[2, : vocab - 5] = float("-inf")                    # fewer entries than top_k above -inf
    logits[5, vocab // 3] = 30.0
    u = torch.tensor([0.0, 0.11, 0.35, 0.5, 0.62, 0.8, 0.97, 0.9999999])
    for k, p, t in [(50, 0.9, 0.7), (1, None, 1.0), (1000, 0.95, 1.0), (7, None, 1.5)]:
        check_exact(sampler, logits, u, k, p, t)


def test_unaligned_and_strided_rows(sampler):
    g = torch.Generator().manual_seed(23)
    big = (torch.randn(12, 4104, generator=g) * 3).bfloat16()
    u = torch.rand(12, generator=g)
    for view in (big[:, 3:4004], big[:, 8:4009], big[:, :4096]):
        got = sampler.sample(view.cuda(), top_k=20, top_p=0.9, temperature=0.7, uniforms=u.cuda()).cpu()
        assert torch.equal(got, exact.sample(view.contiguous(), 0.7, 20, 0.9, u))


def test_extreme_uniforms(sampler):
    logits, _ = cfg5_sampling(8, vocab=32000)
    for val in (0.0, 2.0 ** -149, 1 - 2.0 ** -24, 1.0, 7.0, -1.0, float("nan")):
        check_exact(sampler, logits, torch.full((8,), val), 50, 0.9, 0.7)


def test_every_bf16_value_through_the_temperature_step(sampler):
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    finite = bits[torch.isfinite(bits.float())]
    g = torch.Generator().manual_seed(24)
    rows = torch.stack([finite[torch.randperm(finite.numel(), generator=g)] for _ in range(4)])
    rows = torch.where(rows.float().abs() > 60, torch.zeros_like(rows), rows)   # keep exp() in range
    u = torch.rand(4, generator=g)
    for temp in (0.7, 1.3, 0.01):
        check_exact(sampler, rows, u, 300, 0.95, temp)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_temperature_rule_against_torch_division_on_the_device(dtype):
    """The operator's temperature step is the true quotient round_dtype(float(x) / T) (what torch's CPU division
    returns, which is the oracle the parity target names).  torch's own GPU division by a Python scalar multiplies
    by the fp32 reciprocal instead.  At the benchmark temperature (0.7) and at 1.3 / 0.01 / 0.9 the two rules agree
    on every finite 16-bit pattern; at e.g. 0.6 they differ on about 1.5 % of the patterns, which is recorded
    here so that a change of either side shows up."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
    x = bits[torch.isfinite(bits.float())]
    for temp in (0.7, 1.3, 0.01, 0.9):
        on_device = (x.cuda() / temp).cpu().float()
        assert torch.equal(on_device, exact.scale(x, temp)), temp
    on_device = (x.cuda() / 0.6).cpu().float()
    reciprocal = (x.float() * (torch.tensor(1.0) / torch.tensor(0.6))).to(dtype).float()
    assert torch.equal(on_device, reciprocal)                          # the device rule, restated
    differ = int((on_device != exact.scale(x, 0.6)).sum())
    assert 0 < differ < 0.03 * x.numel()
    assert torch.equal((x / 0.6).float(), exact.scale(x, 0.6))         # the oracle is the CPU quotient


def test_bit_identical_across_runs_and_batch_splits(sampler):
    logits, u = cfg5_sampling(256)
    dl, du = logits.cuda(), u.cuda()
    base = sampler.sample(dl, top_k=50, top_p=0.9, temperature=0.7, uniforms=du)
    for _ in range(3):
        assert torch.equal(base, sampler.sample(dl, top_k=50, top_p=0.9, temperature=0.7, uniforms=du))
    for split in (1, 64, 100):
        parts = [sampler.sample(dl[s:s + split], top_k=50, top_p=0.9, temperature=0.7, uniforms=du[s:s + split])
                 for s in range(0, 256, split)][:6]
        cat = torch.cat(parts)
        assert torch.equal(base[:cat.numel()], cat)


def test_reference_call_shapes_and_generated_uniforms(sampler):
    logits = torch.randn(16, 128256, device="cuda")                      # fp32, as benchmark_sampling.py:58
    ids = sampler.sample(logits, top_k=50, top_p=0.9)
    assert ids.shape == (16,) and ids.dtype == torch.int64 and ids.device.type == "cuda"
    assert ((ids >= 0) & (ids < 128256)).all()
    g1 = torch.Generator(device="cuda").manual_seed(5)
    g2 = torch.Generator(device="cuda").manual_seed(5)
    assert torch.equal(sampler.sample(logits, top_k=50, generator=g1), sampler.sample(logits, top_k=50, generator=g2))
    top1 = sampler.sample(logits, top_k=1)
    assert torch.equal(top1, logits.argmax(dim=-1))
    assert sampler.sample(logits[:0], top_k=5).shape == (0,)


def test_invalid_arguments_raise(sampler):
    logits = torch.zeros(2, 64, dtype=torch.bfloat16, device="cuda")
    for kw in (dict(top_k=0), dict(top_k=-3), dict(top_p=0.0), dict(top_p=1.5), dict(temperature=0.0),
               dict(temperature=-1.0)):
        with pytest.raises(ValueError):
            sampler.sample(logits, **kw)
    with pytest.raises(RuntimeError):
        sampler.sample(logits.cpu(), top_k=5)
    with pytest.raises(ValueError):
        sampler.sample(logits, uniforms=torch.zeros(3, device="cuda"))


def test_fast_and_radix_paths_are_the_same_function(sampler):
    """top_k <= 1024 normally runs on a candidate list in LDS (for top_k <= 64 with wavefront-local sorts and a
    one-wavefront tail, else block-wide); the route flags force the block-wide variant and the radix descents.
    All must return the same ids (and each is checked against the oracle)."""
    g = torch.Generator().manual_seed(31)
    cases = []
    for dtype in DTYPES:
        cases.append((torch.randn(32, 50000, generator=g).mul(3).to(dtype), 50, 0.9, 0.7))
        cases.append((((torch.randn(32, 6000, generator=g) * 8).round() / 4).to(dtype), 7, 0.6, 1.0))   # heavy ties
        cases.append((torch.randn(32, 3000, generator=g).to(dtype), 1000, None, 1.9))
        cases.append((torch.zeros(4, 128256).to(dtype), 50, 0.3, 0.7))                                  # overflow -> radix
    for logits, k, p, temp in cases:
        u = torch.rand(logits.shape[0], generator=g)
        want = exact.sample(logits, temp, k, p, u)
        for f in ROUTES:
            assert torch.equal(run(sampler, logits, u, k, p, temp, f), want), f"route_flags={f}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_wavefront_route_of_small_top_k(sampler, dtype):
    """top_k <= 256 takes the short route (bound from pooled group maxima up to 64, from a radix descent above; tail on
    one wavefront with 1 to 8 candidates per lane); beyond 512 candidates, or with top_k = 257, the block-wide route
    takes over.
    Rows are built to hit each of those sizes: smooth rows (few candidates), coarse grids (tie groups of tens to
    hundreds of entries at the k-th value), a cut inside a tie group, the largest values packed into the share of
    one lane / one wavefront (loose bounds), and all three routes must give the oracle's ids and log-probabilities."""
    g = torch.Generator().manual_seed(77)
    vocab = 40000
    smooth = (torch.randn(16, vocab, generator=g) * 3)
    coarse = (torch.randn(16, vocab, generator=g) * 3 * 2).round() / 2        # ~90 entries per value near the top
    coarser = (torch.randn(16, vocab, generator=g) * 2).round()               # hundreds per value: above 256 candidates
    packed = torch.randn(16, vocab, generator=g)
    packed[:, :8 * 40] += 6.0                                                 # the top values sit in the vectors of 40 lanes
    packed[8:, 8 * 64 * 3:8 * 64 * 4] += 9.0                                  # ... and in one wavefront's lanes
    flat = torch.zeros(4, vocab)
    flat[:, 5::97] = 1.0                                                      # 413 entries tie at the maximum
    for rows, temps in ((smooth, (0.7, 1.0)), (coarse, (1.0, 0.5)), (coarser, (1.0,)), (packed, (0.7,)), (flat, (1.0,))):
        logits = rows.to(dtype)
        u = torch.rand(logits.shape[0], generator=g)
        for k in (1, 2, 17, 50, 63, 64, 65, 130, 200, 256, 257):
            for p in (None, 0.9, 0.3):
                for temp in temps:
                    want, want_lp = exact.sample_rows(logits, temp, k, p, u)
                    for flags in ROUTES:
                        ids, lp = sampler.sample(logits.cuda(), top_k=k, top_p=p, temperature=temp, uniforms=u.cuda(),
                                                 return_logprob=True, route_flags=flags)
                        assert torch.equal(ids.cpu(), want), (k, p, temp, flags)
                        assert (lp.cpu().double() - want_lp).abs().max().item() < 1e-5


def test_unknown_route_flag_is_refused(sampler):
    logits, u = cfg5_sampling(4, vocab=1000)
    with pytest.raises(ValueError, match="flag"):
        sampler.sample(logits.cuda(), top_k=5, uniforms=u.cuda(), route_flags=16)
    with pytest.raises(ValueError, match="flag"):   # the two workgroup sizes exclude each other
        sampler.sample(logits.cuda(), top_k=5, uniforms=u.cuda(),
                       route_flags=_hip.SAMPLE_FLAG_TWO_ROWS_PER_CU | _hip.SAMPLE_FLAG_ONE_ROW_PER_CU)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("vocab", [128256, 131072, 4096, 1000])
def test_two_rows_per_cu_build_returns_the_same_bits(sampler, dtype, vocab):
    """The short top-k route on 512 threads per row (two rows resident per CU, what a batch of more rows than CUs gets)
    against the same route on 1024 threads: ids, filtered log-probability and policy log-probability bit for bit, on
    ordinary rows, a tie group of half the row, an all-equal row and a row with five numbers above -inf (the last three
    leave the short route, in either build for its own reason); ids also against the exact oracle."""
    g = torch.Generator().manual_seed(77)
    batch = 12
    logits = (torch.randn(batch, vocab, generator=g) * 3).to(dtype)
    logits[0, : vocab // 2] = 1.5
    logits[1] = 0.25
    logits[2, 5:] = float("-inf")
    u = torch.rand(batch, generator=g)
    dev_logits, dev_u = logits.cuda(), u.cuda()
    for k in (1, 50, 64, 65, 256):
        for p, temp in ((None, 1.0), (0.9, 0.7), (0.3, 50.0)):
            one = sampler.sample(dev_logits, top_k=k, top_p=p, temperature=temp, uniforms=dev_u, return_logprob=True,
                                 return_policy_logprob=True, route_flags=_hip.SAMPLE_FLAG_ONE_ROW_PER_CU)
            two = sampler.sample(dev_logits, top_k=k, top_p=p, temperature=temp, uniforms=dev_u, return_logprob=True,
                                 return_policy_logprob=True, route_flags=_hip.SAMPLE_FLAG_TWO_ROWS_PER_CU)
            assert torch.equal(one[0], two[0]), (k, p, temp)
            assert torch.equal(one[1].view(torch.int32), two[1].view(torch.int32)), (k, p, temp)
            assert torch.equal(one[2].view(torch.int32), two[2].view(torch.int32)), (k, p, temp)
            assert torch.equal(two[0].cpu(), exact.sample(logits, temp, k, p, u)), (k, p, temp)


def test_random_shapes_and_parameters_on_both_workgroup_sizes(sampler):
    """Forty seeded draws of (dtype, aligned vocabulary size, batch, top_k <= 256, top_p, temperature), rows with ties
    mixed in: both builds of the short top-k route against the exact oracle, ids and filtered log-probability."""
    rnd = torch.Generator().manual_seed(2024)
    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=rnd))]
    for case in range(40):
        dtype = pick(DTYPES)
        epv = 4 if dtype == torch.float32 else 8
        vocab = epv * int(torch.randint(1, 6000, (1,), generator=rnd))
        batch = pick([1, 3, 17, 40])
        k = min(int(torch.randint(1, 257, (1,), generator=rnd)), vocab - 1) if vocab > 1 else None
        p = pick([None, 0.95, 0.9, 0.5, 0.1])
        temp = pick([1.0, 0.7, 1.3, 0.05, 20.0])
        logits = (torch.randn(batch, vocab, generator=rnd) * pick([0.5, 3.0, 8.0]))
        if case % 3 == 0:
            logits = (logits * 2).round() / 2                      # heavy ties
        logits = logits.to(dtype)
        u = torch.rand(batch, generator=rnd)
        if k is None:
            continue
        want, want_lp = exact.sample_rows(logits, temp, k, p, u)
        for flags in (_hip.SAMPLE_FLAG_TWO_ROWS_PER_CU, _hip.SAMPLE_FLAG_ONE_ROW_PER_CU):
            ids, lp = sampler.sample(logits.cuda(), top_k=k, top_p=p, temperature=temp, uniforms=u.cuda(),
                                     return_logprob=True, route_flags=flags)
            assert torch.equal(ids.cpu(), want), (case, dtype, vocab, batch, k, p, temp, flags)
            assert (lp.cpu().double() - want_lp).abs().max().item() < 1e-5, (case, flags)


def test_a_batch_of_more_rows_than_cus_matches_its_rows_sampled_in_small_batches(sampler):
    """The library switches to two rows per CU above one row per CU: ids and both log-probabilities of a 600-row call are
    those of the same rows in calls of 200."""
    logits, u = cfg5_sampling(600)
    dev_logits, dev_u = logits.cuda(), u.cuda()
    big = sampler.sample(dev_logits, top_k=50, top_p=0.9, temperature=0.7, uniforms=dev_u, return_logprob=True,
                         return_policy_logprob=True)
    for lo in (0, 200, 400):
        part = sampler.sample(dev_logits[lo:lo + 200], top_k=50, top_p=0.9, temperature=0.7, uniforms=dev_u[lo:lo + 200],
                              return_logprob=True, return_policy_logprob=True)
        for a, b in zip(big, part):
            assert torch.equal(a[lo:lo + 200].view(torch.int32 if a.dtype == torch.float32 else a.dtype),
                               b.view(torch.int32 if b.dtype == torch.float32 else b.dtype))
    assert torch.equal(big[0].cpu(), exact.sample(logits, 0.7, 50, 0.9, u))


def test_huge_temperature_folds_values_together(sampler):
    g = torch.Generator().manual_seed(32)
    logits = (torch.randn(8, 20000, generator=g) * 3).bfloat16()
    u = torch.rand(8, generator=g)
    for temp in (1e3, 1e30, 3e38):
        check_exact(sampler, logits, u, 50, 0.9, temp)


@pytest.mark.parametrize("dtype", DTYPES)
def test_per_row_parameters_and_sampled_logprob(sampler, dtype):
    g = torch.Generator().manual_seed(41)
    batch, vocab = 40, 20000
    logits = (torch.randn(batch, vocab, generator=g) * 3).to(dtype)
    logits[3] = ((logits[3].float() * 2).round() / 2).to(dtype)          # ties
    u = torch.rand(batch, generator=g)
    ks = torch.randint(1, 200, (batch,), generator=g).to(torch.int32)
    ks[0], ks[1], ks[2] = 0, -5, 5000                                     # off, invalid -> off, radix path
    ps = (torch.rand(batch, generator=g) * 0.9 + 0.05)
    ps[4], ps[5] = 1.0, 7.0                                               # off, invalid -> off
    ts = (torch.rand(batch, generator=g) * 1.5 + 0.3)
    ts[6], ts[7] = 1.0, -2.0                                              # identity, invalid -> 1
    want_ids, want_lp = exact.sample_rows(logits, ts, ks, ps, u)
    for flags in ROUTES:
        ids, lp = sampler.sample(logits.cuda(), top_k=ks.cuda(), top_p=ps.cuda(), temperature=ts.cuda(),
                                 uniforms=u.cuda(), return_logprob=True, route_flags=flags)
        assert torch.equal(ids.cpu(), want_ids)
        assert (lp.cpu().double() - want_lp).abs().max().item() < 1e-5
        assert (lp <= 0).all()
    # scalar parameters through the extended entry point give the scalar entry point's ids
    ids2, lp2 = sampler.sample(logits.cuda(), top_k=50, top_p=0.9, temperature=0.7, uniforms=u.cuda(), return_logprob=True)
    assert torch.equal(ids2, sampler.sample(logits.cuda(), top_k=50, top_p=0.9, temperature=0.7, uniforms=u.cuda()))
    w_ids, w_lp = exact.sample_rows(logits, 0.7, 50, 0.9, u)
    assert torch.equal(ids2.cpu(), w_ids) and (lp2.cpu().double() - w_lp).abs().max().item() < 1e-5
    # mixing a per-row tensor with scalars
    ids3 = sampler.sample(logits.cuda(), top_k=ks.cuda(), top_p=0.8, temperature=1.0, uniforms=u.cuda())
    assert torch.equal(ids3.cpu(), exact.sample_rows(logits, 1.0, ks, 0.8, u)[0])
    # the log-probability is the one of the filtered distribution: top_k = 1 -> log 1 = 0 without ties
    _, lp_greedy = sampler.sample(torch.randn(8, 1000, generator=g).cuda(), top_k=1, uniforms=u[:8].cuda(), return_logprob=True)
    assert (lp_greedy == 0).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_nan_and_infinite_logits_on_both_paths(sampler, dtype):
    """NaN counts as -inf, +inf takes all the mass, rows with fewer than top_k numbers above -inf keep their
    -inf entries: same ids from the candidate-list path, the radix path and the oracle."""
    g = torch.Generator().manual_seed(43)
    base = (torch.randn(24, 5000, generator=g) * 3).to(dtype)
    holes = torch.rand(24, 5000, generator=g) < 0.3
    nan_rows = base.clone(); nan_rows[holes] = float("nan")
    sparse = torch.full((24, 5000), float("-inf")).to(dtype)            # 10 numbers per row, the rest masked / NaN
    cols = torch.randint(0, 5000, (24, 10), generator=g)
    sparse.scatter_(1, cols, (torch.randn(24, 10, generator=g) * 2).to(dtype))
    sparse[:, ::7] = torch.where(torch.isinf(sparse[:, ::7].float()), torch.tensor(float("nan")).to(dtype), sparse[:, ::7])
    pinf = base.clone(); pinf[:, 123] = float("inf"); pinf[::2, 4000] = float("inf")
    allnan = torch.full((4, 5000), float("nan")).to(dtype)
    u = torch.rand(24, generator=g)
    for logits, k, p, temp in [(nan_rows, 50, 0.9, 0.7), (nan_rows, None, 0.8, 1.0), (sparse, 50, 0.9, 0.7),
                               (sparse, 5, None, 1.3), (pinf, 50, 0.9, 0.7), (pinf, None, None, 1.0),
                               (allnan, 50, 0.9, 0.7)]:
        uu = u[:logits.shape[0]]
        want = exact.sample(logits, temp, k, p, uu)
        for flags in ROUTES:
            got = run(sampler, logits, uu, k, p, temp, flags)
            assert torch.equal(got, want), f"route_flags={flags} k={k} p={p} T={temp}"


def test_mass_function_is_bit_exact_against_the_oracle(sampler):
    """W(d) on the GPU (ka_sample_mass_fixed) against oracle/ka_oracle.c for 200k random d in (-31, 0], every
    d = -i/256, and the special values: the integers every sampled id is built from must be identical."""
    import ctypes
    g = torch.Generator().manual_seed(77)
    d = torch.cat([-torch.rand(200000, generator=g) * 31, -torch.arange(0, 8192) / 256.0,
                   torch.tensor([0.0, -0.0, -1e-38, -1e-8, -28.4, -28.42, -28.5, -40.0, -88.0, -1e30, -math.inf,
                                 math.nan, 1.0])]).float()
    dd = d.cuda()
    out = torch.empty(d.numel(), dtype=torch.int64, device="cuda")
    lib = sampler._lib
    rc = lib.ka_sample_mass_fixed(dd.data_ptr(), d.numel(), out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    got = out.cpu().tolist()
    want = [exact.weight(x) for x in d.tolist()]
    bad = [(x, a, b) for x, a, b in zip(d.tolist(), got, want) if a != b]
    assert not bad, bad[:5]


@pytest.mark.parametrize("seed", range(6))
def test_randomised_shapes_modes_and_value_grids(sampler, seed):
    """A sweep over the paths behind `sample`: random vocabulary sizes (ragged tails, tiny rows, rows of one
    tile, rows longer than the register-resident limit), value grids from continuous to heavily tied, all
    three dtypes, every filter combination.  Every id must equal the exact oracle's."""
    g = torch.Generator().manual_seed(1000 + seed)
    vocabs = [1, 7, 8, 9, 1023, 1024, 8191, 8192, 8200, 40000, 65537, 128256, 131072, 131080, 140001]
    for trial in range(10):
        vocab = vocabs[int(torch.randint(0, len(vocabs), (1,), generator=g))]
        dtype = DTYPES[int(torch.randint(0, 3, (1,), generator=g))]
        rows = 6
        spread = float(torch.rand(1, generator=g)) * 6 + 0.2
        logits = torch.randn(rows, vocab, generator=g) * spread
        grid = [0.0, 0.0, 0.25, 1.0, 4.0][int(torch.randint(0, 5, (1,), generator=g))]
        if grid:
            logits = (logits / grid).round() * grid                     # ties: few distinct values
        logits = logits.to(dtype)
        k = [None, None, 1, 5, 50, 1024, 1025, 3000, vocab, vocab + 5][int(torch.randint(0, 10, (1,), generator=g))]
        p = [None, None, 0.05, 0.5, 0.9, 0.999, 1.0][int(torch.randint(0, 7, (1,), generator=g))]
        temp = [1.0, 1.0, 0.7, 1.3, 0.05, 25.0][int(torch.randint(0, 6, (1,), generator=g))]
        u = torch.rand(rows, generator=g)
        got = run(sampler, logits, u, k, p, temp)
        want = exact.sample(logits, temp, k, p, u)
        assert torch.equal(got, want), (f"trial {trial}: vocab={vocab} dtype={dtype} grid={grid} spread={spread:.2f} "
                                        f"k={k} p={p} T={temp}: rows {(got != want).nonzero().flatten().tolist()}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_temperature_merges_raw_values_into_tie_groups(sampler, dtype):
    """The histogram path counts raw values and scales only the occupied ones; raw values that round to the
    same scaled value must act as one tie group (top-k ties kept, top-p cut by index order across them)."""
    g = torch.Generator().manual_seed(51)
    u = torch.rand(12, generator=g)
    for spread, temp in [(3.0, 3.0), (3.0, 25.0), (0.5, 7.0), (6.0, 1000.0), (3.0, 0.31)]:
        logits = (torch.randn(12, 30000, generator=g) * spread).to(dtype)
        for k, p in [(None, 0.9), (None, 0.3), (2000, None), (1500, 0.95), (None, 0.999)]:
            check_exact(sampler, logits, u, k, p, temp)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_masked_vocabulary_rows(sampler, dtype):
    """Constrained decoding masks most of the vocabulary with -inf: more equal entries than a 16-bit histogram
    counter holds.  Every mode must still return the oracle's ids (and never a masked id)."""
    g = torch.Generator().manual_seed(61)
    vocab = 128256
    logits = (torch.randn(8, vocab, generator=g) * 3).to(dtype)
    masked = torch.rand(8, vocab, generator=g) < 0.8                       # ~102,600 entries per row
    logits[masked] = float("-inf")
    logits[7] = float("-inf")                                              # a fully masked row: uniform draw
    logits[6, :] = float("-inf"); logits[6, 77] = 1.5                      # one admissible token
    u = torch.rand(8, generator=g)
    for k, p, temp in [(None, None, 1.0), (None, 0.9, 0.7), (2000, None, 1.0), (50, 0.9, 0.7), (None, 0.5, 1.3),
                       (40000, 0.95, 1.0)]:
        got = check_exact(sampler, logits, u, k, p, temp)
        assert not masked[torch.arange(6), got[:6]].any()
        assert got[6] == 77


def test_more_rows_than_compute_units(sampler):
    """Batches beyond the 256 CUs of the part (several workgroups per CU in turn): ids against the oracle."""
    g = torch.Generator().manual_seed(91)
    logits = (torch.randn(1500, 4104, generator=g) * 3).bfloat16()
    u = torch.rand(1500, generator=g)
    for k, p, temp in ((50, 0.9, 0.7), (None, 0.9, 1.0), (None, None, 0.7), (300, None, 1.0)):
        check_exact(sampler, logits, u, k, p, temp)
    big, ub = cfg5_sampling(600)
    got = run(sampler, big, ub, 50, 0.9, 0.7)
    assert torch.equal(got[:64], exact.sample(big[:64], 0.7, 50, 0.9, ub[:64]))
    assert torch.equal(got[-64:], exact.sample(big[-64:], 0.7, 50, 0.9, ub[-64:]))
    assert torch.equal(got, torch.cat([run(sampler, big[s:s + 200], ub[s:s + 200], 50, 0.9, 0.7) for s in range(0, 600, 200)]))
