"""Pins the sampling oracles (CPU only).

oracle/ka_oracle.c (exact fixed-point definition) is checked against
  * the mathematical exp for its mass function W,
  * torch's own division for the temperature step,
  * a pure-Python evaluation of the definition with sorted() and exact rationals on small rows,
  * closed forms,
and against oracle/sampling_ref.py (torch restatement of the reference's native_sampling), with
which it must agree on every row whose decision margin exceeds fp32 rounding noise.
"""
import math
from fractions import Fraction

import pytest
import torch

from oracle import exact, sampling_ref

DTYPES = [torch.bfloat16, torch.float16, torch.float32]


def f32(x: float) -> float:
    return float(torch.tensor(x, dtype=torch.float32))


# ---------------------------------------------------------------- mass function and scalars
def test_weight_is_floor_of_scaled_exp():
    assert exact.weight(0.0) == 1 << 40
    g = torch.Generator().manual_seed(0)
    ds = (-torch.rand(4000, generator=g) * 30).tolist() + [-1e-8, -1e-3, -27.7, -28.5, -40.0, -1e30, -math.inf]
    for d in ds:
        d = f32(d)
        true = math.ldexp(math.exp(d), 40) if d > -700 else 0.0
        assert abs(exact.weight(d) - math.floor(true)) <= 1 + 4e-15 * true, d
    ws = [exact.weight(f32(-i / 64)) for i in range(2000)]
    assert all(a >= b for a, b in zip(ws, ws[1:]))          # monotone


def test_weight_does_not_depend_on_how_fma_is_provided():
    g = torch.Generator().manual_seed(3)
    for d in (-torch.rand(3000, generator=g) * 30).tolist() + [0.0, -1e-30, -28.4, -28.5]:
        assert exact.weight(f32(d)) == exact.weight_libm(f32(d))


def test_floor_scale_is_exact():
    g = torch.Generator().manual_seed(1)
    for s in torch.rand(300, generator=g).tolist() + [0.0, 2.0 ** -149, 2.0 ** -126, 1 - 2.0 ** -24, 0.9, 0.5]:
        s = f32(s)
        for z in (1, 7, (1 << 40) + 12345, (1 << 57) - 1, (1 << 61) + 99):
            assert exact.floor_scale(s, z) == math.floor(Fraction(s) * z)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("temp", [0.7, 1.3, 0.01, 1.0])
def test_temperature_step_is_torch_division_in_dtype(dtype, temp):
    if dtype == torch.float32:
        x = torch.randn(50000, generator=torch.Generator().manual_seed(2)) * 5
    else:
        bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
        x = bits.view(dtype)
        x = x[torch.isfinite(x.float())]
    want = (x / temp).float() if temp != 1.0 else x.float()
    got = exact.scale(x, temp)
    assert torch.equal(got, want)                            # value equality (-0 == +0)
    assert not torch.signbit(got[got == 0]).any()            # and -0 folded into +0


# ---------------------------------------------------------------- pure-Python evaluation
def brute_force_row(y, k, p, u):
    """The definition, with sorted() and exact rationals.  y: fp32 values after the temperature step."""
    vocab = len(y)
    order = sorted(range(vocab), key=lambda i: (-y[i], i))
    if k and k < vocab:
        kth = y[order[k - 1]]
        order = [i for i in order if y[i] >= kth]
    m = y[order[0]]
    w = {i: exact.weight(0.0 if y[i] == m else f32(y[i] - m)) for i in order}
    if p is not None and p < 1.0:
        z = sum(w.values())
        kept, before = [], 0
        for i in order:
            if Fraction(before) > Fraction(f32(p)) * z:
                break
            kept.append(i)
            before += w[i]
    else:
        kept = list(order)
    zb = sum(w[i] for i in kept)
    cum = 0
    for i in sorted(kept):
        cum += w[i]
        if Fraction(cum) > Fraction(f32(u)) * zb:
            return i, len(order), len(kept), w[i], zb
    raise AssertionError("no index selected")


def coarse_rows(batch, vocab, seed, dtype, step=0.25, spread=3.0):
    """Rows on a coarse grid, so ties at the k-th value and at the top-p cut are common."""
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(batch, vocab, generator=g) * spread / step).round() * step
    return x.to(dtype), torch.rand(batch, generator=g)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k,p,temp", [(5, 0.9, 0.7), (5, None, 1.0), (None, 0.8, 1.0), (None, None, 1.3),
                                      (1, 0.5, 1.0), (200, 0.95, 0.5), (3, 1.0, 2.0), (17, 0.05, 1.0)])
def test_exact_oracle_matches_pure_python_definition(dtype, k, p, temp):
    logits, u = coarse_rows(24, 61, seed=int(1000 * temp) + 7 * (k or 0) + int(100 * (p or 0)), dtype=dtype)
    logits[0, :] = 1.5                      # all-equal row
    logits[1, :] = -math.inf                # nothing but -inf: every entry ties at the maximum
    logits[2, 7] = math.inf                 # +inf wins outright
    logits[3, :40] = -math.inf              # masked prefix
    got, info = exact.sample(logits, temp, k, p, u, return_info=True)
    y = exact.scale(logits, temp)
    for r in range(logits.shape[0]):
        want, na, nb, w_pick, zb = brute_force_row(y[r].tolist(), k, p, float(u[r]))
        assert got[r].item() == want, (r, info[r])
        assert (info[r]["n_topk"], info[r]["n_kept"]) == (na, nb)
        assert (info[r]["w_pick"], info[r]["z_kept"]) == (w_pick, zb)


def test_drawn_token_logprob_matches_pure_python_definition():
    """sample_rows' log-probability (log of w_pick / z_kept) against the brute-force masses, with per-row
    parameters, a cut that falls inside a tie group, and closed forms."""
    logits, u = coarse_rows(12, 61, seed=99, dtype=torch.bfloat16)
    # row 0: five entries tie at the maximum and top_p cuts inside the group: mass before the third is
    # 2/5 > 0.35, so exactly two survive and either has probability 1/2
    logits[0, :] = -3.0
    logits[0, [4, 9, 20, 33, 50]] = 2.0
    temps = [1.0, 0.7, 1.3, 1.0, 0.5, 2.0, 1.0, 0.7, 1.0, 1.0, 0.9, 1.0]
    ks = [0, 5, 5, 0, 17, 3, 1, 200, 0, 61, 7, 2]
    ps = [0.35, 0.9, 1.0, 0.8, 0.05, 1.0, 0.5, 0.95, 1.0, 0.6, 0.3, 0.99]
    ids, lps = exact.sample_rows(logits, temps, ks, ps, u)
    for r in range(12):
        y = exact.scale(logits[r:r + 1], temps[r])[0].tolist()
        want, _, nb, w_pick, zb = brute_force_row(y, ks[r], ps[r], float(u[r]))
        assert ids[r].item() == want
        true = math.log(Fraction(w_pick, zb))
        assert abs(lps[r].item() - true) < 1e-12, (r, lps[r].item(), true)
        assert lps[r].item() <= 0.0
        if nb == 1:
            assert lps[r].item() == 0.0
    _, info = exact.sample(logits[:1], 1.0, 0, 0.35, u[:1], return_info=True)
    assert info[0]["n_kept"] == 2 and ids[0].item() in (4, 9)
    assert abs(lps[0].item() + math.log(2)) < 1e-12
    # closed forms: uniform survivors -> -log(count); top_k = 1 -> 0
    flat = torch.zeros(3, 10, dtype=torch.float32)
    _, lp = exact.sample_rows(flat, None, [0, 0, 1], [1.0, 0.3, 1.0], torch.tensor([0.1, 0.6, 0.9]))
    assert abs(lp[0].item() + math.log(10)) < 1e-12 and abs(lp[1].item() + math.log(4)) < 1e-12
    assert abs(lp[2].item() + math.log(10)) < 1e-12          # ten-way tie at the maximum: top_k = 1 keeps all
    # the probabilities of all survivors sum to one (stratified uniforms visit every survivor)
    row = (torch.randn(1, 40, generator=torch.Generator().manual_seed(8)) * 2).float()
    n = 2000
    got_ids, got_lp = exact.sample_rows(row.expand(n, 40).contiguous(), 0.8, 9, 0.9, (torch.arange(n) + 0.5) / n)
    per_id = {int(i): float(l) for i, l in zip(got_ids, got_lp)}
    assert abs(sum(math.exp(v) for v in per_id.values()) - 1.0) < 1e-9


# ---------------------------------------------------------------- closed forms
def test_top_k_one_is_argmax_for_every_u():
    g = torch.Generator().manual_seed(3)
    logits = (torch.randn(32, 5000, generator=g) * 3).bfloat16()
    first_argmax = torch.tensor([int((row == row.max()).nonzero()[0]) for row in logits.float()])
    ties = torch.tensor([(row == row.max()).sum() for row in logits.float()])
    for u in (0.0, 0.3, 0.999999):
        ids = exact.sample(logits, 0.7, 1, None, torch.full((32,), u))
        assert torch.equal(logits.float().gather(1, ids[:, None]).squeeze(1), logits.float().max(dim=1).values)
        if u == 0.0:
            assert torch.equal(ids, first_argmax)
    assert ties.max() >= 1


def test_extreme_uniforms_pick_first_and_last_survivor():
    logits, _ = coarse_rows(16, 300, seed=4, dtype=torch.float32)
    masked, _ = sampling_ref.filter_logits(logits, 20, 0.9, 1.0)
    alive = torch.isfinite(masked)
    first = torch.tensor([int(a.nonzero()[0]) for a in alive])
    last = torch.tensor([int(a.nonzero()[-1]) for a in alive])
    assert torch.equal(exact.sample(logits, 1.0, 20, 0.9, torch.zeros(16)), first)
    assert torch.equal(exact.sample(logits, 1.0, 20, 0.9, torch.full((16,), 1 - 2.0 ** -24)), last)
    assert torch.equal(exact.sample(logits, 1.0, 20, 0.9, torch.full((16,), 1.5)), last)      # clamped


def test_tiny_top_p_keeps_only_the_first_maximum():
    logits, u = coarse_rows(16, 300, seed=5, dtype=torch.bfloat16)
    ids, info = exact.sample(logits, 1.0, None, 1e-6, u, return_info=True)
    assert all(i["n_kept"] == 1 for i in info)
    assert torch.equal(ids, torch.tensor([int((r == r.max()).nonzero()[0]) for r in logits.float()]))


def test_uniform_row_counts_and_draw():
    logits = torch.zeros(1, 10, dtype=torch.float32)
    for p, kept in ((0.3, 4), (0.25, 3), (0.95, 10), (1.0, 10), (0.05, 1)):
        for u in (0.0, 0.26, 0.51, 0.99):
            ids, info = exact.sample(logits, 1.0, 5, p, torch.tensor([u]), return_info=True)
            assert info[0]["n_topk"] == 10 and info[0]["n_kept"] == kept      # ties: top-k keeps all ten
            assert ids.item() == math.floor(f32(u) * kept)


def test_stratified_uniforms_reproduce_the_probabilities():
    g = torch.Generator().manual_seed(6)
    row = (torch.randn(1, 50, generator=g) * 2).float()
    n = 4000
    u = (torch.arange(n) + 0.5) / n
    ids = exact.sample(row.expand(n, 50).contiguous(), 1.0, 12, 0.9, u)
    masked, _ = sampling_ref.filter_logits(row, 12, 0.9, 1.0)
    probs = torch.softmax(masked.double(), -1)[0]
    counts = torch.bincount(ids, minlength=50).double()
    assert (counts - probs * n).abs().max().item() <= 1.0 + 1e-6
    assert (ids[1:] >= ids[:-1]).all()                       # monotone in u


# ---------------------------------------------------------------- torch restatement vs exact definition
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k,p,temp", [(50, 0.9, 0.7), (50, None, 1.0), (None, 0.9, 1.0), (None, None, 0.7)])
def test_torch_restatement_agrees_outside_rounding_noise(dtype, k, p, temp):
    g = torch.Generator().manual_seed(7)
    logits = (torch.randn(96, 8192, generator=g) * 3).to(dtype)
    u = torch.rand(96, generator=g)
    a = exact.sample(logits, temp, k, p, u)
    b, margin = sampling_ref.sample(logits, k, p, temp, u)
    differ = a != b
    assert (margin[differ] < 1e-6).all(), (differ.nonzero().flatten().tolist(), margin[differ].tolist())
    assert differ.sum().item() <= 1


def test_baseline_sampling_config_agrees_exactly():
    from benchmarks.workloads import cfg5_sampling

    logits, u = cfg5_sampling(64)
    a = exact.sample(logits, 0.7, 50, 0.9, u)
    b, margin = sampling_ref.sample(logits, 50, 0.9, 0.7, u)
    assert torch.equal(a, b) and margin.min().item() > 1e-6


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_nan_logits_count_as_minus_infinity(dtype):
    """The convention for inputs the reference cannot take: a row with NaNs samples exactly like the
    same row with -inf in their place, and a NaN entry is never drawn while a number is available."""
    g = torch.Generator().manual_seed(41)
    logits = (torch.randn(16, 700, generator=g) * 3).to(dtype)
    holes = torch.rand(16, 700, generator=g) < 0.2
    with_nan = logits.clone(); with_nan[holes] = float("nan")
    with_inf = logits.clone(); with_inf[holes] = float("-inf")
    u = torch.rand(16, generator=g)
    for k, p, temp in [(50, 0.9, 0.7), (None, None, 1.0), (600, 0.99, 1.5), (None, 0.5, 1.0)]:
        a = exact.sample(with_nan, temp, k, p, u)
        b = exact.sample(with_inf, temp, k, p, u)
        assert torch.equal(a, b)
        assert not holes[torch.arange(16), a].any()
