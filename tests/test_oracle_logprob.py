"""Pins oracle/logprob_ref.py: closed forms, brute force and fp32-vs-fp64 agreement (CPU only)."""
import math

import pytest
import torch

from oracle import logprob_ref as O


def test_uniform_row_is_minus_log_v():
    for v in (2, 17, 1000, 32000):
        x = torch.full((1, v), 3.25, dtype=torch.bfloat16)
        ids = torch.tensor([v // 2])
        assert abs(O.logprob_ref(x, ids).item() + math.log(v)) < 2e-6 * max(1, math.log(v))
        assert abs(O.logprob_f64(x, ids).item() + math.log(v)) < 1e-12


def test_single_spike_closed_form():
    v, c = 128256, 25.0
    x = torch.zeros(2, v, dtype=torch.bfloat16)
    x[:, 777] = c
    ids = torch.tensor([777, 5])
    lse_minus_c = math.log1p((v - 1) * math.exp(-c))
    want = [-lse_minus_c, -c - lse_minus_c]
    got32, got64 = O.logprob_ref(x, ids), O.logprob_f64(x, ids)
    for k in range(2):
        assert abs(got64[k].item() - want[k]) < 1e-12
        assert abs(got32[k].item() - want[k]) < 1e-5


def test_masked_entries_contribute_nothing():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4, 64, generator=g).bfloat16()
    ids = torch.randint(0, 32, (4,), generator=g)
    masked = torch.cat([x[:, :32], torch.full((4, 32), -math.inf, dtype=torch.bfloat16)], dim=1)
    assert torch.equal(O.logprob_ref(masked, ids), O.logprob_ref(x[:, :32].contiguous(), ids))
    assert torch.allclose(O.logprob_f64(masked, ids), O.logprob_f64(x[:, :32].contiguous(), ids), atol=1e-14)


def test_probabilities_sum_to_one():
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(1, 501, generator=g) * 3).bfloat16()
    all_targets = torch.arange(501)
    rows = x.expand(501, 501)
    assert abs(O.logprob_f64(rows, all_targets).exp().sum().item() - 1.0) < 1e-12
    assert abs(O.logprob_ref(rows, all_targets).double().exp().sum().item() - 1.0) < 1e-5


def test_shift_invariance_with_exact_shift():
    # adding 8.0 keeps every bf16 value in [-4, 4) with <= 4 mantissa bits exactly representable
    g = torch.Generator().manual_seed(5)
    x = (torch.randint(-32, 32, (3, 300), generator=g).float() / 8).bfloat16()
    ids = torch.randint(0, 300, (3,), generator=g)
    shifted = (x.float() + 8.0).bfloat16()
    assert torch.equal(shifted.float() - 8.0, x.float())
    assert torch.allclose(O.logprob_f64(x, ids), O.logprob_f64(shifted, ids), atol=1e-13)
    assert torch.allclose(O.logprob_ref(x, ids), O.logprob_ref(shifted, ids), atol=2e-6)


@pytest.mark.parametrize("vocab", [1, 2, 7, 64])
def test_bruteforce_small_vocab(vocab):
    g = torch.Generator().manual_seed(vocab)
    x = (torch.randn(5, vocab, generator=g) * 4).bfloat16()
    ids = torch.randint(0, vocab, (5,), generator=g)
    got64, got32 = O.logprob_f64(x, ids), O.logprob_ref(x, ids)
    for r in range(5):
        want = O.logprob_bruteforce(x[r].float().tolist(), int(ids[r]))
        assert abs(got64[r].item() - want) < 1e-12
        assert abs(got32[r].item() - want) < 2e-6


def test_fp32_route_within_tolerance_of_fp64_on_cfg1():
    from benchmarks.workloads import cfg1_logits

    logits, ids = cfg1_logits()
    a, b = O.logprob_ref(logits, ids), O.logprob_f64(logits, ids)
    assert a.shape == (4, 128) and a.dtype == torch.float32
    assert (a.double() - b).abs().max().item() < 2e-5


def test_reference_dtype_route_is_the_rounded_one():
    # what the reference returns on ROCm (bf16) is far from the fp32 value: it cannot be the oracle
    from benchmarks.workloads import cfg1_logits

    logits, ids = cfg1_logits()
    ref_bf16 = O.logprob_reference_dtype(logits[:1], ids[:1])
    assert ref_bf16.dtype == torch.bfloat16
    err = (ref_bf16.double() - O.logprob_f64(logits[:1], ids[:1])).abs().max().item()
    assert 1e-3 < err < 0.25


def test_entropy_closed_forms():
    v = 4096
    assert abs(O.entropy_f64(torch.zeros(1, v, dtype=torch.bfloat16)).item() - math.log(v)) < 1e-12
    x = torch.full((1, v), -math.inf, dtype=torch.bfloat16)
    x[0, 3] = 1.0
    assert O.entropy_f64(x).item() == 0.0


def test_entropy_against_a_pure_python_evaluation():
    """Rows that are neither uniform nor one-hot, evaluated term by term with math.fsum: a weighting that only the two
    closed forms above cannot tell from the right one (p * x without the log-sum-exp, a missing sign, log2 for log)
    fails here."""
    rows = [[0.5, -1.25, 3.0, 0.0, 2.0, -0.75, 1.5],
            [-3.0, -3.0, 4.0, 4.0, -math.inf, 0.25, 10.0, -8.0],
            [20.0, 19.5, -20.0]]
    for row in rows:
        m = max(row)
        z = math.fsum(math.exp(x - m) for x in row)
        probs = [math.exp(x - m) / z for x in row]
        want = -math.fsum(p * math.log(p) for p in probs if p > 0.0)
        got = O.entropy_f64(torch.tensor([row], dtype=torch.float32)).item()
        assert abs(got - want) < 1e-12, (row, got, want)
        assert 0.0 < want < math.log(len(row))
    # two equal entries and nothing else: exactly ln 2, whatever their common value
    assert abs(O.entropy_f64(torch.tensor([[-math.inf, 7.0, 7.0, -math.inf]])).item() - math.log(2.0)) < 1e-15


def test_backward_closed_form_is_autograd():
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(16, 999, generator=g) * 3
    ids = torch.randint(0, 999, (16,), generator=g)
    grad = torch.randn(16, generator=g)
    a = O.logprob_backward_ref(logits, ids, grad, dtype=torch.float64)
    b = O.logprob_backward_closed_form(logits, ids, grad)
    assert (a - b).abs().max().item() < 1e-14
    assert (a.sum(-1)).abs().max().item() < 1e-13          # rows of the gradient sum to zero
    # finite differences of the fp64 forward pin the sign and the one-hot term
    x = logits[:2, :50].double()
    i2, g2 = ids[:2] % 50, grad[:2].double()
    base = (O.logprob_f64(x, i2) * g2).sum()
    eps = 1e-6
    an = O.logprob_backward_closed_form(x, i2, g2)
    for (r, c) in ((0, int(i2[0])), (0, 3), (1, 17)):
        xp = x.clone()
        xp[r, c] += eps
        fd = ((O.logprob_f64(xp, i2) * g2).sum() - base) / eps
        assert abs(fd.item() - an[r, c].item()) < 1e-5


def test_lmhead_backward_oracle_forms_agree_and_match_finite_differences():
    """Autograd and the written-out D W / D^T h agree; a central difference of the fp64 forward pins both
    against a transposed operand or a dropped one-hot term."""
    g = torch.Generator().manual_seed(11)
    hidden = torch.randn(6, 16, generator=g).bfloat16()
    weight = (torch.randn(23, 16, generator=g) * 0.3).bfloat16()
    ids = torch.randint(0, 23, (6,), generator=g)
    grad = torch.randn(6, generator=g)
    dh_a, dw_a = O.lmhead_logprob_backward_ref(hidden, weight, ids, grad)
    dh_c, dw_c = O.lmhead_logprob_backward_closed_form(hidden, weight, ids, grad)
    assert torch.allclose(dh_a, dh_c, atol=1e-12) and torch.allclose(dw_a, dw_c, atol=1e-12)

    def loss(h, w):
        lp = torch.log_softmax(h @ w.t(), -1).gather(-1, ids.unsqueeze(-1)).squeeze(-1)
        return (lp * grad.double()).sum()

    h0, w0 = hidden.double(), weight.double()
    eps = 1e-6
    for (r, c) in [(0, 0), (3, 7), (5, 15)]:
        e = torch.zeros_like(h0); e[r, c] = eps
        fd = (loss(h0 + e, w0) - loss(h0 - e, w0)) / (2 * eps)
        assert abs(fd.item() - dh_c[r, c].item()) < 1e-7
    for (r, c) in [(0, 0), (int(ids[2]), 3), (22, 15)]:
        e = torch.zeros_like(w0); e[r, c] = eps
        fd = (loss(h0, w0 + e) - loss(h0, w0 - e)) / (2 * eps)
        assert abs(fd.item() - dw_c[r, c].item()) < 1e-7


def test_lmhead_oracle_is_the_logprob_oracle_on_the_linear_layer():
    """lmhead_logprob_ref is pinned two ways: against logprob_f64 on an fp64 F.linear, and against a
    pure-Python evaluation (explicit dot products + math.fsum) that shares no code with it, so that a
    transposed weight, a wrong gather index or a dropped maximum would fail."""
    g = torch.Generator().manual_seed(21)
    hidden = torch.randn(37, 64, generator=g).bfloat16()
    weight = (torch.randn(301, 64, generator=g) * 0.2).bfloat16()
    ids = torch.randint(0, 301, (37,), generator=g)
    logits64 = torch.nn.functional.linear(hidden.double(), weight.double())
    want64 = O.logprob_f64(logits64, ids)
    got64 = O.lmhead_logprob_ref(hidden, weight, ids, dtype=torch.float64, chunk_rows=16)   # ragged last chunk
    assert got64.shape == (37,) and got64.dtype == torch.float64
    assert (got64 - want64).abs().max().item() < 1e-12
    got32 = O.lmhead_logprob_ref(hidden, weight, ids)
    assert got32.dtype == torch.float32 and (got32.double() - want64).abs().max().item() < 2e-5
    # leading dimensions are kept
    assert torch.equal(O.lmhead_logprob_ref(hidden[:36].view(4, 9, 64), weight, ids[:36].view(4, 9), torch.float64),
                       got64[:36].view(4, 9))

    # non-square [3,8] x [5,8] case, rows and targets all different, evaluated in plain Python
    h = (torch.randn(3, 8, generator=g) * 2).bfloat16()
    w = torch.randn(5, 8, generator=g).bfloat16()
    t = torch.tensor([4, 0, 2])
    got = O.lmhead_logprob_ref(h, w, t, dtype=torch.float64)
    hl, wl = h.double().tolist(), w.double().tolist()
    for r in range(3):
        row = [math.fsum(hl[r][k] * wl[v][k] for k in range(8)) for v in range(5)]
        assert abs(got[r].item() - O.logprob_bruteforce(row, int(t[r]))) < 1e-12
    # closed form: zero hidden row -> uniform distribution over the vocabulary
    z = O.lmhead_logprob_ref(torch.zeros(1, 8, dtype=torch.bfloat16), w, torch.tensor([3]), torch.float64)
    assert abs(z.item() + math.log(5)) < 1e-14
