"""Committed fixtures: the oracles must still reproduce them (CPU), and the HIP kernels must match them (GPU)."""
from pathlib import Path

import pytest
import torch

from oracle import exact, logprob_ref, sampling_ref

GOLDEN = Path(__file__).resolve().parent / "golden"
NAN_ROW = 4  # the -inf-only row: the reference's softmax is NaN there, the build draws uniformly


def load(name):
    return torch.load(GOLDEN / name, weights_only=True)


def sampling_cases(blob):
    for n, (t, k, p) in enumerate(blob["cases"].tolist()):
        yield n, float(t), (int(k) or None), (None if p == 1.0 else float(p))


def test_logprob_oracle_reproduces_fixture():
    b = load("logprob_cfg1_rows4.pt")
    assert torch.equal(logprob_ref.logprob_ref(b["logits"], b["ids"]), b["logp_f32"])
    assert torch.allclose(logprob_ref.logprob_f64(b["logits"], b["ids"]), b["logp_f64"], atol=1e-13, rtol=0)
    assert (b["logp_f32"].double() - b["logp_f64"]).abs().max().item() < 2e-5


def test_sampling_oracles_reproduce_fixture():
    b = load("sampling_rows16.pt")
    for n, t, k, p in sampling_cases(b):
        assert torch.equal(exact.sample(b["logits"], t, k, p, b["uniforms"]), b[f"ids_exact_{n}"])
        ids, _ = sampling_ref.sample(b["logits"], k, p, t, b["uniforms"])
        keep = torch.arange(16) != NAN_ROW
        assert torch.equal(ids[keep], b[f"ids_torch_{n}"][keep])
        assert torch.equal(b[f"ids_exact_{n}"][keep], b[f"ids_torch_{n}"][keep])   # the two oracles agree


@pytest.mark.gpu
def test_logprob_kernel_matches_fixture(sampler):
    b = load("logprob_cfg1_rows4.pt")
    got = sampler.compute_logp(b["logits"].cuda(), b["ids"].cuda()).cpu()
    assert (got - b["logp_f32"]).abs().max().item() <= 1e-4
    assert (got.double() - b["logp_f64"]).abs().max().item() <= 2e-5


@pytest.mark.gpu
def test_sampling_kernel_matches_fixture(sampler):
    b = load("sampling_rows16.pt")
    for n, t, k, p in sampling_cases(b):
        got = sampler.sample(b["logits"].cuda(), top_k=k, top_p=p, temperature=t, uniforms=b["uniforms"].cuda()).cpu()
        assert torch.equal(got, b[f"ids_exact_{n}"]), n
        keep = torch.arange(16) != NAN_ROW
        assert torch.equal(got[keep], b[f"ids_torch_{n}"][keep]), n


def test_extras_oracles_reproduce_fixture():
    b = load("lmhead_extras.pt")
    got = logprob_ref.lmhead_logprob_ref(b["hidden"], b["weight"], b["ids"], dtype=torch.float64)
    assert torch.allclose(got, b["logp_f64"], atol=1e-13, rtol=0)
    full = torch.nn.functional.linear(b["hidden"].double(), b["weight"].double())
    assert torch.allclose(logprob_ref.entropy_f64(full), b["entropy_f64"], atol=1e-13, rtol=0)
    d = logprob_ref.logprob_backward_closed_form(b["bwd_logits"], b["bwd_ids"], b["bwd_grad"])
    assert torch.allclose(d, b["bwd_dlogits_f64"], atol=1e-14, rtol=0) and torch.isfinite(d).all()
    s = load("sampling_rows16.pt")
    n, t, k, p = next(sampling_cases(s))
    _, lp = exact.sample_rows(s["logits"], t, k, p, s["uniforms"])
    assert torch.equal(lp, b["drawn_logprob_case0"])


@pytest.mark.gpu
def test_extras_kernels_match_fixture(sampler):
    b = load("lmhead_extras.pt")
    lp, ent = sampler.fused_linear_logp(b["hidden"].cuda(), b["weight"].cuda(), b["ids"].cuda(), return_entropy=True)
    assert (lp.cpu().double() - b["logp_f64"]).abs().max().item() <= 1e-4
    assert (ent.cpu().double() - b["entropy_f64"]).abs().max().item() <= 1e-4
    logits, ids, grad = b["bwd_logits"].cuda(), b["bwd_ids"].cuda(), b["bwd_grad"].cuda()
    logp = sampler.compute_logp(logits, ids)
    d = sampler.compute_logp_backward(logits, ids, logp, grad).cpu().double()
    want = b["bwd_dlogits_f64"]
    assert ((d - want).abs() <= 2.0 ** -8 * want.abs() + 1e-6).all()
    s = load("sampling_rows16.pt")
    n, t, k, p = next(sampling_cases(s))
    ids2, lp2 = sampler.sample(s["logits"].cuda(), top_k=k, top_p=p, temperature=t, uniforms=s["uniforms"].cuda(),
                               return_logprob=True)
    assert torch.equal(ids2.cpu(), s[f"ids_exact_{n}"])
    assert (lp2.cpu().double() - b["drawn_logprob_case0"]).abs().max().item() <= 1e-5
