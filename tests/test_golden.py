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
