"""Pins oracle/grpo_ref.py without a GPU: closed forms of the clipped surrogate and the k3 KL estimate, and a
central difference of the loss against the autograd derivative."""
import math

import torch

from oracle import grpo_ref


def test_closed_forms():
    new = torch.tensor([-1.0, -1.0, -1.0, -1.0])
    old = torch.tensor([-1.0, -2.0, -2.0, -0.5])          # ratio 1, e, e, e^-0.5
    adv = torch.tensor([2.0, 1.0, -1.0, 1.0])
    loss, kl, d = grpo_ref.grpo_token_terms(new, adv, old, None, 0.2, 0.2, 0.0)
    e, r = math.e, math.exp(-0.5)
    assert torch.allclose(loss, torch.tensor([-2.0, -1.2, e, -r], dtype=torch.float64))   # clipped only for A > 0, ratio > 1.2
    assert torch.allclose(d, torch.tensor([-2.0, 0.0, e, -r], dtype=torch.float64))
    assert not kl.any()
    ref = torch.tensor([-1.0, -0.5, -3.0, -1.0])
    _, kl, d2 = grpo_ref.grpo_token_terms(new, adv, old, ref, 0.2, 0.2, 0.5)
    want = torch.tensor([0.0, math.exp(0.5) - 0.5 - 1, math.exp(-2.0) + 2 - 1, 0.0], dtype=torch.float64)
    assert torch.allclose(kl, want)
    assert torch.allclose(d2 - d, 0.5 * (1 - torch.exp(ref.double() - new.double())))


def test_derivative_matches_central_difference():
    g = torch.Generator().manual_seed(0)
    new = -torch.rand(50, generator=g).double() * 4
    old = new + torch.randn(50, generator=g).double() * 0.4
    ref = new + torch.randn(50, generator=g).double() * 0.4
    adv = torch.randn(50, generator=g).double()
    _, _, d = grpo_ref.grpo_token_terms(new, adv, old, ref, 0.2, 0.3, 0.07)
    eps = 1e-6
    lp, _, _ = grpo_ref.grpo_token_terms(new + eps, adv, old, ref, 0.2, 0.3, 0.07)
    lm, _, _ = grpo_ref.grpo_token_terms(new - eps, adv, old, ref, 0.2, 0.3, 0.07)
    fd = (lp - lm) / (2 * eps)
    ratio = torch.exp(new - old)
    away_from_kinks = ((ratio - 0.8).abs() > 1e-3) & ((ratio - 1.3).abs() > 1e-3)
    assert torch.allclose(fd[away_from_kinks], d[away_from_kinks], atol=1e-6)
