"""CPU statement of the GRPO per-token objective (test infrastructure only).

The reference stops at the log-probabilities (rl_engine/kernels/sampling.py:92-112; README.md:49 names the
advantage step).  This is the standard objective a GRPO trainer applies to them, written with torch ops in
fp64 so that autograd provides the derivative the kernel is checked against.
"""
from __future__ import annotations

import torch


def grpo_token_terms(logp_new, advantages, logp_old=None, logp_ref=None, clip_low=0.2, clip_high=0.2, beta=0.0):
    """(loss, kl, dloss_dlogp) per token in fp64; the derivative comes from autograd."""
    new = logp_new.detach().cpu().double().clone().requires_grad_(True)
    adv = advantages.detach().cpu().double()
    old = new.detach() if logp_old is None else logp_old.detach().cpu().double()
    ratio = torch.exp(new - old)
    s1 = ratio * adv
    s2 = torch.clamp(ratio, 1.0 - clip_low, 1.0 + clip_high) * adv
    surr = torch.minimum(s1, s2)
    if logp_ref is not None:
        d = logp_ref.detach().cpu().double() - new
        kl = torch.exp(d) - d - 1.0
    else:
        kl = torch.zeros_like(new)
    loss = -(surr - beta * kl)
    loss.sum().backward()
    return loss.detach(), kl.detach(), new.grad
