"""Differentiable wrappers of the logprob operators for training loops.

The reference's operators run under ``torch.inference_mode()`` (rl_engine/kernels/sampling.py:38,91) and
cannot be part of a graph.  These two ``torch.autograd.Function`` s put the same kernels into one:

    logp = logp_from_logits(sampler, logits, token_ids)          # d/dlogits
    logp = linear_logp(sampler, hidden, weight, token_ids)       # d/dhidden, d/dweight; logits never stored

Forward and backward both run on the HIP kernels; nothing here computes on the CPU.
"""
from __future__ import annotations

import torch


class _LogpFromLogits(torch.autograd.Function):
    @staticmethod
    def forward(ctx, sampler, logits, token_ids):
        logp = sampler._compute_logp(logits, token_ids)
        ctx.sampler = sampler
        ctx.save_for_backward(logits, token_ids, logp)
        return logp

    @staticmethod
    def backward(ctx, grad_logp):
        logits, token_ids, logp = ctx.saved_tensors
        dlogits = ctx.sampler._compute_logp_backward(logits, token_ids, logp, grad_logp.contiguous())
        return None, dlogits, None


class _LinearLogp(torch.autograd.Function):
    @staticmethod
    def forward(ctx, sampler, hidden, weight, token_ids, chunk_tokens):
        logp = sampler._fused_linear_logp(hidden, weight, token_ids)
        ctx.sampler = sampler
        ctx.chunk_tokens = chunk_tokens
        ctx.save_for_backward(hidden, weight, token_ids)
        return logp

    @staticmethod
    def backward(ctx, grad_logp):
        hidden, weight, token_ids = ctx.saved_tensors
        dhidden, dweight = ctx.sampler._fused_linear_logp_backward(
            hidden, weight, token_ids, grad_logp.contiguous(), ctx.chunk_tokens)
        return None, dhidden, dweight.to(weight.dtype), None, None


def logp_from_logits(sampler, logits: torch.Tensor, token_ids: torch.Tensor) -> torch.Tensor:
    """``compute_logp`` as a node of the autograd graph: fp32 [..], gradient flows to ``logits``."""
    return _LogpFromLogits.apply(sampler, logits, token_ids)


def linear_logp(sampler, hidden: torch.Tensor, weight: torch.Tensor, token_ids: torch.Tensor,
                chunk_tokens: int | None = None) -> torch.Tensor:
    """``fused_linear_logp`` as a node of the autograd graph: gradients flow to ``hidden`` and ``weight``.

    The backward pass rebuilds the logits one chunk of ``chunk_tokens`` rows at a time, so the peak extra
    memory is one chunk of bf16 logits plus the fp32 weight-gradient accumulator.
    """
    return _LinearLogp.apply(sampler, hidden, weight, token_ids, chunk_tokens)
