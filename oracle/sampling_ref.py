"""Torch CPU restatement of the reference's sampling filter, with an inverse-CDF draw.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

`filter_logits` follows benchmarks/benchmark_sampling.py:12-36 (`native_sampling`) line by line:
temperature in the input dtype (:16-17), `.float()` (:19), top-k mask with ties kept (:21-23; the
same rule as rl_engine/kernels/sampling.py:83-86), descending sort, softmax, cumulative sum,
`> top_p`, shift right by one, first entry kept (:25-30), scatter of -inf (:32-34), softmax (:36).
Two places differ from the reference text, both because the reference leaves the result to torch
internals that no other implementation can reproduce:
  * the sort is `stable=True`, so equal values rank by ascending vocabulary index;
  * the draw (:37, `torch.multinomial`) is replaced by an inverse CDF over the final
    probabilities in ascending index order, driven by one caller-supplied uniform per row: the
    first index whose inclusive cumulative probability exceeds u * total.

`sample` also returns, per row, how close the two threshold decisions were (`margin`): rows whose
margin is below a few fp32 ulps are the only ones on which an implementation with different
rounding (the fixed-point oracle in ka_oracle.c, the HIP kernel) may legitimately differ.

Pinned by tests/test_oracle_sampling.py (closed forms and a pure-Python evaluation on small rows).
"""
from __future__ import annotations

import torch


def filter_logits(logits: torch.Tensor, top_k=None, top_p=None, temperature: float = 1.0):
    """Masked fp32 logits [B, V] (dropped entries = -inf) and the top-p decision margin per row."""
    logits = logits.detach().cpu()
    if temperature != 1.0:
        logits = logits / temperature                      # in the input dtype (benchmark_sampling.py:16-17)
    logits = logits.float().clone()                        # :19
    batch, vocab = logits.shape
    margin = torch.full((batch,), float("inf"), dtype=torch.float64)
    if top_k is not None:
        v, _ = torch.topk(logits, min(int(top_k), vocab))  # :22
        logits[logits < v[:, [-1]]] = float("-inf")        # :23 (ties with the k-th value survive)
    if top_p is not None:
        sorted_logits, sorted_indices = torch.sort(logits, descending=True, stable=True)   # :26 (+stable)
        cumulative_probs = torch.cumsum(torch.softmax(sorted_logits, dim=-1), dim=-1)      # :27
        remove = cumulative_probs > top_p                                                  # :28
        remove[..., 1:] = remove[..., :-1].clone()                                         # :29
        remove[..., 0] = False                                                             # :30
        # distance of the nearest *decisive* prefix sum to top_p: prefixes over entries that still carry
        # mass (the -inf tail repeats the last sum and decides nothing)
        alive = torch.isfinite(sorted_logits)
        alive_shift = torch.zeros_like(alive)
        alive_shift[..., :-1] = alive[..., 1:]
        gap = (cumulative_probs.double() - float(torch.tensor(top_p, dtype=torch.float32))).abs()
        gap[~alive_shift] = float("inf")
        margin = gap.min(dim=-1).values
        for i in range(batch):                                                             # :32-34
            logits[i, sorted_indices[i][remove[i]]] = float("-inf")
    return logits, margin


def sample(logits: torch.Tensor, top_k=None, top_p=None, temperature: float = 1.0, uniforms=None):
    """(ids int64 [B], margin float64 [B]): inverse-CDF draw from softmax(filter_logits(...))."""
    masked, margin_p = filter_logits(logits, top_k, top_p, temperature)
    probs = torch.softmax(masked, dim=-1)                  # benchmark_sampling.py:36
    cdf = torch.cumsum(probs.double(), dim=-1)
    total = cdf[:, -1:]
    target = uniforms.detach().cpu().double().view(-1, 1) * total
    hit = cdf > target
    ids = torch.argmax(hit.to(torch.uint8), dim=-1)        # first True
    # draw margin: distance of u*total to the nearest cdf step that carries mass, relative to total
    gap = ((cdf - target).abs() / total)
    gap[probs == 0] = float("inf")
    margin_u = gap.min(dim=-1).values
    return ids.to(torch.int64), torch.minimum(margin_p, margin_u)
