"""Seeded input builders for the benchmark configurations (shared by the benchmarks, the tests and the smoke check)."""
from __future__ import annotations

import torch


def cfg1_logits(device="cpu"):
    """bf16 [4, 128, 32000] ~ N(0, 2^2), ids uniform, seed 0."""
    g = torch.Generator().manual_seed(0)
    logits = (torch.randn(4, 128, 32000, generator=g) * 2.0).bfloat16()
    ids = torch.randint(0, 32000, (4, 128), generator=g)
    return logits.to(device), ids.to(device)


def spike_logits(n_rows: int, vocab: int, seed: int, device, sigma: float = 3.0, spike_frac: float = 0.01,
                 spike: float = 25.0, rows_per_block: int = 2048):
    """bf16 [n_rows, vocab] ~ N(0, sigma^2) with one +spike logit in a Bernoulli(spike_frac) subset of
    rows; ids uniform.  Generated block-wise on `device` from a seeded generator, so any prefix of
    blocks can be regenerated without the rest."""
    dev = torch.device(device)
    logits = torch.empty(n_rows, vocab, dtype=torch.bfloat16, device=dev)
    ids = torch.empty(n_rows, dtype=torch.int64, device=dev)
    for b, s in enumerate(range(0, n_rows, rows_per_block)):
        n = min(rows_per_block, n_rows - s)
        blk, bid = spike_block(n, vocab, seed, b, dev, sigma, spike_frac, spike)
        logits[s:s + n] = blk
        ids[s:s + n] = bid
    return logits, ids


def spike_block(n: int, vocab: int, seed: int, block: int, device, sigma: float = 3.0,
                spike_frac: float = 0.01, spike: float = 25.0):
    """Block `block` of spike_logits: deterministic in (seed, block, device type)."""
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(seed * 1_000_003 + block)
    x = torch.randn(n, vocab, generator=g, device=dev, dtype=torch.float32).mul_(sigma)
    has_spike = torch.rand(n, generator=g, device=dev) < spike_frac
    col = torch.randint(0, vocab, (n,), generator=g, device=dev)
    rows = torch.nonzero(has_spike).squeeze(-1)
    x[rows, col[rows]] = spike
    ids = torch.randint(0, vocab, (n,), generator=g, device=dev)
    # every fourth spike row targets its spike, so both branches of the closed form are exercised
    hit = rows[::4]
    ids[hit] = col[hit]
    return x.bfloat16(), ids


def cfg5_sampling(batch: int, device="cpu", vocab: int = 128256):
    """bf16 [B, V] ~ N(0, 3^2) and one fp32 uniform per row; seed 1234, logits drawn before uniforms."""
    g = torch.Generator().manual_seed(1234)
    logits = (torch.randn(batch, vocab, generator=g) * 3.0).bfloat16()
    u = torch.rand(batch, generator=g)
    return logits.to(device), u.to(device)
