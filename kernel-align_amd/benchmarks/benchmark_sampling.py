"""Sampling operator benchmark: a torch top-k -> top-p -> multinomial pipeline against SamplerBackend.sample.

Counterpart of the reference's benchmarks/benchmark_sampling.py (same flags: --g-sizes, --vocab-size,
--top-k, --top-p; fp32 logits by default as there, --dtype bf16 for the bf16 configuration).  The torch
comparator is the vectorised form of the reference's native_sampling (its per-row Python loop is
replaced by a scatter so that the comparison is kernel time, not interpreter time).  Timings are
averaged over --iters calls between device synchronisations.
"""
from __future__ import annotations

import argparse
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parents[1]
if str(PKG) not in sys.path:
    sys.path.insert(0, str(PKG))


def torch_sampling(logits, top_k=None, top_p=None, temperature=1.0):
    import torch

    if temperature != 1.0:
        logits = logits / temperature
    logits = logits.float()
    if top_k is not None:
        v, _ = torch.topk(logits, min(top_k, logits.size(-1)))
        logits = logits.masked_fill(logits < v[:, [-1]], float("-inf"))
    if top_p is not None:
        sorted_logits, sorted_idx = torch.sort(logits, descending=True)
        cum = torch.cumsum(torch.softmax(sorted_logits, dim=-1), dim=-1)
        remove = cum > top_p
        remove[..., 1:] = remove[..., :-1].clone()
        remove[..., 0] = False
        logits = logits.masked_fill(torch.zeros_like(remove).scatter(1, sorted_idx, remove), float("-inf"))
    return torch.multinomial(torch.softmax(logits, dim=-1), num_samples=1)


def run_benchmark(args) -> list:
    import torch
    from tabulate import tabulate

    from rl_engine.kernels.sampling import SamplerBackend
    from rl_engine.platforms.device import device_ctx

    device = device_ctx.device
    dtype = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}[args.dtype]
    sampler = SamplerBackend().to(device)

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.iters

    rows = []
    for g in [int(x) for x in args.g_sizes.split(",")]:
        logits = (torch.randn(g, args.vocab_size, device=device) * args.sigma).to(dtype)
        u = torch.rand(g, device=device)
        native_ms = timed(lambda: torch_sampling(logits, args.top_k, args.top_p, args.temperature))
        engine_ms = timed(lambda: sampler.sample(logits, top_k=args.top_k, top_p=args.top_p,
                                                 temperature=args.temperature, uniforms=u))
        rows.append([g, f"{native_ms:.3f} ms", f"{engine_ms:.3f} ms", f"{native_ms / engine_ms:.1f}x"])
    print(f"\nRL-ENGINE SAMPLING BENCHMARK  |  {torch.cuda.get_device_name()}  |  {dtype}  |  Vocab={args.vocab_size}, "
          f"TopK={args.top_k}, TopP={args.top_p}, T={args.temperature}")
    print(tabulate(rows, headers=["Batch Size (G)", "torch pipeline", "RL-Engine (HIP)", "Speedup"],
                   tablefmt="fancy_grid"))
    return rows


if __name__ == "__main__":
    ap = argparse.ArgumentParser(description="RL-Engine sampling benchmark (MI355X)")
    ap.add_argument("--g-sizes", type=str, default="32,64,128,256")
    ap.add_argument("--vocab-size", type=int, default=128256)
    ap.add_argument("--top-k", type=int, default=50)
    ap.add_argument("--top-p", type=float, default=0.9)
    ap.add_argument("--temperature", type=float, default=1.0)
    ap.add_argument("--dtype", choices=["fp32", "bf16", "fp16"], default="fp32")
    ap.add_argument("--sigma", type=float, default=1.0)
    ap.add_argument("--iters", type=int, default=20)
    run_benchmark(ap.parse_args())
