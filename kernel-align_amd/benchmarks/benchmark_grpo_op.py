"""Logprob operator benchmark: torch's log_softmax + gather against SamplerBackend.compute_logp.

Counterpart of the reference's benchmarks/benchmark_grpo_op.py (same flags: --g-sizes, --seq-len,
--vocab-size; same two columns of peak device memory and latency), with three differences: every
timing is bracketed by a device synchronisation and averaged over --iters calls, the native result is
freed before the engine path is measured, and the engine rows carry HBM GB/s and the fraction of the
8 TB/s peak computed from the algorithmic bytes (2*V + 12 per token).
"""
from __future__ import annotations

import argparse
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parents[1]
if str(PKG) not in sys.path:
    sys.path.insert(0, str(PKG))

HBM_PEAK = 8.0e12


def run_benchmark(args) -> list:
    import torch
    from tabulate import tabulate

    from rl_engine.kernels.sampling import SamplerBackend
    from rl_engine.platforms.device import device_ctx
    from rl_engine.utils.logger import logger

    device = device_ctx.device
    dtype = device_ctx.get_preferred_dtype()
    sampler = SamplerBackend().to(device)
    logger.info(f"Starting benchmark on {device} with dtype {dtype}: SeqLen={args.seq_len}, Vocab={args.vocab_size}")

    def timed(fn):
        for _ in range(2):
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
        try:
            logits = torch.randn(g, args.seq_len, args.vocab_size, device=device, dtype=dtype)
            ids = torch.randint(0, args.vocab_size, (g, args.seq_len), device=device)
        except torch.cuda.OutOfMemoryError:
            rows.append([g, "OOM", "N/A", "N/A", "N/A", "N/A", "N/A", "N/A"])
            continue
        resident = torch.cuda.memory_allocated()

        def native():
            lp = torch.log_softmax(logits, dim=-1)
            return torch.gather(lp, dim=-1, index=ids.unsqueeze(-1))

        torch.cuda.reset_peak_memory_stats()
        try:
            native_ms = timed(native)
            native_extra = (torch.cuda.max_memory_allocated() - resident) / 2**30
        except torch.cuda.OutOfMemoryError:
            native_ms, native_extra = float("inf"), float("inf")
        torch.cuda.empty_cache()
        torch.cuda.reset_peak_memory_stats()
        engine_ms = timed(lambda: sampler.compute_logp(logits, ids))
        engine_extra = (torch.cuda.max_memory_allocated() - resident) / 2**30
        tokens = g * args.seq_len
        gbps = tokens * (2 * args.vocab_size + 12) / (engine_ms * 1e-3)
        rows.append([g, f"{resident / 2**30:.2f} GiB", f"+{native_extra:.2f} GiB", f"+{engine_extra:.4f} GiB",
                     f"{native_ms:.2f} ms", f"{engine_ms:.3f} ms", f"{native_ms / engine_ms:.1f}x",
                     f"{tokens / engine_ms / 1e3:.2f} M tok/s, {gbps / 1e9:.0f} GB/s ({gbps / HBM_PEAK:.0%} of peak)"])
        del logits, ids
        torch.cuda.empty_cache()
    headers = ["Group Size (G)", "Resident", "Native extra", "RL-Engine extra", "Native Latency",
               "RL-Engine Latency", "Speedup", "RL-Engine throughput"]
    print(f"\nRL-ENGINE GRPO OPERATOR BENCHMARK  |  {torch.cuda.get_device_name()}  |  {dtype}  |  "
          f"SeqLen={args.seq_len}, Vocab={args.vocab_size}")
    print(tabulate(rows, headers=headers, tablefmt="fancy_grid"))
    return rows


if __name__ == "__main__":
    ap = argparse.ArgumentParser(description="RL-Engine operator benchmark (MI355X)")
    ap.add_argument("--g-sizes", type=str, default="8,16,32,64,128,256")
    ap.add_argument("--seq-len", type=int, default=512)
    ap.add_argument("--vocab-size", type=int, default=128256)
    ap.add_argument("--iters", type=int, default=5)
    run_benchmark(ap.parse_args())
