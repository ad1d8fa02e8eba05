"""Fused lm_head -> logprob benchmark (no counterpart in the reference).

    python kernel-align_amd/benchmarks/benchmark_lmhead.py [--rows 32768] [--hidden 4096] [--vocab 128256]

hidden bf16 [rows, hidden] ~ N(0, 1), W bf16 [vocab, hidden] ~ N(0, 0.02^2), ids uniform, seed 0.
Reports time per call, TFLOP/s (2 * rows * hidden * vocab flop) and the fraction of the 2.5 PFLOP/s
dense bf16 MFMA peak, beside torch's own bf16 matmul (hipBLASLt) that materialises the logits and the
unfused matmul -> compute_logp pipeline.
"""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parents[1]
if str(PKG) not in sys.path:
    sys.path.insert(0, str(PKG))

MFMA_PEAK_TFLOPS = 2500.0


def timed(fn, iters, warmup=2):
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--rows", type=int, default=32768)
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--vocab", type=int, default=128256)
    ap.add_argument("--iters", type=int, default=5)
    ap.add_argument("--skip-unfused", action="store_true", help="time only the fused kernel")
    ap.add_argument("--backward", action="store_true",
                    help="also time the chunked backward (dhidden, dweight): 3 GEMMs of the forward's size")
    args = ap.parse_args()

    import torch
    from rl_engine.kernels.sampling import SamplerBackend

    sampler = SamplerBackend().to("cuda")
    g = torch.Generator(device="cuda").manual_seed(0)
    hidden = torch.randn(args.rows, args.hidden, generator=g, device="cuda").bfloat16()
    weight = (torch.randn(args.vocab, args.hidden, generator=g, device="cuda") * 0.02).bfloat16()
    ids = torch.randint(0, args.vocab, (args.rows,), generator=g, device="cuda")
    flop = 2.0 * args.rows * args.hidden * args.vocab

    ms = timed(lambda: sampler.fused_linear_logp(hidden, weight, ids), args.iters)
    out = {"rows": args.rows, "hidden": args.hidden, "vocab": args.vocab, "fused_ms": ms,
           "fused_tflops": flop / ms / 1e9, "fused_frac_of_mfma_peak": flop / ms / 1e9 / MFMA_PEAK_TFLOPS}
    if not args.skip_unfused:
        chunk = min(args.rows, 8192)  # the materialised logits of 8192 rows are 2.1 GB

        def unfused():
            for s in range(0, args.rows, chunk):
                logits = hidden[s:s + chunk] @ weight.T
                sampler.compute_logp(logits, ids[s:s + chunk])

        def gemm_only():
            for s in range(0, args.rows, chunk):
                hidden[s:s + chunk] @ weight.T

        ms_u = timed(unfused, max(2, args.iters // 2))
        ms_g = timed(gemm_only, max(2, args.iters // 2))
        out.update({"unfused_ms": ms_u, "torch_matmul_ms": ms_g, "torch_matmul_tflops": flop / ms_g / 1e9,
                    "unfused_logits_bytes": chunk * args.vocab * 2})
    if args.backward:
        grad = torch.randn(args.rows, generator=g, device="cuda")
        torch.cuda.reset_peak_memory_stats()
        before = torch.cuda.memory_allocated()
        # the gradient matrix of a chunk from the library GEMM + the two logprob kernels (the default) ...
        ms_b = timed(lambda: sampler.fused_linear_logp_backward(hidden, weight, ids, grad), max(2, args.iters // 2), warmup=1)
        out.update({"backward_ms": ms_b, "backward_tflops": 3.0 * flop / ms_b / 1e9,
                    "backward_peak_extra_bytes": torch.cuda.max_memory_allocated() - before})
        # ... and from the forward's kernel with the softmax gradient as its epilogue (lse= option)
        _, lse = sampler.fused_linear_logp(hidden, weight, ids, return_lse=True)
        ms_f = timed(lambda: sampler.fused_linear_logp_backward(hidden, weight, ids, grad, lse=lse), max(2, args.iters // 2), warmup=1)
        out.update({"backward_with_dlogits_kernel_ms": ms_f})
        chunk_rows = min(args.rows, 8192)
        dl = torch.empty(chunk_rows, args.vocab, dtype=torch.bfloat16, device="cuda")
        stream = torch.cuda.current_stream().cuda_stream
        def front_fused():
            assert sampler._lib.ka_lmhead_dlogits_bf16(hidden.data_ptr(), weight.data_ptr(), ids.data_ptr(), lse.data_ptr(),
                                                       grad.data_ptr(), dl.data_ptr(), args.vocab, chunk_rows, args.hidden,
                                                       args.vocab, stream) == 0
        def front_gemm():
            logits = torch.matmul(hidden[:chunk_rows], weight.t())
            logp = sampler.compute_logp(logits, ids[:chunk_rows])
            sampler.compute_logp_backward(logits, ids[:chunk_rows], logp, grad[:chunk_rows], inplace=True)
        out.update({"front_half_rows": chunk_rows, "front_half_dlogits_kernel_ms": timed(front_fused, args.iters),
                    "front_half_gemm_and_logprob_kernels_ms": timed(front_gemm, args.iters)})
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
