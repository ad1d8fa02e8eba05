#!/usr/bin/env python3
"""Headline benchmark: per-token logprob over bf16 logits [G=256, L=512, V=128256] on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one compute_logp call over the whole resident [256, 512, 128256] tensor (33.6 GB),
i.e. 131,072 tokens.  Prints ONE JSON line; `value` is tokens/s with the logits already in HBM.
`roofline` prices the logprob kernel against the 8 TB/s HBM peak from the algorithmic bytes
(2*V + 8 + 4 per token); `cpu_baseline` times the CPU oracle on a bounded sample of the same
tensor on this box's host cores.  Sampling latency at batch 256 rides along in `sampling`.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

REPO = Path(__file__).resolve().parent
for _p in (REPO, REPO / "kernel-align_amd"):
    if str(_p) not in sys.path:
        sys.path.insert(0, str(_p))

HBM_PEAK_GBPS = 8000.0
G, L, V = 256, 512, 128256
BYTES_PER_TOKEN = 2 * V + 8 + 4
# HBM traffic per launch of each kernel, in bytes.  These are NOT measured by this program: they come from
# separate rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this same command (one counter per run), scaled by
# what the counters read for a plain 1 GiB copy in the same run (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000), and
# are repeated here with their source so that a reader can tell them from live figures.  A kernel whose code
# changed after its profile was taken reports null until the profile is redone.
# Each entry: bytes per launch, the profile that records the counter runs, the kernel's source files, and the first 16
# hex digits of the SHA-256 of those files (concatenated in that order) at the time of the counter runs.
CSRC = REPO / "kernel-align_amd" / "csrc"
_SAMPLING_SOURCES = ("ka_common.h", "ka_sampling_common.h", "ka_sampling_topk.h", "ka_sampling_dense.h", "ka_sampling_draw.h",
                     "ka_sampling_kernel.h", "ka_sampling.hip", "ka_sampling_half.hip")
_LMHEAD_SOURCES = ("ka_common.h", "ka_lmhead.hip", "ka_lmhead_narrow.h")
STATIC_TRAFFIC = {
    "logprob_rows": ((2 * 16425200 + 4317.5) * 1024, "profiles/logprob_rows_bf16_G256_L512_V128256.txt",         # 131072 rows
                     ("ka_common.h", "ka_logprob.hip"), "d3ed0936386075a5"),
    "logprob_backward_rows": ((2 * 4108350 + 8208390) * 1024, "profiles/logprob_backward_rows_bf16_G64_L512_V128256.txt",  # 32768 rows
                              ("ka_common.h", "ka_logprob.hip"), "d3ed0936386075a5"),
    "sample_rows": ((2 * 32831.5 + 10.3) * 1024, "profiles/sample_rows_bf16_B64-1024_V128256.txt",                     # B = 256
                    _SAMPLING_SOURCES, "817959ab3c8df18c"),
    "lmhead_partials": ((2 * 3.176e7 + 121088) * 1024, "profiles/lmhead_partials_bf16_H4096_V128256.txt",            # N = 32768; L2 misses: varies +-50 % between calls
                        _LMHEAD_SOURCES, "793ffdf2d7810fe0"),
    "lmhead_n64": ((2 * 517332 + 256) * 1024, "profiles/lmhead_partials_bf16_H4096_V128256.txt", _LMHEAD_SOURCES, "793ffdf2d7810fe0"),
    "lmhead_n256": ((2 * 532202 + 9216) * 1024, "profiles/lmhead_partials_bf16_H4096_V128256.txt", _LMHEAD_SOURCES, "793ffdf2d7810fe0"),
}
# FETCH_SIZE / WRITE_SIZE KiB per dispatch of sample_rows by batch, from the same counter runs as the B = 256 entry above
_SAMPLING_KIB = {64: (8268.3, 2.6), 128: (16314.7, 5.3), 256: (32831.5, 10.3), 512: (65957.6, 21.0), 1024: (131641.0, 42.9)}
PARITY_TOL = 1e-4


def source_fingerprint(files) -> str:
    import hashlib

    h = hashlib.sha256()
    for name in files:
        h.update((CSRC / name).read_bytes())
    return h.hexdigest()[:16]


def traffic_fields(kernel: str, scale: float = 1.0) -> dict:
    """The recorded counter traffic of `kernel` (times `scale`), or null when the kernel's sources are no longer the
    ones the counter runs were taken from."""
    value, source, files, sha = STATIC_TRAFFIC[kernel]
    now = source_fingerprint(files)
    if now != sha:
        return {"traffic": None, "traffic_source": f"not collected for this build of the kernel (sources {now}, counter runs "
                                                   f"in {source} were taken from {sha})"}
    return {"traffic": value * scale,
            "traffic_source": f"static: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs recorded in {source} (sources {sha})"}


def log(msg: str) -> None:
    print(msg, file=sys.stderr, flush=True)


def cpu_baseline(logits, ids, gpu_out, sample_rows: int):
    """Time the fp32 torch CPU oracle on `sample_rows` rows taken evenly from the tensor, and compare what it
    returns with the GPU result of the timed run on those rows (all of them by default)."""
    import torch
    from oracle import logprob_ref

    blk = 2048
    n_blocks = max(1, sample_rows // blk)
    total_rows = logits.shape[0]
    starts = [int(i * (total_rows - blk) / max(1, n_blocks - 1)) // blk * blk for i in range(n_blocks)]
    elapsed, rows, max_err, spike_err, spike_rows, spike_hits = 0.0, 0, 0.0, 0.0, 0, 0
    flat_out = gpu_out.reshape(-1)
    for s in starts:
        lc, ic = logits[s:s + blk].cpu(), ids[s:s + blk].cpu()
        t0 = time.perf_counter()
        want = logprob_ref.logprob_ref(lc, ic)
        elapsed += time.perf_counter() - t0
        rows += lc.shape[0]
        err = (flat_out[s:s + blk].cpu() - want).abs()
        max_err = max(max_err, err.max().item())
        # rows that carry a +25 spike (N(0, 3^2) stays below 16 over 128,256 draws)
        spike_col = lc.argmax(dim=-1)
        is_spike = lc.gather(-1, spike_col.unsqueeze(-1)).squeeze(-1).float() >= 24.0
        if bool(is_spike.any()):
            spike_rows += int(is_spike.sum())
            spike_hits += int((is_spike & (spike_col == ic)).sum())
            spike_err = max(spike_err, err[is_spike].max().item())
    return {
        "value": rows / elapsed,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{rows} of {total_rows} tokens ({n_blocks} blocks of {blk} rows, fp32 torch CPU "
                  f"log_softmax+gather), {elapsed:.1f} s; host cpu_count={os.cpu_count()}",
        "parity": {"rows_compared": rows, "max_abs_err": max_err, "spike_rows": spike_rows,
                   "spike_rows_with_target_on_spike": spike_hits, "spike_rows_max_abs_err": spike_err,
                   "tolerance": PARITY_TOL, "ok": max_err <= PARITY_TOL},
    }


def sampling_latency(sampler, steps: int, warmup: int, cpu: bool = True):
    """Fused sampling on bf16 [B, 128256], T=0.7, top-k 50, top-p 0.9, uniforms from seed 1234."""
    import torch
    from benchmarks.workloads import cfg5_sampling

    out = {"config": "bf16 [B,128256] ~ N(0,3^2), T=0.7, top_k=50, top_p=0.9, one fp32 uniform per row (seed 1234)",
           "roofline_by_batch": {}}
    for batch in (64, 128, 256, 512, 1024):
        logits, u = cfg5_sampling(batch, device="cuda")
        for _ in range(max(warmup, 3)):
            sampler.sample(logits, top_k=50, top_p=0.9, temperature=0.7, uniforms=u)
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n = max(steps, 20)
        t0 = time.perf_counter()
        ev0.record()
        for _ in range(n):
            sampler.sample(logits, top_k=50, top_p=0.9, temperature=0.7, uniforms=u)
        ev1.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / n
        out[f"ms_b{batch}"] = wall_ms
        # Kernel time: the same launches straight through the C ABI with every buffer allocated beforehand, so that
        # the host keeps ahead of the GPU (a Python-level call costs more host time than the kernel runs).
        ids_out = torch.empty(batch, dtype=torch.int64, device="cuda")
        fn = sampler._lib.ka_sample_topk_topp_bf16
        args = (logits.data_ptr(), batch, logits.shape[1], logits.stride(0), 0.7, 50, 0.9, u.data_ptr(), ids_out.data_ptr(),
                None, 0, torch.cuda.current_stream().cuda_stream)
        for _ in range(10):
            fn(*args)
        torch.cuda.synchronize()
        ev0.record()
        for _ in range(200):
            fn(*args)
        ev1.record()
        torch.cuda.synchronize()
        kernel_ms = ev0.elapsed_time(ev1) / 200
        out[f"kernel_ms_b{batch}"] = kernel_ms
        gbps = batch * BYTES_PER_TOKEN / (kernel_ms * 1e-3) / 1e9
        out["roofline_by_batch"][f"b{batch}"] = {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                                 "frac": gbps / HBM_PEAK_GBPS, "kernel_ms": kernel_ms,
                                                 "bytes_per_launch": batch * BYTES_PER_TOKEN,
                                                 **traffic_fields("sample_rows", (2 * _SAMPLING_KIB[batch][0] + _SAMPLING_KIB[batch][1])
                                                                  / (2 * _SAMPLING_KIB[256][0] + _SAMPLING_KIB[256][1]))}
        # a decode step: the id and its log-probability under the unfiltered softmax from the one kernel; checked once
        # against the logprob operator on the drawn ids before it is timed
        d_ids, d_pol = sampler.sample(logits, top_k=50, top_p=0.9, temperature=0.7, uniforms=u, return_policy_logprob=True)
        d_err = (d_pol - sampler.compute_logp(logits, d_ids)).abs().max().item()
        out[f"decode_step_policy_max_abs_diff_b{batch}"] = d_err
        assert d_err <= 1e-5, f"decode step: policy log-probability differs from compute_logp by {d_err}"
        for _ in range(5):
            sampler.sample(logits, top_k=50, top_p=0.9, temperature=0.7, uniforms=u, return_policy_logprob=True)
        torch.cuda.synchronize()
        ev0.record()
        for _ in range(100):
            sampler.sample(logits, top_k=50, top_p=0.9, temperature=0.7, uniforms=u, return_policy_logprob=True)
        ev1.record()
        torch.cuda.synchronize()
        out[f"decode_step_ms_b{batch}"] = ev0.elapsed_time(ev1) / 100
        if batch == 256:
            out["roofline"] = {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                               "frac": gbps / HBM_PEAK_GBPS, **traffic_fields("sample_rows"), "kernel": "sample_rows<Bf16>"}
            # the other filter combinations at the same batch (kernel time per call, microseconds)
            modes = {}
            for name, kw in (("no_filter_T1", dict(temperature=1.0)), ("no_filter_T0.7", dict(temperature=0.7)),
                             ("top_p0.9_T0.7", dict(top_p=0.9, temperature=0.7)),
                             ("top_k2000_top_p0.9_T0.7", dict(top_k=2000, top_p=0.9, temperature=0.7)),
                             ("top_k50_T0.7", dict(top_k=50, temperature=0.7))):
                for _ in range(3):
                    sampler.sample(logits, uniforms=u, **kw)
                torch.cuda.synchronize()
                ev0.record()
                for _ in range(20):
                    sampler.sample(logits, uniforms=u, **kw)
                ev1.record()
                torch.cuda.synchronize()
                modes[name] = ev0.elapsed_time(ev1) / 20 * 1e3
            out["other_modes_us_b256"] = modes
            if cpu:
                # The torch restatement of the reference's native_sampling and the exact C definition, timed on
                # the host on the same rows (median of 3); both also check the ids of the GPU run.
                from oracle import exact, sampling_ref
                got = sampler.sample(logits, top_k=50, top_p=0.9, temperature=0.7, uniforms=u).cpu()
                lc, uc = logits.cpu(), u.cpu()
                times = {"torch_restatement": [], "exact_c": []}
                for _ in range(3):
                    t0 = time.perf_counter()
                    want_t, _ = sampling_ref.sample(lc, top_k=50, top_p=0.9, temperature=0.7, uniforms=uc)
                    times["torch_restatement"].append(time.perf_counter() - t0)
                    t0 = time.perf_counter()
                    want_c = exact.sample(lc, 0.7, 50, 0.9, uc)
                    times["exact_c"].append(time.perf_counter() - t0)
                out["cpu_baseline"] = {
                    "unit": "ms", "batch": batch, "cores": torch.get_num_threads(), "kind": "port",
                    "torch_restatement_ms": sorted(times["torch_restatement"])[1] * 1e3,
                    "exact_c_ms_single_thread": sorted(times["exact_c"])[1] * 1e3,
                    "ids_equal_exact": bool(torch.equal(got, want_c)),
                    "ids_equal_torch_restatement": bool(torch.equal(got, want_t.to(got.dtype).view(-1)))}
    return out


def backward_throughput(sampler, iters: int = 5):
    """Backward of the logprob operator, in place, on bf16 logits [64, 512, 128256] (seed 0)."""
    import torch
    from benchmarks.workloads import spike_logits

    from rl_engine.kernels import sampling as sampling_mod

    n = 64 * 512
    rows_per_launch = min(n, sampling_mod.DEFAULT_CHUNK_TOKENS)
    logits, ids = spike_logits(n, V, seed=0, device="cuda")
    grad = torch.ones(n, device="cuda")
    logp = sampler.compute_logp(logits, ids)
    work = logits.clone()
    for _ in range(2):
        sampler.compute_logp_backward(work, ids, logp, grad, inplace=True)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(iters):  # the values degrade from pass to pass, the traffic does not
        sampler.compute_logp_backward(work, ids, logp, grad, inplace=True)
    ev1.record()
    torch.cuda.synchronize()
    ms = ev0.elapsed_time(ev1) / iters
    gbps = n * (4 * V + 16) / (ms * 1e-3) / 1e9
    return {"config": "bf16 logits [64,512,128256], gradient written in place; 4*V + 16 bytes per token",
            "ms": ms, "tokens_per_s": n / (ms * 1e-3),
            "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": gbps / HBM_PEAK_GBPS, **traffic_fields("logprob_backward_rows", rows_per_launch / 32768),
                         "kernel": "logprob_backward_rows<Bf16,1024,4,vec>", "rows_per_launch": rows_per_launch,
                         "bytes_per_launch": rows_per_launch * (4 * V + 16)}}


def lmhead_throughput(sampler, iters: int = 3):
    """Fused lm_head -> logprob on hidden bf16 [32768, 4096] x W bf16 [128256, 4096] (seed 0)."""
    import torch

    n, h, v = 64 * 512, 4096, V
    g = torch.Generator(device="cuda").manual_seed(0)
    hidden = torch.randn(n, h, generator=g, device="cuda").bfloat16()
    weight = (torch.randn(v, h, generator=g, device="cuda") * 0.02).bfloat16()
    ids = torch.randint(0, v, (n,), generator=g, device="cuda")
    for _ in range(2):
        sampler.fused_linear_logp(hidden, weight, ids)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(iters):
        out = sampler.fused_linear_logp(hidden, weight, ids)
    ev1.record()
    torch.cuda.synchronize()
    ms = ev0.elapsed_time(ev1) / iters
    tflops = 2.0 * n * h * v / (ms * 1e-3) / 1e12
    assert bool(torch.isfinite(out).all())
    # Decode-sized calls (the call in front of a sampling step): one token block, bound by streaming W once from HBM.
    decode = {}
    w_bytes = v * h * 2
    for rows in (64, 256):
        hs, is_ = hidden[:rows], ids[:rows]
        assert torch.equal(sampler.fused_linear_logp(hs, weight, is_), out[:rows]), "a row's result depends on the row count"
        for _ in range(3):
            sampler.fused_linear_logp(hs, weight, is_)
        torch.cuda.synchronize()
        ev0.record()
        for _ in range(20):
            sampler.fused_linear_logp(hs, weight, is_)
        ev1.record()
        torch.cuda.synchronize()
        ms_small = ev0.elapsed_time(ev1) / 20
        alg = w_bytes + rows * (h * 2 + 8 + 4)
        gbps = alg / (ms_small * 1e-3) / 1e9
        decode[f"n{rows}"] = {"ms": ms_small, "bit_identical_to_the_rows_of_the_large_call": True,
                              "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                           "frac": gbps / HBM_PEAK_GBPS, "bytes_per_call": alg,
                                           **traffic_fields(f"lmhead_n{rows}"),
                                           "kernel": ("lmhead_partials_narrow" if rows <= 128 else "lmhead_partials (units as "
                                                      "work items)") + " + lmhead_combine_units"}}
    return {"config": "hidden bf16 [32768,4096] ~ N(0,1), W bf16 [128256,4096] ~ N(0,0.02^2), seed 0; logits never stored",
            "ms": ms, "tokens_per_s": n / (ms * 1e-3),
            "roofline": {"bound": "mfma", "achieved": tflops, "peak": 2500.0, "unit": "TFLOP/s",
                         "frac": tflops / 2500.0, **traffic_fields("lmhead_partials"), "kernel": "lmhead_partials"},
            "decode_sized": decode}


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-sample-rows", type=int, default=131072,
                    help="rows of the tensor the CPU oracle is timed on (0 = skip)")
    ap.add_argument("--chunk-tokens", type=int, default=None, help="rows per kernel launch")
    ap.add_argument("--skip-lmhead", action="store_true", help="leave the fused lm_head->logprob figure out")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy (torch copy_) three times, so a counter "
                         "run of this command holds a kernel of known traffic to scale FETCH/WRITE_SIZE by")
    args = ap.parse_args()
    if args.gpus != 1:
        log(f"bench.py measures one GPU: --gpus {args.gpus} is not supported in this build "
            "(token rows are independent; more GPUs would each take a slice of the rows)")
        return 2

    import torch
    from rl_engine.utils.logger import logger

    for handler in logger.handlers:  # stdout carries the JSON line only
        handler.setStream(sys.stderr)
    from benchmarks.workloads import spike_logits
    from rl_engine.kernels import _hip as _hip_mod
    from rl_engine.kernels import sampling as sampling_mod
    from rl_engine.kernels.sampling import SamplerBackend

    if not torch.cuda.is_available():
        log("bench.py needs an MI355X: no GPU visible")
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    sampler = SamplerBackend().to(dev)
    chunk = args.chunk_tokens or sampling_mod.DEFAULT_CHUNK_TOKENS

    n_rows = G * L
    log(f"generating bf16 logits [{G},{L},{V}] ({n_rows * V * 2 / 1e9:.1f} GB) on {torch.cuda.get_device_name(0)}")
    logits, ids = spike_logits(n_rows, V, seed=0, device=dev)
    logits3, ids2 = logits.view(G, L, V), ids.view(G, L)
    torch.cuda.synchronize()

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        sampler.compute_logp(logits3, ids2, chunk_tokens=chunk)
    torch.cuda.synchronize()
    # Device memory one call needs beyond what is resident before it (logits + ids): the [G, L] fp32 result and
    # whatever the operator allocates on the way (nothing of the size of the logits).
    resident = torch.cuda.memory_allocated(dev)
    torch.cuda.reset_peak_memory_stats(dev)
    sampler.compute_logp(logits3, ids2, chunk_tokens=chunk)
    torch.cuda.synchronize()
    extra_device_bytes = torch.cuda.max_memory_allocated(dev) - resident

    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(args.steps):
        out = sampler.compute_logp(logits3, ids2, chunk_tokens=chunk)
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    launches_per_step = (n_rows + chunk - 1) // chunk
    # The events sit on the stream the kernels were launched on (torch's current stream).
    launch_ms = ev0.elapsed_time(ev1) / (args.steps * launches_per_step)
    rows_per_launch = n_rows / launches_per_step
    achieved_gbps = rows_per_launch * BYTES_PER_TOKEN / (launch_ms * 1e-3) / 1e9
    tokens_per_s = n_rows / (ms_per_step * 1e-3)

    result = {
        "metric": "logprob tokens/s (G=256,L=512,V=128256)",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "GRPO large-group logprob: bf16 logits [256,512,128256] ~ N(0,3^2) + 1% spike "
                               "rows, ids uniform, seed 0", "chunk_tokens": chunk,
                   "launches_per_step": launches_per_step, "input_dtype": "bf16", "output_dtype": "f32"},
        "hbm_gbps": n_rows * BYTES_PER_TOKEN / (ms_per_step * 1e-3) / 1e9,
        "extra_device_bytes": extra_device_bytes,
        "resident_bytes": resident,
        # what the library holds on the device whatever is called: the static array behind
        # ka_lmhead_logprob_bf16_noalloc (loaded with the code object) and, once fused_linear_logp has run, the pool arena
        "library_static_scratch_bytes": _hip_mod.LMHEAD_STATIC_SCRATCH_BYTES,
        "pool_capacity_bytes": sampler.pool.capacity,
        "roofline": {"bound": "hbm", "achieved": achieved_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved_gbps / HBM_PEAK_GBPS,
                     **traffic_fields("logprob_rows", rows_per_launch / 131072),
                     "kernel": "logprob_rows<Bf16,256,4,vec>", "launch_ms": launch_ms,
                     "bytes_per_launch": rows_per_launch * BYTES_PER_TOKEN},
    }
    assert bool(torch.isfinite(out).all()), "non-finite logprob in the timed run"
    if args.cpu_sample_rows > 0:
        log("timing the CPU oracle on a sample of the same tensor")
        result["cpu_baseline"] = cpu_baseline(logits, ids, out, args.cpu_sample_rows)
    del logits3, ids2, logits, ids
    torch.cuda.empty_cache()
    result["logprob_backward"] = backward_throughput(sampler)
    result["sampling"] = sampling_latency(sampler, args.steps, args.warmup, cpu=args.cpu_sample_rows > 0)
    if not args.skip_lmhead:
        result["fused_lm_head"] = lmhead_throughput(sampler)
    result["pool_allocated_bytes_at_exit"] = sampler.pool.allocated_bytes()
    print(json.dumps(result), flush=True)
    parity = result.get("cpu_baseline", {}).get("parity")
    if parity is not None and not parity["ok"]:
        log(f"PARITY FAILURE: max |GPU - CPU oracle| = {parity['max_abs_err']:.3e} > {PARITY_TOL}")
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
