"""Where the cycles of one sampling call go: builds the sampling kernels with -DKA_SAMPLE_STAMPS (workgroup 0 then
writes the shader clock at named points of the top-k route and of the dense-histogram route) and prints the phases for
B in {1, 64, 256} (top-k + top-p) and B in {64, 256} (top-p alone, at T = 0.7 and T = 1).

    python kernel-align_amd/benchmarks/sampling_phases.py [--top-k 50] [--top-p 0.9] [--temperature 0.7]

The stamped library is a separate build under kernel-align_amd/build/ (the product library carries no stamps).
Needs an MI355X.
"""
from __future__ import annotations

import argparse
import ctypes
import os
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parents[1]
REPO = PKG.parent
for _p in (REPO, PKG):
    if str(_p) not in sys.path:
        sys.path.insert(0, str(_p))

NAMES = {1: "read + lane maxima", 2: "bound", 3: "bound widened", 4: "candidate vectors", 10: "candidates", 5: "ranked",
         6: "prefix of masses", 7: "top-p cut", 8: "draw", 9: "end"}
ORDER_SHORT = (1, 2, 3, 4, 10, 5, 6, 7, 8, 9)
ORDER_BLOCK = (1, 2, 3, 4, 5, 7, 9)


def build_stamped() -> Path:
    out = PKG / "build" / "libka_sampling_stamped.so"
    out.parent.mkdir(exist_ok=True)
    cmd = ["hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-DKA_SAMPLE_STAMPS",
           f"-I{REPO / 'include'}", f"-I{PKG / 'csrc'}", str(PKG / "csrc" / "ka_api.hip"),
           str(PKG / "csrc" / "ka_sampling.hip"), "-o", str(out)]
    subprocess.run(cmd, check=True, stderr=subprocess.DEVNULL)
    return out


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--top-k", type=int, default=50)
    ap.add_argument("--top-p", type=float, default=0.9)
    ap.add_argument("--temperature", type=float, default=0.7)
    ap.add_argument("--lib", default=None, help="a stamped library built earlier (skips the build)")
    args = ap.parse_args()
    lib_path = Path(args.lib) if args.lib else build_stamped()
    os.environ["KERNEL_ALIGN_HIP_LIB"] = str(lib_path)
    import torch
    from benchmarks.workloads import cfg5_sampling
    from rl_engine.kernels import _hip

    # the stamped library holds the sampling entry points only
    _hip.SIGNATURES = {k: v for k, v in _hip.SIGNATURES.items()
                       if k.startswith(("ka_sample", "ka_version", "ka_last", "ka_status"))}
    from rl_engine.kernels.sampling import SamplerBackend

    sampler = SamplerBackend().cuda()
    lib = _hip.load()
    lib.ka_debug_read_stamps.argtypes = [ctypes.c_void_p, ctypes.c_int]
    buf = (ctypes.c_ulonglong * 288)()
    for batch in (1, 64, 256):
        logits, u = cfg5_sampling(batch, device="cuda")
        for flags, label, order in ((0, "short route", ORDER_SHORT),
                                    (_hip.SAMPLE_FLAG_BLOCK_WIDE_TOPK, "block-wide route", ORDER_BLOCK)):
            for _ in range(5):
                sampler.sample(logits, top_k=args.top_k, top_p=args.top_p, temperature=args.temperature, uniforms=u,
                               route_flags=flags)
            torch.cuda.synchronize()
            lib.ka_debug_read_stamps(buf, 288)
            st = list(buf)
            t0 = min(st[w * 16] for w in range(16))
            last_read = max(st[w * 16 + 1] for w in range(16)) - t0
            prev, parts = st[0], []
            for i in order:
                if st[i] and st[i] >= prev:
                    parts.append(f"{NAMES[i]} +{st[i] - prev}")
                    prev = st[i]
            print(f"B={batch:4d} {label:16s} {prev - st[0]:6d} cycles (wavefront 0; last wavefront has read its share at "
                  f"{last_read}): " + " | ".join(parts), flush=True)
    # the dense-histogram route (top-p without top-k): its own stamp names
    dense_names = {1: "histogram pass", 2: "occupied keys compacted", 3: "masses of the occupied keys",
                   4: "filters + mass table", 11: "survivors listed", 12: "drawn", 13: "masses of every share (streaming)",
                   14: "entry located"}
    for batch in (64, 256):
        logits, u = cfg5_sampling(batch, device="cuda")
        for temp, top_p in ((0.7, args.top_p), (1.0, args.top_p), (1.0, None)):
            for _ in range(3):
                sampler.sample(logits, top_p=top_p, temperature=temp, uniforms=u)
            torch.cuda.synchronize()
            lib.ka_debug_read_stamps(buf, 288)
            st = list(buf)
            prev, parts = st[0], []
            # (stamps of a route that this call did not take are left over from an earlier call: the later end wins)
            for i in ((1, 2, 3, 4, 11, 12) if st[12] > st[14] else (1, 2, 3, 4, 13, 14)):
                if st[i] > prev:
                    parts.append(f"{dense_names[i]} +{st[i] - prev}")
                    prev = st[i]
            tail = ""
            print(f"B={batch:4d} top_p={top_p} T={temp}: stamped {prev - st[0]:6d} cycles: " + " | ".join(parts) + tail, flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
