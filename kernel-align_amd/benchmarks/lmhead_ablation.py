"""What the fused lm_head kernel's time is made of: builds variants of csrc/ka_lmhead.hip with its LM_ABL_* switches
(no slab copies / no fragment reads / no epilogue / copies that always hit L2 / no wait for the copies) and its copy
schedule macros, times each at the headline shape (hidden [32768, 4096] x W [128256, 4096]), and reports the shader clock each one ran at (the part is power
limited under this kernel, so a variant's time is cycles / clock with a clock that depends on what the variant does).

    python kernel-align_amd/benchmarks/lmhead_ablation.py [--sustained]

Variants with an LM_ABL_* switch compute wrong results on purpose; only timings are meaningful.  The variant
libraries are built under kernel-align_amd/build/ and hold the lm_head entry points only.  Needs an MI355X.
"""
from __future__ import annotations

import argparse
import ctypes
import subprocess
import sys
import time
from ctypes import c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

PKG = Path(__file__).resolve().parents[1]
REPO = PKG.parent

VARIANTS = {
    "production": [],
    "copies per group 2 (all sixteen behind the barrier)": ["-DLM_COPY_SCHEDULE=4"],
    "no copies": ["-DLM_ABL_NOCOPY"],
    "no fragment reads": ["-DLM_ABL_NOREAD"],
    "no epilogue": ["-DLM_ABL_NOEPI"],
    "no copies, no fragment reads": ["-DLM_ABL_NOCOPY", "-DLM_ABL_NOREAD"],
    "MFMAs only": ["-DLM_ABL_NOCOPY", "-DLM_ABL_NOREAD", "-DLM_ABL_NOEPI"],
    "copies always hit L2": ["-DLM_ABL_HOTCOPY"],
    "copies not waited for": ["-DLM_ABL_NOVMWAIT"],
    "no barrier": ["-DLM_ABL_NOBAR"],
}


def build(name: str, flags: list[str]) -> Path:
    out = PKG / "build" / ("liblmhead_" + "".join(ch if ch.isalnum() else "_" for ch in name) + ".so")
    out.parent.mkdir(exist_ok=True)
    cmd = ["hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-DLM_ABL_CLOCK", *flags,
           f"-I{REPO / 'include'}", f"-I{PKG / 'csrc'}", str(PKG / "csrc" / "ka_api.hip"),
           str(PKG / "csrc" / "ka_lmhead.hip"), "-o", str(out)]
    subprocess.run(cmd, check=True, stderr=subprocess.DEVNULL)
    return out


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--sustained", action="store_true", help="time each variant over a 4 s loop (thermal steady state)")
    args = ap.parse_args()
    libs = {name: build(name, flags) for name, flags in VARIANTS.items()}
    import torch

    n, h, v = 32768, 4096, 128256
    g = torch.Generator(device="cuda").manual_seed(0)
    hidden = torch.randn(n, h, generator=g, device="cuda").bfloat16()
    weight = (torch.randn(v, h, generator=g, device="cuda") * 0.02).bfloat16()
    ids = torch.randint(0, v, (n,), generator=g, device="cuda")
    out = torch.empty(n, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    flop = 2.0 * n * h * v
    for name, path in libs.items():
        lib = ctypes.CDLL(str(path))
        lib.ka_lmhead_workspace_bytes.restype = c_size_t
        lib.ka_lmhead_workspace_bytes.argtypes = [c_int64] * 3
        lib.ka_lmhead_logprob_bf16.restype = c_int
        lib.ka_lmhead_logprob_bf16.argtypes = [c_void_p] * 4 + [c_int64] * 3 + [c_void_p, c_size_t, c_void_p]
        ws_bytes = lib.ka_lmhead_workspace_bytes(n, h, v)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")

        def call():
            rc = lib.ka_lmhead_logprob_bf16(hidden.data_ptr(), weight.data_ptr(), ids.data_ptr(), out.data_ptr(), n, h, v,
                                            ws.data_ptr(), ws_bytes, stream)
            assert rc == 0

        call(); call()
        torch.cuda.synchronize()
        times = []
        t_end = time.time() + (4.0 if args.sustained else 0.0)
        while True:
            e0.record()
            for _ in range(3):
                call()
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) / 3)
            if len(times) >= 4 and time.time() >= t_end:
                break
        ms = sorted(times)[len(times) // 2] if args.sustained else min(times)
        # with LM_ABL_CLOCK workgroup 0 leaves (shader cycles / 100 MHz ticks) of its life in the pad of partial 0
        mhz = ws[:16].view(torch.float32)[3].item() * 100.0
        print(f"{name:52s} {ms:7.2f} ms  {flop / ms / 1e9:7.0f} TFLOP/s  shader clock {mhz:5.0f} MHz  "
              f"-> {ms * mhz / 1e3:6.1f} M cycles", flush=True)
    x = hidden[:8192]
    for _ in range(2):
        x @ weight.T
    torch.cuda.synchronize()
    e0.record()
    for _ in range(5):
        x @ weight.T
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / 5 * 4
    print(f"{'hipBLASLt bf16 GEMM of the same product (4 x 8192 rows)':52s} {ms:7.2f} ms  {flop / ms / 1e9:7.0f} TFLOP/s")
    return 0


if __name__ == "__main__":
    sys.exit(main())
