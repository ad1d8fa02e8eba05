"""Build and run the hardware micro-benchmarks next to this file (hipcc, gfx950).

    python kernel-align_amd/benchmarks/micro/run_micro.py [hbm_read_ceiling|mfma_peak|hbm_rmw_ceiling|lds_read_patterns|l2_read_bandwidth|lmhead_copy_overlap ...]

They measure the ceilings the kernels are discussed against: the pure HBM read stream, the bf16 MFMA
peak of the instruction itself, ds_read_b128 throughput per LDS swizzle, L2 -> CU bandwidth, and how far the
lm_head kernel's copy pattern overlaps with its MFMAs.
"""
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
OUT = HERE.parents[1] / "build"


def main() -> int:
    names = sys.argv[1:] or sorted(p.stem for p in HERE.glob("*.hip"))
    OUT.mkdir(exist_ok=True)
    for name in names:
        exe = OUT / f"micro_{name}"
        subprocess.run(["hipcc", "--offload-arch=gfx950", "-O3", "-Wno-unused-result", str(HERE / f"{name}.hip"), "-o", str(exe)], check=True)
        print(f"== {name}", flush=True)
        subprocess.run([str(exe)], check=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
