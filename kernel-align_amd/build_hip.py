"""Build libkernel_align_hip.so from csrc/*.hip with hipcc for gfx950.

Usage: python kernel-align_amd/build_hip.py [--verbose] [--keep-temps]

The library is written to kernel-align_amd/lib/ (in-tree, git-ignored).  hipcc
cross-compiles the device code, so no GPU is needed to build.
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_ROOT = Path(__file__).resolve().parent
REPO_ROOT = PKG_ROOT.parent
CSRC = PKG_ROOT / "csrc"
LIB_DIR = PKG_ROOT / "lib"
OBJ_DIR = PKG_ROOT / "build"
LIB_PATH = LIB_DIR / "libkernel_align_hip.so"
ARCH = "gfx950"

# Packed-fp32 VALU forms are switched off: only scalar fp32 arithmetic is emitted.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{REPO_ROOT / 'include'}",
    f"-I{CSRC}",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found: the HIP library cannot be built")
    return exe


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(str(c) for c in cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass reports the packed-fp32 feature as unknown; that is expected.
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(map(str, cmd))}\n{proc.stdout}\n{err}")
    if verbose and err.strip():
        print(err, flush=True)


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def build_library(verbose: bool = False, keep_temps: bool = False, jobs: int | None = None) -> Path:
    """Compile every csrc/*.hip and link the shared library.  Always recompiles."""
    hipcc = _hipcc()
    LIB_DIR.mkdir(exist_ok=True)
    OBJ_DIR.mkdir(exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    objs = [OBJ_DIR / (s.stem + ".o") for s in srcs]
    extra = ["-save-temps=obj"] if keep_temps else []

    def compile_one(pair):
        src, obj = pair
        _run([hipcc, *HIPCC_FLAGS, *extra, "-c", str(src), "-o", str(obj)], verbose)

    workers = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 8)
    with ThreadPoolExecutor(max_workers=max(1, workers)) as pool:
        list(pool.map(compile_one, zip(srcs, objs)))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)], verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--verbose", action="store_true")
    ap.add_argument("--keep-temps", action="store_true", help="keep .s / .bc files beside the objects")
    args = ap.parse_args()
    path = build_library(verbose=args.verbose, keep_temps=args.keep_temps)
    print(f"built {path} ({path.stat().st_size} bytes)")
    sys.exit(0)
