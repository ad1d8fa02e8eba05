"""Build the C restatement under oracle/ into oracle/_build/ (test infrastructure only)."""
from __future__ import annotations

import os
import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
OUT_DIR = HERE / "_build"
LIB = OUT_DIR / "libka_oracle.so"
# No contraction, no fast-math: every operation is a single IEEE-754 operation.
CFLAGS = ["-O2", "-std=c11", "-fPIC", "-shared", "-ffp-contract=off", "-fno-fast-math", "-Wall", "-Wextra"]


def build_oracle() -> Path:
    src = HERE / "ka_oracle.c"
    OUT_DIR.mkdir(exist_ok=True)
    tmp = LIB.with_suffix(".so.tmp")
    proc = subprocess.run(["gcc", *CFLAGS, "-o", str(tmp), str(src), "-lm"], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"gcc failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build_oracle())
