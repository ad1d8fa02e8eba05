"""Vocabulary of the ROCm-only engine.

The reference's rl_engine/platforms/constants.py:82-97 bundles a dozen enums of
which the operators read only the backend name; this build keeps the enums the
hot path touches and names a single backend, the in-tree HIP library.
"""
from __future__ import annotations

from enum import Enum


class DeviceType(Enum):
    ROCM = "rocm"
    CPU = "cpu"  # reported when no GPU is visible; no operator runs there


class BackendLib(Enum):
    HIP_NATIVE = "hip_native"  # hand-written gfx950 kernels in libkernel_align_hip.so


class PrecisionType(Enum):
    FP32 = "float32"
    FP16 = "float16"
    BF16 = "bfloat16"


class SamplingMethod(Enum):
    GREEDY = "greedy"
    TEMPERATURE = "temperature"
    TOP_K = "top_k"
    TOP_P = "top_p"
    TOP_K_TOP_P = "top_k_top_p"


class Constants:
    """Namespace object, so call sites read `constants.BackendLib.HIP_NATIVE`."""

    DeviceType = DeviceType
    BackendLib = BackendLib
    PrecisionType = PrecisionType
    SamplingMethod = SamplingMethod


constants = Constants()
