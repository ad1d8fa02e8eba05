"""Device probe singleton (ROCm only).

Same attributes as the reference's DeviceContext
(rl_engine/platforms/device.py:8-44): ``device``, ``is_rocm``, ``device_type``,
``backend_version`` and ``get_preferred_dtype()``.  The CUDA branch is gone: a
visible GPU is an AMD GPU driven through HIP, and bf16 is its preferred dtype.
"""
from __future__ import annotations

import torch

from rl_engine.platforms.constants import DeviceType
from rl_engine.utils.logger import logger


class DeviceContext:
    def __init__(self) -> None:
        self.rank = 0
        self.backend_version = "N/A"
        self.arch = None
        has_gpu = torch.cuda.is_available()
        if has_gpu and torch.version.hip is None:
            raise RuntimeError("rl_engine is ROCm-only: this torch build has no HIP runtime")
        if has_gpu:
            self.device = torch.device("cuda")  # torch's name for a HIP device
            self.is_rocm = True
            self.device_type = DeviceType.ROCM.value
            self.backend_version = torch.version.hip
            props = torch.cuda.get_device_properties(0)
            self.arch = getattr(props, "gcnArchName", "").split(":")[0] or None
            logger.info_once(
                f"RL-Engine on AMD ROCm {self.backend_version}: {props.name} ({self.arch}), "
                f"{props.total_memory / 2**30:.0f} GiB HBM, {props.multi_processor_count} CUs"
            )
        else:
            self.device = torch.device("cpu")
            self.is_rocm = False
            self.device_type = DeviceType.CPU.value
            logger.warning("No GPU detected: rl_engine operators need an AMD GPU and will raise if called.")

    def get_preferred_dtype(self) -> torch.dtype:
        """bf16: what the gfx950 kernels are tuned for (reference: device.py:37-42)."""
        return torch.bfloat16


device_ctx = DeviceContext()
