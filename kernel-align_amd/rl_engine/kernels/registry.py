"""Name-level operator registry (ROCm only).

Keeps the interface of the reference's rl_engine/kernels/registry.py:32-60
(``kernel_registry.dispatch(op_type) -> str``, ``get_op_path``) but every name
now points at code that exists: the HIP-backed methods of SamplerBackend.
``resolve`` additionally returns the bound callable.
"""
from __future__ import annotations

from enum import Enum, EnumMeta
from typing import Callable, Dict

from rl_engine.platforms.device import device_ctx
from rl_engine.utils.logger import logger


class _OpEnumMeta(EnumMeta):
    def __getitem__(cls, name: str):
        try:
            return super().__getitem__(name)
        except KeyError:
            raise ValueError(
                f"Operator '{name}' not found. Supported backends: {', '.join(cls.__members__)}"
            ) from None


class OpBackend(Enum, metaclass=_OpEnumMeta):
    HIP_LOGPROB = "rl_engine.kernels.sampling.SamplerBackend.compute_logp"
    HIP_FUSED_LMHEAD_LOGPROB = "rl_engine.kernels.sampling.SamplerBackend.fused_linear_logp"
    HIP_SAMPLING = "rl_engine.kernels.sampling.SamplerBackend.sample"
    # Operators the reference's callers ask for by name (e.g. "attention", rollout.py:23) that lie outside the
    # HIP hot path: dispatch() still answers with a name, as registry.py:41-55 always does; resolve() refuses.
    NOT_ON_HIP_PATH = "rl_engine.kernels.registry.not_on_hip_path"


class KernelRegistry:
    def __init__(self) -> None:
        self._runtime_overrides: Dict[OpBackend, str] = {}
        self._sampler = None
        logger.info(f"KernelRegistry initialized for {device_ctx.device_type}")

    def dispatch(self, op_type: str) -> str:
        """Name of the backend serving `op_type` (substring match, as in registry.py:41-55)."""
        if "lm_head" in op_type or "linear" in op_type:
            return OpBackend.HIP_FUSED_LMHEAD_LOGPROB.name
        if "logp" in op_type:
            return OpBackend.HIP_LOGPROB.name
        if "sampl" in op_type:
            return OpBackend.HIP_SAMPLING.name
        return OpBackend.NOT_ON_HIP_PATH.name

    def get_op_path(self, backend: OpBackend) -> str:
        return self._runtime_overrides.get(backend, backend.value)

    def resolve(self, op_type: str) -> Callable:
        """The bound method that implements `op_type`, on a lazily built shared SamplerBackend."""
        backend = OpBackend[self.dispatch(op_type)]
        if backend is OpBackend.NOT_ON_HIP_PATH:
            raise ValueError(f"no HIP operator serves '{op_type}' (known: logp, lm_head/linear, sampling)")
        if self._sampler is None:
            from rl_engine.kernels.sampling import SamplerBackend

            self._sampler = SamplerBackend()
        return getattr(self._sampler, self.get_op_path(backend).rsplit(".", 1)[1])


def not_on_hip_path(*_args, **_kwargs):
    """Target of OpBackend.NOT_ON_HIP_PATH: there is no kernel behind the name."""
    raise NotImplementedError("this operator is not part of the HIP hot path (logprob, lm_head logprob, sampling)")


kernel_registry = KernelRegistry()
