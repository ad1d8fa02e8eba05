"""rl_engine: MI355X-native implementation of Kernel-Align's logprob and sampling operators.

The Python op API mirrors the reference package of the same name
(rl_engine/kernels/sampling.py, rl_engine/platforms/device.py,
rl_engine/utils/logger.py); the compute runs in hand-written HIP kernels for
gfx950, loaded from libkernel_align_hip.so through ctypes.
"""

__version__ = "0.1.0"
