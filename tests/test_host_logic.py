"""Host side of the op API on a machine without a GPU: construction, validation, pool, side API."""
import logging

import pytest
import torch

from rl_engine.executors.rollout import RolloutExecutor
from rl_engine.kernels.pool import MAX_POOL_BYTES, PoolExhausted, WorkspacePool
from rl_engine.kernels.registry import OpBackend, kernel_registry
from rl_engine.kernels.sampling import SamplerBackend
from rl_engine.platforms.device import device_ctx
from rl_engine.utils.logger import logger


def test_sampler_constructs_like_the_reference_module():
    s = SamplerBackend()
    assert isinstance(s, torch.nn.Module) and list(s.parameters()) == []
    assert s.backend == "hip_native"
    assert s.to("cpu") is s


def test_no_cpu_path():
    s = SamplerBackend()
    with pytest.raises(RuntimeError, match="no CPU path"):
        s.compute_logp(torch.zeros(2, 3, 8, dtype=torch.bfloat16), torch.zeros(2, 3, dtype=torch.int64))
    with pytest.raises(RuntimeError, match="no CPU path"):
        s.sample(torch.zeros(2, 8), top_k=2)
    with pytest.raises(RuntimeError, match="no CPU path"):
        s.fused_linear_logp(torch.zeros(2, 8, dtype=torch.bfloat16), torch.zeros(4, 8, dtype=torch.bfloat16),
                            torch.zeros(2, dtype=torch.int64))


def test_pool_is_fixed_size_and_never_grows():
    pool = WorkspacePool(1 << 20)
    assert pool.capacity == 1 << 20 and pool.allocated_bytes() == 0
    with pytest.raises(ValueError):
        WorkspacePool(MAX_POOL_BYTES + 1)
    with pytest.raises(ValueError):
        WorkspacePool(0)
    pool._arenas[0] = torch.empty(pool.capacity, dtype=torch.uint8)   # stand-in arena on the CPU
    dev = torch.device("cuda", 0)
    a = pool.reserve(1000, dev)
    b = pool.reserve(5000, dev)
    assert a.numel() == 1000 and b.numel() == 5000
    assert b.data_ptr() - a.data_ptr() == 1024 and b.data_ptr() % 256 == a.data_ptr() % 256
    with pytest.raises(PoolExhausted):
        pool.reserve(1 << 20, dev)
    pool.reset()
    assert pool.reserve(1 << 20, dev).numel() == 1 << 20


def test_device_context_and_logger():
    assert device_ctx.get_preferred_dtype() == torch.bfloat16
    assert device_ctx.device_type in ("rocm", "cpu")
    assert device_ctx.is_rocm == torch.cuda.is_available()
    seen = []
    import logging

    class Grab(logging.Handler):
        def emit(self, record):
            seen.append(record.getMessage())

    h = Grab()
    logger.addHandler(h)
    try:
        for _ in range(3):
            logger.info_once("only once %s", "x")
        logger.warn_once("warn once")
        logger.warn_once("warn once")
        logger.info_on_rank("rank zero")
        logger.info_on_rank("rank one", 1)
    finally:
        logger.removeHandler(h)
    assert seen == ["only once x", "warn once", "rank zero"]


def test_registry_and_executor():
    assert kernel_registry.dispatch("fused_logp") == "HIP_LOGPROB"
    assert kernel_registry.dispatch("sampling") == "HIP_SAMPLING"
    assert kernel_registry.dispatch("fused_lm_head_logp") == "HIP_FUSED_LMHEAD_LOGPROB"
    assert kernel_registry.get_op_path(OpBackend.HIP_LOGPROB).endswith("SamplerBackend.compute_logp")
    # the reference's dispatch always answers with a name (registry.py:41-55); its callers pass "attention"
    assert kernel_registry.dispatch("attention") == "NOT_ON_HIP_PATH"
    assert isinstance(kernel_registry.get_op_path(OpBackend.NOT_ON_HIP_PATH), str)
    with pytest.raises(ValueError, match="no HIP operator"):
        kernel_registry.resolve("attention")
    with pytest.raises(ValueError, match="Supported backends"):
        OpBackend["FLASHINFER"]
    fn = kernel_registry.resolve("fused_logp")
    assert fn.__name__ == "compute_logp"
    out = RolloutExecutor({"top_k": 50}).execute_rollout()
    assert out["status"] == "success" and out["kernels"] == ["HIP_LOGPROB", "NOT_ON_HIP_PATH"]
    assert out["sampling_kernel"] == "HIP_SAMPLING"


def test_reference_dispatch_smoke_flow():
    """The flow of the reference's smoke script (rl_engine/tests/test_dispatch.py:9-27), with assertions:
    once-only logging, the device probe's attributes, dispatch of the two names its callers pass, and the
    executor's result shape."""
    from rl_engine.platforms.device import device_ctx

    seen = []

    class Grab(logging.Handler):
        def emit(self, record):
            seen.append(record.getMessage())

    h = Grab()
    logger.addHandler(h)
    try:
        logger.info("standard info log")
        for _ in range(3):
            logger.info_once("a unique message that appears only once")
    finally:
        logger.removeHandler(h)
    assert seen == ["standard info log", "a unique message that appears only once"]
    assert isinstance(device_ctx.device_type, str) and isinstance(device_ctx.is_rocm, bool)
    logp_op = kernel_registry.dispatch("fused_logp")
    attn_op = kernel_registry.dispatch("attention")
    assert isinstance(logp_op, str) and isinstance(attn_op, str) and logp_op != attn_op
    assert OpBackend[logp_op] is OpBackend.HIP_LOGPROB and OpBackend[attn_op] is OpBackend.NOT_ON_HIP_PATH
    result = RolloutExecutor().execute_rollout()
    assert result["status"] == "success" and result["kernels"] == [logp_op, attn_op]


def test_generate_checks_its_arguments_and_never_falls_back_to_the_cpu():
    executor = RolloutExecutor({"top_k": 4})
    with pytest.raises(ValueError, match="prompt_ids"):
        executor.generate(lambda ids: None, torch.zeros(3, dtype=torch.int64), 2)
    with pytest.raises(ValueError, match="uniforms"):
        executor.generate(lambda ids: None, torch.zeros(2, 3, dtype=torch.int64), 2, uniforms=torch.zeros(2, 3))
    with pytest.raises((RuntimeError, ValueError)):     # CPU logits are refused by the operators
        executor.generate(lambda ids: torch.zeros(2, 16), torch.zeros(2, 3, dtype=torch.int64), 1)


def test_chunk_rows_validation():
    """Every chunked operator takes its launch granularity from one checked helper: a value below one row would
    make the launch loop empty and return uninitialised memory."""
    from rl_engine.kernels.sampling import DEFAULT_CHUNK_TOKENS, _chunk_rows

    assert _chunk_rows(None) == DEFAULT_CHUNK_TOKENS and _chunk_rows(7) == 7
    for bad in (0, -1, -8192):
        with pytest.raises(ValueError, match="chunk_tokens"):
            _chunk_rows(bad)
