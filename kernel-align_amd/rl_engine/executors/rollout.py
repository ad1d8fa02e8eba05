"""Rollout executor: picks the operators for the sampling phase.

Interface of the reference's rl_engine/executors/rollout.py:8-35.  The reference
is a stub that returns two backend names; here the names are those of the HIP
operators, and ``step`` runs them on a batch of next-token logits.
"""
from __future__ import annotations

from typing import Optional, Tuple

from rl_engine.kernels.registry import kernel_registry
from rl_engine.utils.logger import logger


class RolloutExecutor:
    def __init__(self, model_config: Optional[dict] = None):
        self.config = model_config or {}
        logger.info("Initializing RolloutExecutor on the HIP operators...")

    def _select_operators(self) -> Tuple[str, str]:
        logp_be = kernel_registry.dispatch("fused_logp")
        sample_be = kernel_registry.dispatch("sampling")
        logger.info_once(f"Selected Logp backend: {logp_be}")
        logger.info_once(f"Selected Sampling backend: {sample_be}")
        return logp_be, sample_be

    def execute_rollout(self):
        logp_op, sample_op = self._select_operators()
        logger.info_once(f"Starting rollout via {logp_op}...")
        return {"status": "success", "kernels": [logp_op, sample_op]}

    def step(self, logits, uniforms=None):
        """One decode step: sample a token per row of `logits` [B, V] and return (ids, logprobs)."""
        sample = kernel_registry.resolve("sampling")
        logp = kernel_registry.resolve("fused_logp")
        ids = sample(logits, top_k=self.config.get("top_k"), top_p=self.config.get("top_p"),
                     temperature=self.config.get("temperature", 1.0), uniforms=uniforms)
        return ids, logp(logits, ids)
