"""Rollout executor: picks the operators for the sampling phase.

Interface of the reference's rl_engine/executors/rollout.py:8-35.  The reference
is a stub that returns two backend names; here the names are those of the HIP
operators, and ``step`` runs them on a batch of next-token logits.
"""
from __future__ import annotations

from typing import Callable, Optional, Tuple

import torch

from rl_engine.kernels.registry import kernel_registry
from rl_engine.utils.logger import logger


class RolloutExecutor:
    def __init__(self, model_config: Optional[dict] = None):
        self.config = model_config or {}
        logger.info("Initializing RolloutExecutor on the HIP operators...")

    def _select_operators(self) -> Tuple[str, str]:
        """The two names the reference selects (rollout.py:17-28): the logprob operator and "attention",
        which is outside the HIP hot path and is answered with the NOT_ON_HIP_PATH name."""
        logp_be = kernel_registry.dispatch("fused_logp")
        attn_be = kernel_registry.dispatch("attention")
        logger.info_once(f"Selected Logp backend: {logp_be}")
        logger.info_once(f"Selected Attention backend: {attn_be}")
        return logp_be, attn_be

    def execute_rollout(self):
        """Same result shape as rollout.py:30-35, plus the name of the sampling operator `step` runs."""
        logp_op, attn_op = self._select_operators()
        logger.info_once(f"Starting rollout via {logp_op}...")
        return {"status": "success", "kernels": [logp_op, attn_op],
                "sampling_kernel": kernel_registry.dispatch("sampling")}

    def step(self, logits, uniforms=None):
        """One decode step: sample a token per row of `logits` [B, V] and return (ids, logprobs)."""
        sample = kernel_registry.resolve("sampling")
        # both kernels from one operator call: at small batches the host time of a call exceeds the kernels' time
        return sample(logits, top_k=self.config.get("top_k"), top_p=self.config.get("top_p"),
                      temperature=self.config.get("temperature", 1.0), uniforms=uniforms, return_policy_logprob=True)

    def generate(self, next_logits: Callable, prompt_ids, max_new_tokens: int, uniforms=None,
                 eos_id: Optional[int] = None):
        """Autoregressive rollout of a group: ``next_logits(ids [B, t]) -> [B, V]`` supplies the logits of
        the next position; each step samples with the configured filters and records the log-probability
        of the drawn token under the unfiltered distribution (what the GRPO ratio is built from).

        prompt_ids: int64 [B, T0].  uniforms: optional fp32 [max_new_tokens, B], one draw per row and step.
        Rows that have produced ``eos_id`` keep emitting it with log-probability 0.  No step synchronises
        with the host.  Returns (ids [B, T0 + max_new_tokens], logprobs fp32 [B, max_new_tokens]).
        """
        if prompt_ids.dim() != 2:
            raise ValueError("prompt_ids must be [B, T0]")
        batch, t0 = prompt_ids.shape
        if uniforms is not None and tuple(uniforms.shape) != (max_new_tokens, batch):
            raise ValueError(f"uniforms must have shape ({max_new_tokens}, {batch})")
        ids = torch.empty(batch, t0 + max_new_tokens, dtype=torch.int64, device=prompt_ids.device)
        ids[:, :t0] = prompt_ids
        logprobs = torch.zeros(batch, max_new_tokens, dtype=torch.float32, device=prompt_ids.device)
        done = torch.zeros(batch, dtype=torch.bool, device=prompt_ids.device)
        for step in range(max_new_tokens):
            logits = next_logits(ids[:, :t0 + step])
            tok, lp = self.step(logits, None if uniforms is None else uniforms[step])
            if eos_id is not None:
                tok = torch.where(done, torch.full_like(tok, eos_id), tok)
                lp = torch.where(done, torch.zeros_like(lp), lp)
                done = done | (tok == eos_id)
            ids[:, t0 + step] = tok
            logprobs[:, step] = lp
        return ids, logprobs
