"""CPU oracle of the per-token logprob operator.  Test infrastructure only.

Reference math (rl_engine/kernels/sampling.py:108-110 and the native comparator
benchmarks/benchmark_grpo_op.py:52-54):

    out[..., l] = log_softmax(logits, dim=-1).gather(-1, token_ids.unsqueeze(-1)).squeeze(-1)

The reference runs this in the logits' own dtype (bf16 on ROCm,
rl_engine/platforms/device.py:37-42), which returns bf16 and is ~7e-2 away from
the true value; the oracle upcasts to fp32 first (`logprob_ref`), which is the
"reference CPU torch path" at fp32 output, and also offers an fp64 evaluation
(`logprob_f64`) and a pure-Python one (`logprob_bruteforce`) that share no code
with it.

Pinned by (tests/test_oracle_logprob.py): closed forms (uniform row, one spike
over zeros, -inf masked entries, sum of exp(logp) over all targets == 1, shift
invariance), the brute-force evaluation on small vocabularies, and agreement of
the fp32 and fp64 routes.  The reference holds no golden vectors for this path.
"""
from __future__ import annotations

import math

import torch


def logprob_ref(logits: torch.Tensor, token_ids: torch.Tensor, chunk_rows: int = 2048) -> torch.Tensor:
    """fp32 torch CPU path: log_softmax(logits.float(), -1).gather(-1, ids).  Shape logits.shape[:-1]."""
    vocab = logits.shape[-1]
    rows = logits.reshape(-1, vocab)
    ids = token_ids.reshape(-1).to(torch.int64)
    out = torch.empty(rows.shape[0], dtype=torch.float32)
    for s in range(0, rows.shape[0], chunk_rows):
        x = rows[s:s + chunk_rows].to(device="cpu", dtype=torch.float32)
        lp = torch.log_softmax(x, dim=-1)
        out[s:s + chunk_rows] = lp.gather(-1, ids[s:s + chunk_rows].cpu().unsqueeze(-1)).squeeze(-1)
    return out.view(tuple(logits.shape[:-1]))


def logprob_reference_dtype(logits: torch.Tensor, token_ids: torch.Tensor) -> torch.Tensor:
    """The reference exactly as written (sampling.py:108-110): computed and returned in logits.dtype."""
    lp = torch.log_softmax(logits.cpu(), dim=-1)
    return lp.gather(-1, token_ids.cpu().to(torch.int64).unsqueeze(-1)).squeeze(-1)


def logprob_f64(logits: torch.Tensor, token_ids: torch.Tensor, chunk_rows: int = 1024) -> torch.Tensor:
    """fp64 evaluation x_t - (max + log(sum(exp(x - max)))), written out rather than via log_softmax."""
    vocab = logits.shape[-1]
    rows = logits.reshape(-1, vocab)
    ids = token_ids.reshape(-1).to(torch.int64).cpu()
    out = torch.empty(rows.shape[0], dtype=torch.float64)
    for s in range(0, rows.shape[0], chunk_rows):
        x = rows[s:s + chunk_rows].to(device="cpu", dtype=torch.float64)
        m = x.max(dim=-1, keepdim=True).values
        lse = m.squeeze(-1) + torch.log(torch.exp(x - m).sum(dim=-1))
        out[s:s + chunk_rows] = x.gather(-1, ids[s:s + chunk_rows].unsqueeze(-1)).squeeze(-1) - lse
    return out.view(tuple(logits.shape[:-1]))


def entropy_f64(logits: torch.Tensor, chunk_rows: int = 1024) -> torch.Tensor:
    """Entropy -sum p log p of each row's softmax in fp64 (0 * -inf counted as 0)."""
    vocab = logits.shape[-1]
    rows = logits.reshape(-1, vocab)
    out = torch.empty(rows.shape[0], dtype=torch.float64)
    for s in range(0, rows.shape[0], chunk_rows):
        x = rows[s:s + chunk_rows].to(device="cpu", dtype=torch.float64)
        lp = torch.log_softmax(x, dim=-1)
        p = lp.exp()
        out[s:s + chunk_rows] = -(torch.where(p > 0, p * lp, torch.zeros_like(p))).sum(-1)
    return out.view(tuple(logits.shape[:-1]))


def logprob_bruteforce(row, target: int) -> float:
    """Pure-Python evaluation of one row (list of floats) with math.fsum; for tiny vocabularies."""
    m = max(row)
    total = math.fsum(math.exp(v - m) for v in row if v != -math.inf)
    return row[target] - (m + math.log(total))


def lmhead_logprob_ref(hidden: torch.Tensor, weight: torch.Tensor, token_ids: torch.Tensor,
                       dtype=torch.float32, chunk_rows: int = 256) -> torch.Tensor:
    """Oracle of the fused lm_head -> logprob operator: logprob of `hidden @ weight.T` kept in `dtype`
    (fp32 or fp64; the bf16 inputs are exact in both), i.e. compute_logp(lm_head(hidden)) of
    rl_engine/kernels/sampling.py:92-112 with an unrounded linear layer."""
    hdim = hidden.shape[-1]
    rows = hidden.reshape(-1, hdim).cpu()
    ids = token_ids.reshape(-1).to(torch.int64).cpu()
    w = weight.cpu().to(dtype)
    out = torch.empty(rows.shape[0], dtype=dtype)
    for s in range(0, rows.shape[0], chunk_rows):
        logits = torch.nn.functional.linear(rows[s:s + chunk_rows].to(dtype), w)
        m = logits.max(dim=-1, keepdim=True).values
        lse = m.squeeze(-1) + torch.log(torch.exp(logits - m).sum(dim=-1))
        out[s:s + chunk_rows] = logits.gather(-1, ids[s:s + chunk_rows].unsqueeze(-1)).squeeze(-1) - lse
    return out.view(tuple(hidden.shape[:-1]))


def logprob_backward_ref(logits: torch.Tensor, token_ids: torch.Tensor, grad_logp: torch.Tensor,
                         dtype=torch.float32) -> torch.Tensor:
    """Gradient of logprob_ref with respect to the logits, by torch autograd on the CPU (in `dtype`):
    what autograd builds for rl_engine/kernels/sampling.py:108-110 when it is not under inference_mode."""
    x = logits.detach().cpu().to(dtype).clone().requires_grad_(True)
    lp = torch.log_softmax(x, dim=-1).gather(-1, token_ids.cpu().to(torch.int64).unsqueeze(-1)).squeeze(-1)
    lp.backward(grad_logp.detach().cpu().to(dtype))
    return x.grad


def logprob_backward_closed_form(logits: torch.Tensor, token_ids: torch.Tensor, grad_logp: torch.Tensor) -> torch.Tensor:
    """The same gradient written out in fp64: g * (onehot - softmax)."""
    x = logits.detach().cpu().double()
    p = torch.softmax(x, dim=-1)
    onehot = torch.zeros_like(p).scatter_(-1, token_ids.cpu().to(torch.int64).unsqueeze(-1), 1.0)
    return grad_logp.detach().cpu().double().unsqueeze(-1) * (onehot - p)


def lmhead_logprob_backward_ref(hidden: torch.Tensor, weight: torch.Tensor, token_ids: torch.Tensor,
                                grad_logp: torch.Tensor, dtype=torch.float64):
    """(dhidden, dweight) of lmhead_logprob_ref by torch autograd on the CPU in `dtype`: the gradient of
    compute_logp(lm_head(hidden)) (rl_engine/kernels/sampling.py:108-110 behind an nn.Linear)."""
    h = hidden.detach().cpu().to(dtype).clone().requires_grad_(True)
    w = weight.detach().cpu().to(dtype).clone().requires_grad_(True)
    logits = torch.nn.functional.linear(h, w)
    lp = torch.log_softmax(logits, dim=-1).gather(-1, token_ids.cpu().to(torch.int64).unsqueeze(-1)).squeeze(-1)
    lp.backward(grad_logp.detach().cpu().to(dtype))
    return h.grad, w.grad


def lmhead_logprob_backward_closed_form(hidden: torch.Tensor, weight: torch.Tensor, token_ids: torch.Tensor,
                                        grad_logp: torch.Tensor):
    """The same two gradients written out in fp64: D = g * (onehot - softmax(h W^T)); dh = D W; dW = D^T h."""
    h = hidden.detach().cpu().double().reshape(-1, hidden.shape[-1])
    w = weight.detach().cpu().double()
    d = logprob_backward_closed_form(h @ w.t(), token_ids.reshape(-1), grad_logp.reshape(-1))
    return (d @ w).reshape(hidden.shape), d.t() @ h
