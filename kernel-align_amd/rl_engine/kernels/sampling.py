"""SamplerBackend: the logprob and sampling operators on hand-written gfx950 kernels.

Drop-in for the reference's rl_engine/kernels/sampling.py:9-112: a parameter-less
nn.Module with ``compute_logp(logits, token_ids)`` and
``sample(logits, top_k, top_p, temperature, deterministic)``.  Every call goes
to libkernel_align_hip.so on the current HIP stream; nothing runs on the CPU and
nothing falls back to torch ops.
"""
from __future__ import annotations

from contextlib import contextmanager

import torch
import torch.nn as nn

from rl_engine.kernels import _hip
from rl_engine.kernels.pool import PoolExhausted, WorkspacePool
from rl_engine.platforms.constants import constants
from rl_engine.utils.logger import logger

# Rows (tokens) per kernel launch of compute_logp and its backward.  The kernels keep no per-launch state and no
# chunk-sized buffer, so this is launch granularity only: it bounds how long one launch occupies the GPU and never
# changes a result bit.  Every launch ends with a tail in which the device runs empty: at V = 128,256 launches of
# 8192 / 32768 / 131072 rows reach 6.86 / 7.01 / 7.09 TB/s, so the default is a large group (256 x 512 tokens).
DEFAULT_CHUNK_TOKENS = 131072
# Rows per chunk of the fused lm_head backward, which does hold a chunk-sized buffer ([rows, V] bf16: 2.1 GB at
# V = 128,256).
LMHEAD_BACKWARD_CHUNK_TOKENS = 8192

_LOGPROB_FN = {torch.bfloat16: "ka_logprob_bf16", torch.float16: "ka_logprob_f16",
               torch.float32: "ka_logprob_f32"}
_ENTROPY_FN = {torch.bfloat16: "ka_logprob_entropy_bf16", torch.float16: "ka_logprob_entropy_f16",
               torch.float32: "ka_logprob_entropy_f32"}
_BACKWARD_FN = {torch.bfloat16: "ka_logprob_backward_bf16", torch.float16: "ka_logprob_backward_f16",
                torch.float32: "ka_logprob_backward_f32"}
_DTYPE_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}
_SAMPLE_FN = {torch.bfloat16: "ka_sample_topk_topp_bf16", torch.float16: "ka_sample_topk_topp_f16",
              torch.float32: "ka_sample_topk_topp_f32"}


def _require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU: rl_engine has no CPU path (got {t.device})")


class _NoGuard:
    """Stands in for torch.cuda.device(...) when the tensor's device is the current one already."""

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _on_device(device):
    """A context manager that makes `device` current for the launch.  Entering torch.cuda.device() and asking
    torch.cuda.current_stream() cost more host time than a small kernel runs, so the common case (the tensor lives
    on the current device) takes neither."""
    index = device.index
    if index is None or index == torch._C._cuda_getDevice():
        return _NO_GUARD
    return torch.cuda.device(index)


def _raw_stream() -> int:
    """Handle of the current HIP stream of the current device (what torch.cuda.current_stream().cuda_stream returns)."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _chunk_rows(chunk_tokens, default=None) -> int:
    """Rows per launch of a chunked operator; anything below one row would make the launch loop empty."""
    chunk = (DEFAULT_CHUNK_TOKENS if default is None else default) if chunk_tokens is None else int(chunk_tokens)
    if chunk < 1:
        raise ValueError(f"chunk_tokens must be >= 1 (got {chunk_tokens})")
    return chunk


def _rows_view(logits: torch.Tensor) -> torch.Tensor:
    """[.., V] -> [N, V] with unit stride along V and a uniform row stride, copying only if needed."""
    vocab = logits.shape[-1]
    if logits.dim() == 2 and logits.stride(1) == 1 and (logits.shape[0] <= 1 or logits.stride(0) >= vocab):
        return logits
    if logits.is_contiguous():
        return logits.view(-1, vocab)
    logger.warn_once("logits are not row-contiguous: copying them before the kernel launch")
    return logits.contiguous().view(-1, vocab)


class SamplerBackend(nn.Module):
    def __init__(self, pool_bytes: int | None = None):
        super().__init__()
        self.backend = self._detect_backend()
        self._init_backend_assets(pool_bytes)

    def _detect_backend(self) -> str:
        logger.info_once("AMD GPU (ROCm): using the in-tree HIP kernels")
        return constants.BackendLib.HIP_NATIVE.value

    def _init_backend_assets(self, pool_bytes: int | None) -> None:
        # Loading here makes a missing or incomplete library fail at construction.
        self._lib = _hip.load()
        self.pool = WorkspacePool(pool_bytes)
        logger.info_once(f"Loaded {self._lib.ka_version().decode()}")

    @contextmanager
    def _workspace(self, nbytes: int, device):
        """Device pointer of `nbytes` of scratch for launches on the current stream (None for no bytes).  The
        pool orders users of different streams and threads, so one SamplerBackend may be shared by them."""
        if nbytes == 0:
            yield None
            return
        with self.pool.lease(nbytes, device) as view:
            yield view.data_ptr()

    # ------------------------------------------------------------------ logprob
    @torch.inference_mode()
    def compute_logp(self, logits, token_ids, out_dtype=torch.float32, chunk_tokens=None):
        return self._compute_logp(logits, token_ids, out_dtype, chunk_tokens)

    def _compute_logp(self, logits, token_ids, out_dtype=torch.float32, chunk_tokens=None):
        """Per-token log-probabilities ``log_softmax(logits, -1)[..., token_ids]``.

        logits: [G, L, V] (or [N, V]) bf16 / fp16 / fp32 on the GPU; token_ids: integer tensor of
        shape logits.shape[:-1].  Returns fp32 of shape [G, L] (reference:
        sampling.py:92-112 returns logits.dtype; pass ``out_dtype=logits.dtype`` for that).
        The rows are fed to the kernel ``chunk_tokens`` at a time; no chunk-sized buffer exists.
        """
        _require_gpu(logits, "logits")
        if logits.dim() < 2:
            raise ValueError("logits must be [..., V]")
        if tuple(token_ids.shape) != tuple(logits.shape[:-1]):
            raise ValueError(f"token_ids shape {tuple(token_ids.shape)} != logits.shape[:-1] "
                             f"{tuple(logits.shape[:-1])}")
        fn_name = _LOGPROB_FN.get(logits.dtype)
        if fn_name is None:
            raise TypeError(f"unsupported logits dtype {logits.dtype}")
        fn = getattr(self._lib, fn_name)
        rows = _rows_view(logits)
        n_rows, vocab = rows.shape
        ids = token_ids.to(device=logits.device, dtype=torch.int64).contiguous().view(-1)
        out = torch.empty(n_rows, dtype=torch.float32, device=logits.device)
        chunk = _chunk_rows(chunk_tokens)
        row_stride = rows.stride(0) if n_rows > 1 else vocab
        esize = rows.element_size()
        with _on_device(logits.device):
            stream = _raw_stream()
            base, ids_base, out_base = rows.data_ptr(), ids.data_ptr(), out.data_ptr()
            for start in range(0, n_rows, chunk):
                n = min(chunk, n_rows - start)
                status = fn(base + start * row_stride * esize, n, vocab, row_stride,
                            ids_base + start * 8, out_base + start * 4, stream)
                _hip.check(status, fn_name)
        if out_dtype != torch.float32:
            out = out.to(out_dtype)
        return out.view(tuple(logits.shape[:-1]))

    @torch.inference_mode()
    def compute_logp_entropy(self, logits, token_ids, chunk_tokens=None):
        """compute_logp plus the entropy of every row's softmax, from the same single pass (bf16 / fp16 / fp32)."""
        _require_gpu(logits, "logits")
        fn_name = _ENTROPY_FN.get(logits.dtype)
        if fn_name is None:
            raise TypeError(f"unsupported logits dtype {logits.dtype}")
        if logits.dim() < 2:
            raise ValueError("logits must be [..., V]")
        if tuple(token_ids.shape) != tuple(logits.shape[:-1]):
            raise ValueError("token_ids shape must equal logits.shape[:-1]")
        chunk = _chunk_rows(chunk_tokens)
        fn = getattr(self._lib, fn_name)
        rows = _rows_view(logits)
        n_rows, vocab = rows.shape
        ids = token_ids.to(device=logits.device, dtype=torch.int64).contiguous().view(-1)
        out = torch.empty(n_rows, dtype=torch.float32, device=logits.device)
        ent = torch.empty(n_rows, dtype=torch.float32, device=logits.device)
        row_stride = rows.stride(0) if n_rows > 1 else vocab
        esize = rows.element_size()
        with _on_device(logits.device):
            stream = _raw_stream()
            for start in range(0, n_rows, chunk):
                n = min(chunk, n_rows - start)
                status = fn(rows.data_ptr() + start * row_stride * esize, n, vocab, row_stride,
                            ids.data_ptr() + start * 8, out.data_ptr() + start * 4, ent.data_ptr() + start * 4, stream)
                _hip.check(status, fn_name)
        shape = tuple(logits.shape[:-1])
        return out.view(shape), ent.view(shape)

    @torch.inference_mode()
    def compute_logp_backward(self, logits, token_ids, logp, grad_logp, inplace=False, chunk_tokens=None):
        return self._compute_logp_backward(logits, token_ids, logp, grad_logp, inplace, chunk_tokens)

    def _compute_logp_backward(self, logits, token_ids, logp, grad_logp, inplace=False, chunk_tokens=None):
        """Gradient of ``compute_logp`` with respect to the logits, in the logits' dtype.

        ``dlogits[..., v] = grad_logp[...] * ((v == token_id) - softmax(logits)[..., v])``.  ``logp`` is the
        fp32 result of ``compute_logp(logits, token_ids)``; the kernel recovers each row's log-sum-exp from
        it and touches every logit once.  With ``inplace=True`` the gradient overwrites ``logits`` (which
        must be row-contiguous) and no second [G, L, V] tensor is allocated.
        """
        _require_gpu(logits, "logits")
        fn_name = _BACKWARD_FN.get(logits.dtype)
        if fn_name is None:
            raise TypeError(f"unsupported logits dtype {logits.dtype}")
        lead = tuple(logits.shape[:-1])
        if tuple(token_ids.shape) != lead or tuple(logp.shape) != lead or tuple(grad_logp.shape) != lead:
            raise ValueError("token_ids, logp and grad_logp must have shape logits.shape[:-1]")
        rows = _rows_view(logits)
        n_rows, vocab = rows.shape
        if inplace and rows.data_ptr() != logits.data_ptr():
            raise ValueError("inplace=True needs row-contiguous logits")
        ids = token_ids.to(device=logits.device, dtype=torch.int64).contiguous().view(-1)
        lp = logp.to(device=logits.device, dtype=torch.float32).contiguous().view(-1)
        g = grad_logp.to(device=logits.device, dtype=torch.float32).contiguous().view(-1)
        out_rows = rows if inplace else torch.empty((n_rows, vocab), dtype=logits.dtype, device=logits.device)
        row_stride = rows.stride(0) if n_rows > 1 else vocab
        out_stride = out_rows.stride(0) if n_rows > 1 else vocab
        esize = rows.element_size()
        chunk = _chunk_rows(chunk_tokens)
        fn = getattr(self._lib, fn_name)
        with _on_device(logits.device):
            stream = _raw_stream()
            for start in range(0, n_rows, chunk):
                n = min(chunk, n_rows - start)
                status = fn(rows.data_ptr() + start * row_stride * esize, n, vocab, row_stride,
                            ids.data_ptr() + start * 8, lp.data_ptr() + start * 4, g.data_ptr() + start * 4,
                            out_rows.data_ptr() + start * out_stride * esize, out_stride, stream)
                _hip.check(status, fn_name)
        return logits if inplace else out_rows.view(logits.shape)

    @torch.inference_mode()
    def grpo_token_loss(self, logp_new, advantages, logp_old=None, logp_ref=None, clip_low=0.2, clip_high=0.2,
                        beta=0.0):
        """Per-token GRPO terms from log-probabilities: ``(loss, kl, dloss_dlogp)``, each fp32 of logp_new's shape.

        ``ratio = exp(logp_new - logp_old)`` (1 when ``logp_old`` is None), clipped surrogate with
        ``advantages`` (same shape, or [G] / [G, 1] for one advantage per sequence of a [G, L] batch), k3 KL
        estimate to ``logp_ref`` weighted by ``beta``.  ``dloss_dlogp`` is what ``compute_logp_backward`` takes
        as ``grad_logp``.
        """
        _require_gpu(logp_new, "logp_new")
        shape = tuple(logp_new.shape)

        def flat(t, name):
            if t is None:
                return None
            if tuple(t.shape) != shape:
                raise ValueError(f"{name} shape {tuple(t.shape)} != logp_new shape {shape}")
            return t.to(device=logp_new.device, dtype=torch.float32).contiguous().view(-1)

        adv = advantages
        if adv.dim() >= 1 and adv.dim() <= len(shape) and tuple(adv.shape) != shape:
            if adv.dim() == 1 and len(shape) == 2 and adv.shape[0] == shape[0]:
                adv = adv.unsqueeze(-1)
            try:
                adv = adv.expand(shape)
            except RuntimeError:
                raise ValueError(f"advantages shape {tuple(advantages.shape)} does not broadcast to {shape}") from None
        new, old, ref, adv = flat(logp_new, "logp_new"), flat(logp_old, "logp_old"), flat(logp_ref, "logp_ref"), \
            flat(adv, "advantages")
        n = new.numel()
        loss = torch.empty(n, dtype=torch.float32, device=new.device)
        kl = torch.empty_like(loss)
        dlogp = torch.empty_like(loss)
        with _on_device(new.device):
            status = self._lib.ka_grpo_token_terms(
                new.data_ptr(), old.data_ptr() if old is not None else None,
                ref.data_ptr() if ref is not None else None, adv.data_ptr(), n, float(clip_low), float(clip_high),
                float(beta), loss.data_ptr(), kl.data_ptr(), dlogp.data_ptr(),
                _raw_stream())
        _hip.check(status, "ka_grpo_token_terms")
        return loss.view(shape), kl.view(shape), dlogp.view(shape)

    # ----------------------------------------------------------------- sampling
    @torch.inference_mode()
    def sample(self, logits, top_k=None, top_p=None, temperature=1.0, deterministic=True,
               uniforms=None, generator=None, return_logprob=False, route_flags=0, return_policy_logprob=False):
        """Draw one token id per row after temperature -> top-k -> top-p filtering.

        logits: [B, V] bf16 / fp16 / fp32 on the GPU.  Returns int64 [B] (reference:
        sampling.py:39-88; filter semantics of benchmarks/benchmark_sampling.py:12-37).
        ``uniforms`` ([B] fp32 in [0, 1)) drives the draw; if None they come from
        ``torch.rand(B, generator=generator)`` on the logits' device.  The kernels are always
        deterministic, so ``deterministic`` is accepted and ignored.

        ``top_k``, ``top_p`` and ``temperature`` may each be a [B] tensor of per-row values (a row value
        that is not valid switches that filter off for the row).  With ``return_logprob=True`` the result
        is ``(ids, logprob)`` where logprob (fp32 [B]) is the log-probability of the drawn token under the
        filtered, renormalised distribution it was drawn from.  ``route_flags`` (``_hip.SAMPLE_FLAG_*``) makes the
        library take one of its slower routes for the same function; results do not depend on it.
        With ``return_policy_logprob=True`` the last element of the result is the drawn token's log-probability
        under the unfiltered softmax of the raw logits - ``compute_logp(logits, ids)`` to 1e-5, what a GRPO ratio is
        built from - computed by the sampling kernel itself (with ``top_k <= 256`` while the row streams by), so that
        a decode step needs neither a second operator call nor a second kernel.
        """
        _require_gpu(logits, "logits")
        if logits.dim() != 2:
            raise ValueError("logits must be [B, V]")
        if logits.dtype not in _SAMPLE_FN:
            raise TypeError(f"unsupported logits dtype {logits.dtype}")
        batch, vocab = logits.shape
        dev = logits.device

        def rows_or_scalar(value, name, dtype, default, check):
            if isinstance(value, torch.Tensor):
                if tuple(value.shape) != (batch,):
                    raise ValueError(f"{name} tensor must have shape ({batch},)")
                return default, value.to(device=dev, dtype=dtype).contiguous()
            scalar = default if value is None else value
            check(scalar)
            return scalar, None

        def check_k(v):
            if top_k is not None and int(v) < 1:
                raise ValueError(f"top_k must be >= 1 (got {top_k})")

        def check_p(v):
            if not 0.0 < float(v) <= 1.0:
                raise ValueError(f"top_p must be in (0, 1] (got {top_p})")

        def check_t(v):
            if not float(v) > 0.0:
                raise ValueError(f"temperature must be > 0 (got {temperature})")

        k, k_rows = rows_or_scalar(top_k, "top_k", torch.int32, 0, check_k)
        p, p_rows = rows_or_scalar(top_p, "top_p", torch.float32, 1.0, check_p)
        t, t_rows = rows_or_scalar(temperature, "temperature", torch.float32, 1.0, check_t)
        k, p, t = int(k), float(p), float(t)
        rows = _rows_view(logits)
        if uniforms is None:
            uniforms = torch.rand(batch, generator=generator, device=dev, dtype=torch.float32)
        else:
            if tuple(uniforms.shape) != (batch,):
                raise ValueError(f"uniforms must have shape ({batch},)")
            uniforms = uniforms.to(device=dev, dtype=torch.float32).contiguous()
        out = torch.empty(batch, dtype=torch.int64, device=dev)
        logprob = torch.empty(batch, dtype=torch.float32, device=dev) if return_logprob else None
        if batch == 0:
            empty = torch.empty(0, dtype=torch.float32, device=dev)
            if return_policy_logprob:
                return (out, logprob, empty) if return_logprob else (out, empty)
            return (out, logprob) if return_logprob else out
        ws_bytes = self._lib.ka_sample_workspace_bytes(batch, vocab)
        row_stride = rows.stride(0) if batch > 1 else vocab
        extended = (return_logprob or return_policy_logprob or k_rows is not None or p_rows is not None
                    or t_rows is not None or route_flags)
        policy = torch.empty(batch, dtype=torch.float32, device=dev) if return_policy_logprob else None
        def launch(ws_ptr):
            stream = _raw_stream()
            if extended:
                ptr = lambda x: None if x is None else x.data_ptr()  # noqa: E731
                return "ka_sample_ex", self._lib.ka_sample_ex(
                    _DTYPE_CODE[logits.dtype], rows.data_ptr(), batch, vocab, row_stride, t, ptr(t_rows), k,
                    ptr(k_rows), p, ptr(p_rows), uniforms.data_ptr(), out.data_ptr(), ptr(logprob), ptr(policy),
                    int(route_flags), ws_ptr, ws_bytes, stream)
            name = _SAMPLE_FN[logits.dtype]
            return name, getattr(self._lib, name)(
                rows.data_ptr(), batch, vocab, row_stride, t, k, p, uniforms.data_ptr(),
                out.data_ptr(), ws_ptr, ws_bytes, stream)

        with _on_device(dev):
            if ws_bytes == 0:  # the kernels keep their state in LDS and registers: no lease, no event
                fn_name, status = launch(None)
            else:
                with self._workspace(ws_bytes, dev) as ws_ptr:
                    fn_name, status = launch(ws_ptr)
        _hip.check(status, fn_name)
        if return_policy_logprob:
            return (out, logprob, policy) if return_logprob else (out, policy)
        return (out, logprob) if return_logprob else out

    # ---------------------------------------------------------------- fused GEMM
    @torch.inference_mode()
    def fused_linear_logp(self, hidden, weight, token_ids, return_entropy=False, return_lse=False):
        return self._fused_linear_logp(hidden, weight, token_ids, return_entropy, return_lse)

    def _fused_linear_logp(self, hidden, weight, token_ids, return_entropy=False, return_lse=False):
        """``compute_logp(hidden @ weight.T, token_ids)`` without materialising the logits.

        hidden: bf16 [..., H]; weight: bf16 [V, H] (nn.Linear.weight layout); token_ids: integer
        tensor of shape hidden.shape[:-1].  Returns fp32 of that shape; with ``return_entropy=True`` a pair
        ``(logp, entropy)`` where entropy is that of each row's softmax over the vocabulary, from the same pass;
        with ``return_lse=True`` a pair ``(logp, lse)`` where lse is each row's log-sum-exp over the vocabulary, which
        ``fused_linear_logp_backward`` takes (one or the other: the two options exclude each other).
        """
        if return_entropy and return_lse:
            raise ValueError("return_entropy and return_lse exclude each other")
        _require_gpu(hidden, "hidden")
        _require_gpu(weight, "weight")
        if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
            raise TypeError("fused_linear_logp takes bf16 hidden and weight")
        if weight.dim() != 2 or hidden.shape[-1] != weight.shape[1]:
            raise ValueError("weight must be [V, H] with H == hidden.shape[-1]")
        if tuple(token_ids.shape) != tuple(hidden.shape[:-1]):
            raise ValueError("token_ids shape must equal hidden.shape[:-1]")
        hdim = hidden.shape[-1]
        vocab = weight.shape[0]
        h2 = hidden.contiguous().view(-1, hdim)
        w2 = weight.contiguous()
        n_rows = h2.shape[0]
        ids = token_ids.to(device=hidden.device, dtype=torch.int64).contiguous().view(-1)
        out = torch.empty(n_rows, dtype=torch.float32, device=hidden.device)
        ent = torch.empty(n_rows, dtype=torch.float32, device=hidden.device) if (return_entropy or return_lse) else None
        lead = tuple(hidden.shape[:-1])
        if n_rows == 0:
            return (out.view(lead), ent.view(lead)) if ent is not None else out.view(lead)
        rows_per_call = self._lmhead_rows_per_call(n_rows, hdim, vocab)
        with _on_device(hidden.device):
            stream = _raw_stream()
            for start in range(0, n_rows, rows_per_call):
                n = min(rows_per_call, n_rows - start)
                ws_bytes = self._lib.ka_lmhead_workspace_bytes(n, hdim, vocab)
                with self._workspace(ws_bytes, hidden.device) as ws_ptr:
                    if ent is not None:
                        fn = self._lib.ka_lmhead_logprob_entropy_bf16 if return_entropy else self._lib.ka_lmhead_logprob_lse_bf16
                        status = fn(
                            h2.data_ptr() + start * hdim * 2, w2.data_ptr(), ids.data_ptr() + start * 8,
                            out.data_ptr() + start * 4, ent.data_ptr() + start * 4, n, hdim, vocab, ws_ptr, ws_bytes,
                            stream)
                    else:
                        status = self._lib.ka_lmhead_logprob_bf16(
                            h2.data_ptr() + start * hdim * 2, w2.data_ptr(), ids.data_ptr() + start * 8,
                            out.data_ptr() + start * 4, n, hdim, vocab, ws_ptr, ws_bytes, stream)
                _hip.check(status, "ka_lmhead_logprob_bf16")
        return (out.view(lead), ent.view(lead)) if ent is not None else out.view(lead)

    def _lmhead_rows_per_call(self, n_rows: int, hdim: int, vocab: int) -> int:
        """Rows of one kernel call such that its partials fit the pool: all of them, or the largest multiple of the
        256-token tile that fits (slicing the rows changes no row's result).  The workspace holds 16 B per row and
        vocabulary split - four times that for calls of so few rows that the kernel spreads every split over four
        workgroups - so the size is asked for, not computed here."""
        need = self._lib.ka_lmhead_workspace_bytes
        if need(n_rows, hdim, vocab) <= self.pool.capacity:
            return n_rows
        rows = self.pool.capacity // max(need(1 << 20, hdim, vocab) >> 20, 1) // 256 * 256
        while rows >= 256 and need(rows, hdim, vocab) > self.pool.capacity:
            rows -= 256
        if rows < 256:
            raise PoolExhausted(f"the {self.pool.capacity} B pool cannot hold the lm_head partials of one "
                                f"256-token tile ({need(256, hdim, vocab)} B)")
        return rows

    @torch.inference_mode()
    def fused_linear_logp_backward(self, hidden, weight, token_ids, grad_logp, chunk_tokens=None,
                                   dweight_dtype=torch.float32, lse=None):
        return self._fused_linear_logp_backward(hidden, weight, token_ids, grad_logp, chunk_tokens, dweight_dtype, lse)

    def _fused_linear_logp_backward(self, hidden, weight, token_ids, grad_logp, chunk_tokens=None,
                                    dweight_dtype=torch.float32, lse=None):
        """Gradients of ``fused_linear_logp`` with respect to hidden and weight, one token chunk at a time.

        Per chunk of ``chunk_tokens`` rows: the chunk's logits are rebuilt with the library bf16 GEMM, turned into
        their gradient in place by the logprob forward + backward kernels, and contracted with weight
        (``dhidden``) and with the chunk's hidden rows (``dweight``, accumulated over chunks in
        ``dweight_dtype``).  Only one chunk of logits ([chunk_tokens, V] bf16) exists at any time.
        With ``lse`` (fp32 of shape hidden.shape[:-1], from ``fused_linear_logp(..., return_lse=True)``) the chunk's
        gradient matrix comes from one kernel instead (``ka_lmhead_dlogits_bf16``: the forward's MFMA kernel with the
        softmax-gradient as its epilogue, on fp32 logits that are never stored or rounded).  Measured at
        [8192, 4096] x [128256, 4096] that kernel takes 7.6 ms against 6.9 ms for the GEMM and the two logprob kernels
        (its 8-byte stores of a 2.1 GB matrix are not overlapped with MFMAs), so it is an option, not the default.
        Returns ``(dhidden [..., H] bf16, dweight [V, H] dweight_dtype)``.
        """
        _require_gpu(hidden, "hidden")
        _require_gpu(weight, "weight")
        if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
            raise TypeError("fused_linear_logp_backward takes bf16 hidden and weight")
        if weight.dim() != 2 or hidden.shape[-1] != weight.shape[1]:
            raise ValueError("weight must be [V, H] with H == hidden.shape[-1]")
        lead = tuple(hidden.shape[:-1])
        if tuple(token_ids.shape) != lead or tuple(grad_logp.shape) != lead:
            raise ValueError("token_ids and grad_logp must have shape hidden.shape[:-1]")
        hdim = hidden.shape[-1]
        h2 = hidden.contiguous().view(-1, hdim)
        w2 = weight.contiguous()
        n_rows = h2.shape[0]
        ids = token_ids.to(device=hidden.device, dtype=torch.int64).contiguous().view(-1)
        g = grad_logp.to(device=hidden.device, dtype=torch.float32).contiguous().view(-1)
        if lse is not None:
            if tuple(lse.shape) != lead:
                raise ValueError("lse must have shape hidden.shape[:-1]")
            _require_gpu(lse, "lse")
            lse = lse.to(dtype=torch.float32).contiguous().view(-1)
            if w2.shape[0] % 4 != 0:  # the kernel writes four entries of a row per store: such a vocabulary keeps the GEMM path
                lse = None
        chunk = _chunk_rows(chunk_tokens, LMHEAD_BACKWARD_CHUNK_TOKENS)
        if dweight_dtype not in (torch.float32, torch.bfloat16):
            raise TypeError("dweight_dtype must be torch.float32 or torch.bfloat16")
        dhidden = torch.empty_like(h2)
        if n_rows == 0:
            return dhidden.view(hidden.shape), torch.zeros(w2.shape, dtype=dweight_dtype, device=weight.device)
        dweight = torch.empty(w2.shape, dtype=dweight_dtype, device=weight.device)
        # bf16 x bf16 GEMMs that write (first chunk) or accumulate into (later chunks) the dweight buffer directly:
        # no bf16 rounding of a chunk's contribution and no separate add pass over the [V, H] buffer.
        wide = {"out_dtype": torch.float32} if dweight_dtype == torch.float32 else {}
        for start in range(0, n_rows, chunk):
            stop = min(start + chunk, n_rows)
            if lse is not None:
                logits = torch.empty(stop - start, w2.shape[0], dtype=torch.bfloat16, device=hidden.device)
                with _on_device(hidden.device):
                    _hip.check(self._lib.ka_lmhead_dlogits_bf16(
                        h2.data_ptr() + start * hdim * 2, w2.data_ptr(), ids.data_ptr() + start * 8,
                        lse.data_ptr() + start * 4, g.data_ptr() + start * 4, logits.data_ptr(), w2.shape[0],
                        stop - start, hdim, w2.shape[0], _raw_stream()), "ka_lmhead_dlogits_bf16")
            else:
                logits = torch.matmul(h2[start:stop], w2.t())                   # [n, V] bf16, fp32 accumulation
                logp = self._compute_logp(logits, ids[start:stop])
                self._compute_logp_backward(logits, ids[start:stop], logp, g[start:stop], inplace=True)
            torch.matmul(logits, w2, out=dhidden[start:stop])                   # logits now holds dlogits
            if start == 0:
                torch.mm(logits.t(), h2[start:stop], out=dweight, **wide)
            else:
                torch.addmm(dweight, logits.t(), h2[start:stop], out=dweight, **wide)
            del logits
        return dhidden.view(hidden.shape), dweight
