"""ctypes binding of oracle/ka_oracle.c (the exactly specified sampling oracle).  Test infrastructure only."""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_int32, c_int64, c_uint64, c_void_p
from pathlib import Path

import torch

from oracle import build as _build

_DTYPES = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}


class RowInfo(ctypes.Structure):
    _fields_ = [("n_topk", c_int64), ("n_kept", c_int64), ("z_topk", c_uint64), ("z_kept", c_uint64),
                ("kth_value", c_float), ("max_value", c_float), ("w_pick", c_uint64)]


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        path = Path(_build.LIB)
        if not path.exists():
            _build.build_oracle()
        handle = ctypes.CDLL(str(path))
        handle.ka_oracle_weight.restype = c_uint64
        handle.ka_oracle_weight.argtypes = [c_float]
        handle.ka_oracle_weight_libm.restype = c_uint64
        handle.ka_oracle_weight_libm.argtypes = [c_float]
        handle.ka_oracle_floor_scale.restype = c_uint64
        handle.ka_oracle_floor_scale.argtypes = [c_float, c_uint64]
        handle.ka_oracle_scale.restype = None
        handle.ka_oracle_scale.argtypes = [c_void_p, c_int, c_int64, c_float, c_void_p]
        handle.ka_oracle_sample.restype = c_int
        handle.ka_oracle_sample.argtypes = [c_void_p, c_int, c_int64, c_int64, c_int64, c_float, c_int32, c_float,
                                            c_void_p, c_void_p, c_void_p]
        _lib = handle
    return _lib


def weight(d: float) -> int:
    """W(d) = trunc(2^40 * exp(d)) as the oracle evaluates it."""
    return int(lib().ka_oracle_weight(d))


def weight_libm(d: float) -> int:
    """The same function built on libm's fma() instead of the hardware instruction."""
    return int(lib().ka_oracle_weight_libm(d))


def floor_scale(s: float, z: int) -> int:
    return int(lib().ka_oracle_floor_scale(s, z))


def scale(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """Temperature step alone: fp32 values of (logits / T rounded to logits.dtype), -0 folded to +0."""
    src = logits.detach().cpu().contiguous()
    dst = torch.empty(src.numel(), dtype=torch.float32)
    lib().ka_oracle_scale(src.data_ptr(), _DTYPES[src.dtype], src.numel(), temperature, dst.data_ptr())
    return dst.view(src.shape)


def sample(logits: torch.Tensor, temperature: float = 1.0, top_k=None, top_p=None, uniforms=None,
           return_info: bool = False):
    """Token ids (int64 [B]) for logits [B, V]; top_k None/0 and top_p None/1 switch a filter off."""
    src = logits.detach().cpu().contiguous()
    assert src.dim() == 2
    batch, vocab = src.shape
    u = uniforms.detach().cpu().to(torch.float32).contiguous()
    assert u.shape == (batch,)
    out = torch.empty(batch, dtype=torch.int64)
    info = (RowInfo * batch)()
    rc = lib().ka_oracle_sample(src.data_ptr(), _DTYPES[src.dtype], batch, vocab, vocab, float(temperature),
                                int(top_k or 0), float(1.0 if top_p is None else top_p), u.data_ptr(),
                                out.data_ptr(), ctypes.cast(info, c_void_p))
    if rc != 0:
        raise ValueError(f"ka_oracle_sample rejected its arguments (rc={rc})")
    if return_info:
        return out, [dict(n_topk=i.n_topk, n_kept=i.n_kept, z_topk=i.z_topk, z_kept=i.z_kept,
                          kth_value=i.kth_value, max_value=i.max_value, w_pick=i.w_pick) for i in info]
    return out


def sample_rows(logits: torch.Tensor, temperature, top_k, top_p, uniforms):
    """Per-row parameters: each of temperature / top_k / top_p is a scalar, None, or a length-B sequence.
    A row's invalid value switches that filter off (T <= 0 or NaN -> 1, top_k < 0 -> off, top_p outside
    (0, 1] -> off), as the kernel does.  Returns (ids int64 [B], logprob float64 [B]) where logprob is the
    log of the sampled entry's probability under the filtered, renormalised distribution."""
    import math

    batch = logits.shape[0]

    def per_row(v, default):
        if v is None:
            return [default] * batch
        if isinstance(v, torch.Tensor):
            v = v.detach().cpu().tolist()
        if isinstance(v, (list, tuple)):
            assert len(v) == batch
            return list(v)
        return [v] * batch

    ts, ks, ps = per_row(temperature, 1.0), per_row(top_k, 0), per_row(top_p, 1.0)
    ids = torch.empty(batch, dtype=torch.int64)
    lps = torch.empty(batch, dtype=torch.float64)
    for r in range(batch):
        t = float(torch.tensor(ts[r], dtype=torch.float32))
        t = t if t > 0.0 else 1.0
        k = int(ks[r]) if ks[r] is not None and int(ks[r]) > 0 else 0
        p = float(torch.tensor(1.0 if ps[r] is None else ps[r], dtype=torch.float32))
        p = p if 0.0 < p <= 1.0 else 1.0
        out, info = sample(logits[r:r + 1], t, k, p, uniforms[r:r + 1], return_info=True)
        ids[r] = out[0]
        lps[r] = math.log(info[0]["w_pick"]) - math.log(info[0]["z_kept"])
    return ids, lps
