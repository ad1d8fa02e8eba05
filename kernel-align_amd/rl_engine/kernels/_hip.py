"""ctypes binding of libkernel_align_hip.so (see include/kernel_align_hip.h).

There is no fallback: if the library is missing, or lacks a symbol, loading
raises and every operator that needs it fails with that error.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_uint32, c_void_p
from pathlib import Path

KA_OK = 0
KA_ERR_BAD_ARG = -1
KA_ERR_UNSUPPORTED = -2
KA_ERR_WORKSPACE = -3
KA_ERR_HIP = -4

# Revision of include/kernel_align_hip.h that the signatures below were written against (KA_ABI_REVISION).
ABI_REVISION = 4

LIB_NAME = "libkernel_align_hip.so"
ENV_LIB = "KERNEL_ALIGN_HIP_LIB"

_LOGPROB_ARGS = [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p]
_ENTROPY_ARGS = [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]
_BACKWARD_ARGS = [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]
_SAMPLE_ARGS = [c_void_p, c_int64, c_int64, c_int64, c_float, c_int32, c_float, c_void_p, c_void_p,
                c_void_p, c_size_t, c_void_p]

# name -> (restype, argtypes); must list every symbol the header declares.
SIGNATURES = {
    "ka_version": (c_char_p, []),
    "ka_abi_revision": (c_int, []),
    "ka_last_error": (c_char_p, []),
    "ka_status_string": (c_char_p, [c_int]),
    "ka_logprob_bf16": (c_int, _LOGPROB_ARGS),
    "ka_logprob_f16": (c_int, _LOGPROB_ARGS),
    "ka_logprob_f32": (c_int, _LOGPROB_ARGS),
    "ka_logprob_entropy_bf16": (c_int, _ENTROPY_ARGS),
    "ka_logprob_entropy_f16": (c_int, _ENTROPY_ARGS),
    "ka_logprob_entropy_f32": (c_int, _ENTROPY_ARGS),
    "ka_logprob_backward_bf16": (c_int, _BACKWARD_ARGS),
    "ka_logprob_backward_f16": (c_int, _BACKWARD_ARGS),
    "ka_logprob_backward_f32": (c_int, _BACKWARD_ARGS),
    "ka_grpo_token_terms": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_float, c_float, c_float,
                                    c_void_p, c_void_p, c_void_p, c_void_p]),
    "ka_sample_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "ka_sample_topk_topp_bf16": (c_int, _SAMPLE_ARGS),
    "ka_sample_topk_topp_f16": (c_int, _SAMPLE_ARGS),
    "ka_sample_topk_topp_f32": (c_int, _SAMPLE_ARGS),
    "ka_sample_ex": (c_int, [c_int, c_void_p, c_int64, c_int64, c_int64, c_float, c_void_p, c_int32, c_void_p, c_float,
                             c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_void_p, c_size_t, c_void_p]),
    "ka_sample_mass_fixed": (c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
    "ka_lmhead_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "ka_lmhead_logprob_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                       c_void_p, c_size_t, c_void_p]),
    "ka_lmhead_logprob_lse_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                           c_int64, c_void_p, c_size_t, c_void_p]),
    "ka_lmhead_dlogits_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                       c_int64, c_int64, c_void_p]),
    "ka_lmhead_logprob_entropy_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                               c_int64, c_void_p, c_size_t, c_void_p]),
    "ka_lmhead_logprob_bf16_noalloc": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                               c_void_p]),
}

# Route selection flags of ka_sample_ex (verification only; results do not depend on them).
SAMPLE_FLAG_GENERAL_PATH = 1
SAMPLE_FLAG_BLOCK_WIDE_TOPK = 2
SAMPLE_FLAG_TWO_ROWS_PER_CU = 4
SAMPLE_FLAG_ONE_ROW_PER_CU = 8

# Size of the static device array behind ka_lmhead_logprob_bf16_noalloc (KA_LMHEAD_STATIC_SCRATCH_BYTES).
LMHEAD_STATIC_SCRATCH_BYTES = 16 << 20


class HipLibraryError(RuntimeError):
    """The HIP library is missing, incomplete, or one of its calls failed."""


def library_path() -> Path:
    override = os.environ.get(ENV_LIB)
    if override:
        return Path(override)
    return Path(__file__).resolve().parents[2] / "lib" / LIB_NAME


_lib = None


def load() -> ctypes.CDLL:
    """Load the library once and bind every entry point; raise HipLibraryError otherwise."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not path.exists():
        raise HipLibraryError(
            f"{path} not found: build it with `python kernel-align_amd/build_hip.py` "
            f"(or point {ENV_LIB} at it); rl_engine has no non-HIP path"
        )
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as exc:
        raise HipLibraryError(f"cannot load {path}: {exc}") from exc
    for name, (restype, argtypes) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise HipLibraryError(f"{path} does not export {name}") from exc
        fn.restype = restype
        fn.argtypes = argtypes
    found = lib.ka_abi_revision()
    if found != ABI_REVISION:
        raise HipLibraryError(f"{path} implements interface revision {found}, this binding was written against "
                              f"revision {ABI_REVISION}: rebuild the library (python kernel-align_amd/build_hip.py)")
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    """Turn a KA_ERR_* status into the Python exception the op API documents."""
    if status == KA_OK:
        return
    lib = load()
    msg = lib.ka_last_error().decode("utf-8", "replace")
    name = lib.ka_status_string(status).decode()
    text = f"{what}: {name}: {msg}"
    if status in (KA_ERR_BAD_ARG, KA_ERR_UNSUPPORTED, KA_ERR_WORKSPACE):
        raise ValueError(text)
    raise HipLibraryError(text)
