"""The C-ABI library loads without a GPU, exports every symbol the header declares, and rejects bad
arguments with the documented status codes.  No kernel is launched here."""
import ctypes
import re
from pathlib import Path

import pytest

from rl_engine.kernels import _hip

REPO = Path(__file__).resolve().parents[1]
HEADER = REPO / "include" / "kernel_align_hip.h"


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(ka_[a-z0-9_]+)\s*\(", text)))


def test_header_binding_and_library_agree():
    names = declared_symbols()
    assert len(names) >= 13
    assert sorted(_hip.SIGNATURES) == names, "ctypes binding and header list different entry points"
    lib = _hip.load()
    for name in names:
        assert getattr(lib, name) is not None


def test_interface_revision_is_checked(monkeypatch):
    """The header, the binding and the library carry the same interface revision, and a binding written against
    another revision refuses the library instead of calling it with arguments in the wrong places."""
    lib = _hip.load()
    header_rev = int(re.search(r"#define KA_ABI_REVISION (\d+)", HEADER.read_text()).group(1))
    assert lib.ka_abi_revision() == header_rev == _hip.ABI_REVISION
    monkeypatch.setattr(_hip, "_lib", None)
    monkeypatch.setattr(_hip, "ABI_REVISION", header_rev + 1)
    with pytest.raises(_hip.HipLibraryError, match="interface revision"):
        _hip.load()
    monkeypatch.setattr(_hip, "ABI_REVISION", header_rev)
    assert _hip.load().ka_abi_revision() == header_rev


def test_version_and_status_strings():
    lib = _hip.load()
    assert b"gfx950" in lib.ka_version()
    assert lib.ka_status_string(0) == b"KA_OK"
    assert lib.ka_status_string(-1) == b"KA_ERR_BAD_ARG"
    assert lib.ka_status_string(-3) == b"KA_ERR_WORKSPACE"
    assert lib.ka_status_string(-99) == b"KA_ERR_UNKNOWN"


def test_logprob_argument_checks():
    lib = _hip.load()
    p = ctypes.c_void_p(4096)
    assert lib.ka_logprob_bf16(None, 0, 128, 128, None, None, None) == _hip.KA_OK          # empty batch
    assert lib.ka_logprob_bf16(None, 4, 128, 128, p, p, None) == _hip.KA_ERR_BAD_ARG
    assert b"null" in lib.ka_last_error()
    assert lib.ka_logprob_bf16(p, -1, 128, 128, p, p, None) == _hip.KA_ERR_BAD_ARG
    assert lib.ka_logprob_f32(p, 4, 0, 128, p, p, None) == _hip.KA_ERR_BAD_ARG
    assert lib.ka_logprob_f16(p, 4, 128, 64, p, p, None) == _hip.KA_ERR_BAD_ARG              # stride < vocab
    assert lib.ka_logprob_bf16(p, 4, 1 << 31, 1 << 31, p, p, None) == _hip.KA_ERR_UNSUPPORTED
    with pytest.raises(ValueError, match="KA_ERR_BAD_ARG"):
        _hip.check(lib.ka_logprob_bf16(p, 4, 128, 64, p, p, None), "ka_logprob_bf16")


def test_sampling_argument_checks():
    lib = _hip.load()
    p = ctypes.c_void_p(4096)
    call = lib.ka_sample_topk_topp_bf16
    assert call(None, 0, 128, 128, 1.0, 0, 1.0, None, None, None, 0, None) == _hip.KA_OK
    assert call(None, 2, 128, 128, 1.0, 0, 1.0, p, p, None, 0, None) == _hip.KA_ERR_BAD_ARG
    assert call(p, 2, 128, 128, 0.0, 0, 1.0, p, p, None, 0, None) == _hip.KA_ERR_BAD_ARG    # temperature
    assert call(p, 2, 128, 128, 1.0, -1, 1.0, p, p, None, 0, None) == _hip.KA_ERR_BAD_ARG   # top_k
    assert call(p, 2, 128, 128, 1.0, 5, 0.0, p, p, None, 0, None) == _hip.KA_ERR_BAD_ARG    # top_p
    assert call(p, 2, 128, 128, 1.0, 5, 1.5, p, p, None, 0, None) == _hip.KA_ERR_BAD_ARG
    assert call(p, 2, 1 << 22, 1 << 22, 1.0, 5, 0.9, p, p, None, 0, None) == _hip.KA_ERR_UNSUPPORTED
    assert lib.ka_sample_workspace_bytes(256, 128256) >= 0
    ex = lib.ka_sample_ex
    assert ex(0, None, 0, 128, 128, 1.0, None, 0, None, 1.0, None, None, None, None, None, 0, None, 0, None) == _hip.KA_OK
    assert ex(7, p, 2, 128, 128, 1.0, None, 0, None, 1.0, None, p, p, None, None, 0, None, 0, None) == _hip.KA_ERR_BAD_ARG   # dtype code
    assert ex(0, p, 2, 128, 128, 0.0, None, 0, None, 1.0, None, p, p, None, None, 0, None, 0, None) == _hip.KA_ERR_BAD_ARG   # scalar T
    assert ex(0, p, 2, 128, 128, 1.0, None, 0, None, 1.0, None, p, p, None, None, 16, None, 0, None) == _hip.KA_ERR_BAD_ARG   # flag bits
    assert ex(0, p, 2, 128, 128, 1.0, None, 0, None, 1.0, None, p, p, None, None, 12, None, 0, None) == _hip.KA_ERR_BAD_ARG   # both workgroup sizes
    assert b"flag" in lib.ka_last_error()
    # a per-row array replaces its scalar, which is then not checked: the call gets past the scalar checks and
    # is stopped by the next host check (stride < vocab), so nothing is ever launched on these made-up pointers
    assert ex(0, p, 2, 128, 64, 0.0, p, -1, p, 9.0, p, p, p, None, None, 0, None, 0, None) == _hip.KA_ERR_BAD_ARG
    assert b"stride" in lib.ka_last_error()


def test_lmhead_argument_checks_and_workspace_size():
    lib = _hip.load()
    p = ctypes.c_void_p(4096)
    call = lib.ka_lmhead_logprob_bf16
    ws = lib.ka_lmhead_workspace_bytes
    # 16 B per row and vocabulary split; the split count depends on the vocabulary only.  Four times that (one
    # partial per unit of a split) while token blocks x splits < 256: the call of few rows that spreads over all CUs
    assert ws(0, 4096, 128256) == 0
    assert ws(1, 4096, 128256) == 16 * 64 * 4 and ws(32768, 4096, 128256) == 32768 * 16 * 64
    assert ws(768, 4096, 128256) == 768 * 16 * 64 * 4 and ws(769, 4096, 128256) == 769 * 16 * 64
    assert ws(5, 64, 256) == 5 * 16 * 4 and ws(5, 64, 257) == 5 * 32 * 4 and ws(5, 64, 8 * 256) == 5 * 16 * 8 * 4
    assert ws(5, 64, 9 * 256) == 5 * 16 * 8 * 4 and ws(5, 64, 65 * 256) == 5 * 16 * 16 * 4
    assert ws(70000, 64, 9 * 256) == 70000 * 16 * 8
    assert ws(7, 64, 128256) == ws(7, 8192, 128256)
    assert call(None, None, None, None, 0, 4096, 128256, None, 0, None) == _hip.KA_OK             # no rows
    assert call(None, p, p, p, 4, 4096, 128256, p, 1 << 20, None) == _hip.KA_ERR_BAD_ARG
    assert call(p, p, p, p, -1, 4096, 128256, p, 1 << 20, None) == _hip.KA_ERR_BAD_ARG
    assert call(p, p, p, p, 4, 100, 128256, p, 1 << 20, None) == _hip.KA_ERR_UNSUPPORTED           # H % 64
    assert call(ctypes.c_void_p(4100), p, p, p, 4, 4096, 128256, p, 1 << 20, None) == _hip.KA_ERR_UNSUPPORTED
    assert call(p, p, p, p, 4, 4096, 1 << 31, p, 1 << 40, None) == _hip.KA_ERR_UNSUPPORTED         # vocab of 2^31
    assert call(p, p, p, p, 4, 4096, 128256, None, 0, None) == _hip.KA_ERR_WORKSPACE
    assert call(p, p, p, p, 4, 4096, 128256, p, 4 * 16 * 64 * 4 - 1, None) == _hip.KA_ERR_WORKSPACE
    assert b"workspace" in lib.ka_last_error()
    ent = lib.ka_lmhead_logprob_entropy_bf16
    assert ent(None, None, None, None, None, 0, 4096, 128256, None, 0, None) == _hip.KA_OK
    assert ent(p, p, p, p, None, 4, 4096, 128256, p, 1 << 20, None) == _hip.KA_ERR_BAD_ARG           # entropy missing
    assert ent(p, p, p, p, p, 4, 4096, 128256, p, 4 * 16 * 64 * 4 - 1, None) == _hip.KA_ERR_WORKSPACE
    # the forward that also returns the log-sum-exp, and the backward's first half that takes it
    with_lse = lib.ka_lmhead_logprob_lse_bf16
    assert with_lse(None, None, None, None, None, 0, 4096, 128256, None, 0, None) == _hip.KA_OK
    assert with_lse(p, p, p, p, None, 4, 4096, 128256, p, 1 << 20, None) == _hip.KA_ERR_BAD_ARG       # lse missing
    assert with_lse(p, p, p, p, p, 4, 4096, 128256, p, 4 * 16 * 64 * 4 - 1, None) == _hip.KA_ERR_WORKSPACE
    dl = lib.ka_lmhead_dlogits_bf16
    assert dl(None, None, None, None, None, None, 0, 0, 4096, 128256, None) == _hip.KA_OK           # no rows
    assert dl(p, p, p, p, p, p, 128256, -1, 4096, 128256, None) == _hip.KA_ERR_BAD_ARG
    assert dl(p, p, p, None, p, p, 128256, 4, 4096, 128256, None) == _hip.KA_ERR_BAD_ARG            # lse missing
    assert dl(p, p, p, p, p, p, 128255, 4, 4096, 128256, None) == _hip.KA_ERR_BAD_ARG               # stride < vocab
    assert dl(p, p, p, p, p, p, 128258, 4, 4096, 128256, None) == _hip.KA_ERR_BAD_ARG               # stride % 4
    assert dl(p, p, p, p, p, ctypes.c_void_p(4100), 128256, 4, 4096, 128256, None) == _hip.KA_ERR_BAD_ARG   # 8-byte alignment
    assert dl(p, p, p, p, p, p, 128256, 4, 100, 128256, None) == _hip.KA_ERR_UNSUPPORTED            # H % 64
    # the variant without a workspace argument: same checks, and a size limit instead of a workspace check
    na = lib.ka_lmhead_logprob_bf16_noalloc
    assert na(None, None, None, None, 0, 4096, 128256, None) == _hip.KA_OK
    assert na(None, p, p, p, 4, 4096, 128256, None) == _hip.KA_ERR_BAD_ARG
    assert na(p, p, p, p, 4, 100, 128256, None) == _hip.KA_ERR_UNSUPPORTED
    assert ws(16384, 4096, 128256) == _hip.LMHEAD_STATIC_SCRATCH_BYTES
    assert na(p, p, p, p, 16385, 4096, 128256, None) == _hip.KA_ERR_WORKSPACE
    assert b"static scratch" in lib.ka_last_error()
    header = HEADER.read_text()
    assert "#define KA_LMHEAD_STATIC_SCRATCH_BYTES (16u << 20)" in header


def test_grpo_and_backward_argument_checks():
    lib = _hip.load()
    p = ctypes.c_void_p(4096)
    g = lib.ka_grpo_token_terms
    assert g(None, None, None, None, 0, 0.2, 0.2, 0.0, None, None, None, None) == _hip.KA_OK
    assert g(None, None, None, p, 8, 0.2, 0.2, 0.0, p, p, p, None) == _hip.KA_ERR_BAD_ARG       # logp_new missing
    assert g(p, None, None, p, -3, 0.2, 0.2, 0.0, p, p, p, None) == _hip.KA_ERR_BAD_ARG
    b = lib.ka_logprob_backward_bf16
    assert b.argtypes is not None
    assert lib.ka_sample_mass_fixed(None, 0, None, None) == _hip.KA_OK
    assert lib.ka_sample_mass_fixed(None, 4, p, None) == _hip.KA_ERR_BAD_ARG


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setenv(_hip.ENV_LIB, str(tmp_path / "nope.so"))
    monkeypatch.setattr(_hip, "_lib", None)
    with pytest.raises(_hip.HipLibraryError, match="not found"):
        _hip.load()
    from rl_engine.kernels.sampling import SamplerBackend

    with pytest.raises(_hip.HipLibraryError):
        SamplerBackend()
