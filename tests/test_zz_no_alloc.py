"""Collected last on purpose (a failure here must not hide other tests).  ka_lmhead_logprob_bf16_noalloc (partials in a static device array) against ka_lmhead_logprob_bf16 (partials
in a caller's workspace), called through the C ABI: same bits, on two calls in a row of which the second is
smaller, and no device allocation between the two calls.  Needs an MI355X."""
import pytest
import torch

from oracle import logprob_ref as O
from rl_engine.kernels import _hip

pytestmark = pytest.mark.gpu


def _inputs(n, h, v, seed):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, h, generator=g).bfloat16()
    weight = (torch.randn(v, h, generator=g) * 0.1).bfloat16()
    ids = torch.randint(0, v, (n,), generator=g)
    return hidden, weight, ids


def _with_workspace(lib, hidden, weight, ids, stream):
    n, h = hidden.shape
    v = weight.shape[0]
    out = torch.full((n,), float("nan"), dtype=torch.float32, device=hidden.device)
    ws_bytes = lib.ka_lmhead_workspace_bytes(n, h, v)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=hidden.device)
    _hip.check(lib.ka_lmhead_logprob_bf16(hidden.data_ptr(), weight.data_ptr(), ids.data_ptr(), out.data_ptr(),
                                          n, h, v, ws.data_ptr(), ws_bytes, stream), "ka_lmhead_logprob_bf16")
    torch.cuda.synchronize()
    return out


def test_noalloc_entry_matches_workspace_entry_twice_in_a_row():
    assert torch.cuda.is_available(), "gpu tests need a GPU"
    lib = _hip.load()
    dev = torch.device("cuda", 0)
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream().cuda_stream
        # first call: 1,000 rows x 20,000 entries (79 tiles = 16 splits: 256,000 B of partials, ragged last token
        # block and last tile); second call: fewer rows and a smaller vocabulary, so it covers only a part of what
        # the first call left in the array
        cases = [_inputs(1000, 128, 20000, seed=5), _inputs(77, 128, 3000, seed=6)]
        on_gpu = [tuple(t.to(dev) for t in case) for case in cases]
        want = [_with_workspace(lib, *case, stream) for case in on_gpu]
        outs = [torch.full((case[0].shape[0],), float("nan"), dtype=torch.float32, device=dev) for case in on_gpu]
        torch.cuda.synchronize()
        for (hidden, weight, ids), out in zip(on_gpu, outs):
            n, h = hidden.shape
            status = lib.ka_lmhead_logprob_bf16_noalloc(hidden.data_ptr(), weight.data_ptr(), ids.data_ptr(),
                                                        out.data_ptr(), n, h, weight.shape[0], stream)
            _hip.check(status, "ka_lmhead_logprob_bf16_noalloc")
        torch.cuda.synchronize()
        for got, ref, (hidden, weight, ids) in zip(outs, want, cases):
            assert torch.equal(got, ref)                                                # bit for bit
            oracle = O.lmhead_logprob_ref(hidden, weight, ids, dtype=torch.float64)
            assert (got.cpu().double() - oracle).abs().max().item() <= 1e-4
        # and once more in the other order (large after small); the device's set-up is done by now, so these
        # calls must leave the amount of free device memory and torch's allocation count where they were
        before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
        free_before, _ = torch.cuda.mem_get_info(dev)
        for k in (1, 0):
            hidden, weight, ids = on_gpu[k]
            outs[k].fill_(float("nan"))
            _hip.check(lib.ka_lmhead_logprob_bf16_noalloc(hidden.data_ptr(), weight.data_ptr(), ids.data_ptr(),
                                                          outs[k].data_ptr(), hidden.shape[0], hidden.shape[1],
                                                          weight.shape[0], stream), "ka_lmhead_logprob_bf16_noalloc")
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info(dev)
        assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before
        assert free_after >= free_before
        assert torch.equal(outs[0], want[0]) and torch.equal(outs[1], want[1])


def test_noalloc_entry_rejects_what_does_not_fit():
    assert torch.cuda.is_available(), "gpu tests need a GPU"
    lib = _hip.load()
    dev = torch.device("cuda", 0)
    limit = _hip.LMHEAD_STATIC_SCRATCH_BYTES
    h, v = 64, 128256
    fits = limit // (lib.ka_lmhead_workspace_bytes(1 << 20, h, v) >> 20)   # bytes per row of a call of many rows
    assert lib.ka_lmhead_workspace_bytes(fits, h, v) <= limit < lib.ka_lmhead_workspace_bytes(fits + 1, h, v)
    assert fits == 16384
    # real (small) buffers, a row count beyond the limit: the call must refuse before it launches anything
    hidden = torch.zeros(8, h, dtype=torch.bfloat16, device=dev)
    weight = torch.zeros(8, h, dtype=torch.bfloat16, device=dev)
    ids = torch.zeros(8, dtype=torch.int64, device=dev)
    out = torch.zeros(8, dtype=torch.float32, device=dev)
    status = lib.ka_lmhead_logprob_bf16_noalloc(hidden.data_ptr(), weight.data_ptr(), ids.data_ptr(), out.data_ptr(),
                                                fits + 1, h, v, None)
    assert status == _hip.KA_ERR_WORKSPACE and b"static scratch" in lib.ka_last_error()
    with pytest.raises(ValueError, match="KA_ERR_WORKSPACE"):
        _hip.check(status, "ka_lmhead_logprob_bf16_noalloc")
    assert lib.ka_lmhead_logprob_bf16_noalloc(None, None, None, None, 0, h, v, None) == _hip.KA_OK
