"""The differentiable wrappers (rl_engine.kernels.autograd) and the chunked lm_head backward against fp64
autograd / closed forms on the CPU.  Needs an MI355X.

Tolerances: logp_from_logits returns its gradient in the logits' dtype (bf16: relative 2^-8).  The lm_head
backward rebuilds bf16 logits and bf16 logit gradients before two bf16 GEMMs, so its results carry bf16
rounding of three intermediates: compared by relative Frobenius error, 2e-2.
"""
import pytest
import torch

from oracle import logprob_ref as O
from rl_engine.kernels.autograd import linear_logp, logp_from_logits

pytestmark = pytest.mark.gpu


def rel_err(got, want):
    return ((got.double().cpu() - want).norm() / want.norm()).item()


def test_logp_from_logits_backward_matches_autograd(sampler):
    g = torch.Generator().manual_seed(0)
    logits = (torch.randn(3, 17, 2056, generator=g) * 3).bfloat16()
    ids = torch.randint(0, 2056, (3, 17), generator=g)
    w = torch.randn(3, 17, generator=g)
    x = logits.cuda().requires_grad_(True)
    lp = logp_from_logits(sampler, x, ids.cuda())
    assert lp.requires_grad and lp.dtype == torch.float32
    (lp * w.cuda()).sum().backward()
    want = O.logprob_backward_closed_form(logits, ids, w)
    err = (x.grad.double().cpu() - want).abs()
    assert (err <= 2.0 ** -8 * want.abs() + 1e-6).all()
    assert torch.allclose(lp.detach().cpu(), O.logprob_ref(logits, ids), atol=1e-4, rtol=0)


@pytest.mark.parametrize("n,h,v,chunk", [(300, 256, 1000, None), (300, 256, 1000, 128), (64, 128, 4099, 50)])
def test_linear_logp_backward(sampler, n, h, v, chunk):
    g = torch.Generator().manual_seed(n + v)
    hidden = torch.randn(n, h, generator=g).bfloat16()
    weight = (torch.randn(v, h, generator=g) * 0.05).bfloat16()
    ids = torch.randint(0, v, (n,), generator=g)
    w = torch.randn(n, generator=g)
    hx = hidden.cuda().requires_grad_(True)
    wx = weight.cuda().requires_grad_(True)
    lp = linear_logp(sampler, hx, wx, ids.cuda(), chunk_tokens=chunk)
    (lp * w.cuda()).sum().backward()
    dh_ref, dw_ref = O.lmhead_logprob_backward_ref(hidden, weight, ids, w)
    dh_cf, dw_cf = O.lmhead_logprob_backward_closed_form(hidden, weight, ids, w)
    assert rel_err(dh_cf, dh_ref) < 1e-10 and rel_err(dw_cf, dw_ref) < 1e-10   # the oracle's two forms agree
    assert hx.grad.dtype == torch.bfloat16 and wx.grad.dtype == torch.bfloat16
    assert rel_err(hx.grad, dh_ref) < 2e-2
    assert rel_err(wx.grad, dw_ref) < 2e-2
    assert torch.allclose(lp.detach().cpu(), O.lmhead_logprob_ref(hidden, weight, ids), atol=2e-2, rtol=0)


@pytest.mark.parametrize("n,h,v", [(300, 256, 1000), (513, 128, 4100), (40, 64, 256)])
def test_dlogits_kernel_against_the_closed_form(sampler, n, h, v):
    """The backward's first half from the forward's MFMA kernel: lse of the forward against fp64, the gradient matrix
    g * (onehot - softmax) against the fp64 closed form on fp64 logits (bf16 rounding of the result: relative 2^-8),
    entries beyond the vocabulary of a padded row untouched, and the full backward through it tighter than through the
    GEMM path (its logits are never rounded to bf16)."""
    g = torch.Generator().manual_seed(n * 7 + v)
    hidden = torch.randn(n, h, generator=g).bfloat16()
    weight = (torch.randn(v, h, generator=g) * 0.05).bfloat16()
    ids = torch.randint(0, v, (n,), generator=g)
    w = torch.randn(n, generator=g)
    hd, wd, idd, gd = hidden.cuda(), weight.cuda(), ids.cuda(), w.cuda()
    logp, lse = sampler.fused_linear_logp(hd, wd, idd, return_lse=True)
    assert torch.equal(logp, sampler.fused_linear_logp(hd, wd, idd))
    logits64 = hidden.double() @ weight.double().t()
    assert (lse.double().cpu() - torch.logsumexp(logits64, -1)).abs().max().item() < 1e-4
    stride = v + 8
    dl = torch.full((n, stride), 7.0, dtype=torch.bfloat16, device="cuda")
    from rl_engine.kernels import _hip
    _hip.check(sampler._lib.ka_lmhead_dlogits_bf16(hd.data_ptr(), wd.data_ptr(), idd.data_ptr(), lse.data_ptr(),
                                                   gd.data_ptr(), dl.data_ptr(), stride, n, h, v,
                                                   torch.cuda.current_stream().cuda_stream), "ka_lmhead_dlogits_bf16")
    want = O.logprob_backward_closed_form(logits64, ids, w)
    got = dl[:, :v].double().cpu()
    assert ((got - want).abs() <= 2.0 ** -8 * want.abs() + 1e-6).all()
    assert (dl[:, v:] == 7.0).all()
    dh, dw = sampler.fused_linear_logp_backward(hd, wd, idd, gd, chunk_tokens=128, lse=lse)
    dh_ref, dw_ref = O.lmhead_logprob_backward_ref(hidden, weight, ids, w)
    assert rel_err(dh, dh_ref) < 1e-2 and rel_err(dw, dw_ref) < 1e-2
    dh_g, dw_g = sampler.fused_linear_logp_backward(hd, wd, idd, gd, chunk_tokens=128)
    assert rel_err(dh, dh_g.double().cpu()) < 2e-2 and rel_err(dw, dw_g.double().cpu()) < 2e-2


def test_backward_holds_one_chunk_of_the_gradient_matrix(sampler):
    """Peak device memory of the backward beyond its two results: one [chunk, V] bf16 matrix (plus the small per-row
    vectors), whatever the number of rows - with either first half."""
    g = torch.Generator(device="cuda").manual_seed(9)
    n, h, v, chunk = 4096, 256, 32000, 512
    hidden = torch.randn(n, h, generator=g, device="cuda").bfloat16()
    weight = (torch.randn(v, h, generator=g, device="cuda") * 0.05).bfloat16()
    ids = torch.randint(0, v, (n,), generator=g, device="cuda")
    grad = torch.randn(n, generator=g, device="cuda")
    _, lse = sampler.fused_linear_logp(hidden, weight, ids, return_lse=True)
    for kw in ({}, {"lse": lse}):
        sampler.fused_linear_logp_backward(hidden, weight, ids, grad, chunk_tokens=chunk, **kw)   # warm: library workspaces
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        before = torch.cuda.memory_allocated()
        dh, dw = sampler.fused_linear_logp_backward(hidden, weight, ids, grad, chunk_tokens=chunk, **kw)
        torch.cuda.synchronize()
        extra = torch.cuda.max_memory_allocated() - before
        results = dh.numel() * 2 + dw.numel() * 4
        one_chunk = chunk * v * 2
        assert extra <= results + one_chunk + (4 << 20), (extra, results, one_chunk)


def test_chunked_backward_direct_call_and_shapes(sampler):
    g = torch.Generator().manual_seed(5)
    hidden = torch.randn(2, 40, 192, generator=g).bfloat16().cuda()
    weight = (torch.randn(777, 192, generator=g) * 0.05).bfloat16().cuda()
    ids = torch.randint(0, 777, (2, 40), generator=g).cuda()
    grad = torch.randn(2, 40, generator=g).cuda()
    dh, dw = sampler.fused_linear_logp_backward(hidden, weight, ids, grad, chunk_tokens=32)
    assert dh.shape == hidden.shape and dh.dtype == torch.bfloat16
    assert dw.shape == weight.shape and dw.dtype == torch.float32
    dh_ref, dw_ref = O.lmhead_logprob_backward_ref(hidden.reshape(-1, 192), weight, ids.reshape(-1), grad.reshape(-1))
    assert rel_err(dh.reshape(-1, 192), dh_ref.reshape(-1, 192)) < 2e-2
    assert rel_err(dw, dw_ref) < 2e-2
    dh16, dw16 = sampler.fused_linear_logp_backward(hidden, weight, ids, grad, chunk_tokens=32,
                                                    dweight_dtype=torch.bfloat16)
    assert dw16.dtype == torch.bfloat16 and torch.equal(dh16, dh)
    assert rel_err(dw16, dw_ref) < 2e-2
    one_chunk = sampler.fused_linear_logp_backward(hidden, weight, ids, grad, chunk_tokens=80)[1]
    assert rel_err(one_chunk, dw.double().cpu()) < 1e-3                       # chunking only regroups the fp32 accumulation
    with pytest.raises(ValueError):
        sampler.fused_linear_logp_backward(hidden, weight, ids[:1], grad)
    with pytest.raises(TypeError):
        sampler.fused_linear_logp_backward(hidden.float(), weight, ids, grad)
    with pytest.raises(TypeError):
        sampler.fused_linear_logp_backward(hidden, weight, ids, grad, dweight_dtype=torch.float16)
