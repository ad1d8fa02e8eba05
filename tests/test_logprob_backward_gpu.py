"""Backward of the logprob operator against torch autograd on the CPU.  Needs an MI355X.

Tolerance: the gradient is returned in the logits' dtype, so a bf16 / fp16 result is compared at half an
ulp of that dtype (relative 2^-8 / 2^-11) plus 1e-6 absolute; fp32 at 1e-5 relative + 1e-7 absolute.
"""
import pytest
import torch

from oracle import logprob_ref as O

pytestmark = pytest.mark.gpu
RTOL = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 1e-5}


def make(n, v, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(n, v, generator=g) * 3).to(dtype)
    ids = torch.randint(0, v, (n,), generator=g)
    grad = torch.randn(n, generator=g)
    return logits, ids, grad


def check(got, logits, ids, grad):
    want = O.logprob_backward_closed_form(logits, ids, grad)
    err = (got.double() - want).abs()
    tol = RTOL[logits.dtype] * want.abs() + (1e-7 if logits.dtype == torch.float32 else 1e-6)
    assert (err <= tol).all(), f"max excess {(err - tol).max().item():.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n,v", [(64, 32000), (5, 2049), (3, 7), (33, 128256)])
def test_matches_autograd(sampler, dtype, n, v):
    logits, ids, grad = make(n, v, dtype, n + v)
    dl, di, dg = logits.cuda(), ids.cuda(), grad.cuda()
    logp = sampler.compute_logp(dl, di)
    got = sampler.compute_logp_backward(dl, di, logp, dg)
    assert got.dtype == dtype and got.shape == logits.shape
    check(got.cpu(), logits, ids, grad)


def test_in_place_and_3d(sampler):
    logits, ids, grad = make(8 * 16, 32000, torch.bfloat16, 5)
    dl = logits.cuda().view(8, 16, 32000)
    di, dg = ids.cuda().view(8, 16), grad.cuda().view(8, 16)
    logp = sampler.compute_logp(dl, di)
    ref = sampler.compute_logp_backward(dl, di, logp, dg)
    before = torch.cuda.memory_allocated()
    out = sampler.compute_logp_backward(dl, di, logp, dg, inplace=True)
    assert out.data_ptr() == dl.data_ptr() and torch.cuda.memory_allocated() - before < (1 << 20)
    assert torch.equal(out, ref)
    check(out.view(-1, 32000).cpu(), logits, ids, grad)


def test_unaligned_rows_and_determinism(sampler):
    g = torch.Generator().manual_seed(6)
    big = (torch.randn(16, 4104, generator=g) * 3).bfloat16().cuda()
    ids = torch.randint(0, 4001, (16,), generator=g).cuda()
    grad = torch.randn(16, generator=g).cuda()
    for view in (big[:, 3:4004], big[:, 8:4009]):
        logp = sampler.compute_logp(view, ids)
        got = sampler.compute_logp_backward(view, ids, logp, grad)
        check(got.cpu(), view.cpu().contiguous(), ids.cpu(), grad.cpu())
        assert torch.equal(got, sampler.compute_logp_backward(view, ids, logp, grad))
    parts = torch.cat([sampler.compute_logp_backward(big[s:s + 4, :4096], ids[s:s + 4],
                                                     sampler.compute_logp(big[s:s + 4, :4096], ids[s:s + 4]), grad[s:s + 4])
                       for s in range(0, 16, 4)])
    whole = sampler.compute_logp_backward(big[:, :4096], ids, sampler.compute_logp(big[:, :4096], ids), grad)
    assert torch.equal(parts, whole)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_masked_target_gets_the_finite_gradient_autograd_gives(sampler, dtype):
    """A target whose logit is -inf has logp = -inf, so the log-sum-exp cannot be recovered from it: the kernel
    recomputes it for such a row and returns -g * softmax (what autograd gives), not NaN."""
    logits, ids, grad = make(12, 5003, dtype, 77)
    logits[3, ids[3]] = float("-inf")
    logits[8, 100:] = float("-inf")
    ids[8] = 4000                                  # masked target in a row with a masked tail
    dl, di, dg = logits.cuda(), ids.cuda(), grad.cuda()
    logp = sampler.compute_logp(dl, di)
    assert logp[3].item() == float("-inf") and logp[8].item() == float("-inf")
    got = sampler.compute_logp_backward(dl, di, logp, dg).cpu()
    assert torch.isfinite(got).all()
    check(got, logits, ids, grad)
    auto = O.logprob_backward_ref(logits, ids, grad, dtype=torch.float64)
    assert torch.isfinite(auto).all() and (got.double() - auto).abs().max().item() < 2e-2
    inplace = sampler.compute_logp_backward(dl.clone(), di, logp, dg, inplace=True)
    assert torch.equal(inplace.cpu(), got)
    with pytest.raises(ValueError, match="chunk_tokens"):
        sampler.compute_logp_backward(dl, di, logp, dg, chunk_tokens=-1)
