"""The GRPO per-token epilogue (ka_grpo_token_terms) against the fp64 torch statement and closed forms.
Needs an MI355X.  Tolerance: fp32 elementwise arithmetic with expf, 2e-6 relative + 1e-6 absolute."""
import pytest
import torch

from oracle import grpo_ref

pytestmark = pytest.mark.gpu


def close(got, want, name):
    err = (got.double().cpu() - want).abs()
    tol = 2e-6 * want.abs() + 1e-6
    assert (err <= tol).all(), f"{name}: max excess {(err - tol).max().item():.3e}"


@pytest.mark.parametrize("with_old,with_ref,beta", [(True, True, 0.04), (True, False, 0.0), (False, True, 0.1),
                                                    (False, False, 0.0)])
def test_matches_fp64_statement_and_autograd(sampler, with_old, with_ref, beta):
    g = torch.Generator().manual_seed(3)
    shape = (7, 301)
    new = -torch.rand(shape, generator=g) * 6
    old = new + torch.randn(shape, generator=g) * 0.3 if with_old else None
    ref = new + torch.randn(shape, generator=g) * 0.5 if with_ref else None
    adv = torch.randn(shape, generator=g)
    loss, kl, dlogp = sampler.grpo_token_loss(new.cuda(), adv.cuda(), None if old is None else old.cuda(),
                                              None if ref is None else ref.cuda(), 0.2, 0.28, beta)
    w_loss, w_kl, w_d = grpo_ref.grpo_token_terms(new, adv, old, ref, 0.2, 0.28, beta)
    close(loss, w_loss, "loss")
    close(kl, w_kl, "kl")
    close(dlogp, w_d, "dlogp")


def test_closed_forms(sampler):
    n = 1000
    new = torch.linspace(-5, 0, n)
    adv = torch.linspace(-2, 2, n)
    # on policy, reference equal to the policy: ratio 1, kl 0, loss = -A, derivative = -A
    loss, kl, d = sampler.grpo_token_loss(new.cuda(), adv.cuda(), new.cuda(), new.cuda(), 0.2, 0.2, 0.5)
    assert torch.equal(loss.cpu(), -adv) and torch.equal(d.cpu(), -adv) and not kl.any()
    # ratio = e above the clip range: positive advantages are clipped (constant, no gradient), negative ones are not
    old = new - 1.0
    loss, _, d = sampler.grpo_token_loss(new.cuda(), adv.cuda(), old.cuda(), None, 0.2, 0.2, 0.0)
    pos = adv > 0
    assert torch.allclose(loss.cpu()[pos], -(1.2 * adv[pos]), rtol=1e-6) and not d.cpu()[pos].any()
    e = torch.exp(torch.tensor(1.0))
    assert torch.allclose(loss.cpu()[~pos], -(e * adv[~pos]), rtol=1e-6)
    assert torch.allclose(d.cpu()[~pos], -(e * adv[~pos]), rtol=1e-6)
    # the k3 estimate is non-negative and zero only at ref == new
    _, kl, _ = sampler.grpo_token_loss(new.cuda(), adv.cuda(), None, (new + torch.randn(n)).cuda(), 0.2, 0.2, 1.0)
    assert (kl >= 0).all()


def test_sequence_advantages_broadcast_and_feed_the_backward_kernel(sampler):
    g = torch.Generator().manual_seed(9)
    logits = (torch.randn(4, 9, 3000, generator=g) * 2).bfloat16().cuda()
    ids = torch.randint(0, 3000, (4, 9), generator=g).cuda()
    adv_seq = torch.randn(4, generator=g).cuda()                       # one advantage per sequence
    logp = sampler.compute_logp(logits, ids)
    loss, _, dlogp = sampler.grpo_token_loss(logp, adv_seq)
    assert torch.equal(loss, -adv_seq.unsqueeze(-1).expand(4, 9))
    dlogits = sampler.compute_logp_backward(logits, ids, logp, dlogp)
    # d loss / d logits = dlogp * (onehot - softmax): checked against autograd of the whole chain in fp64
    x = logits.double().cpu().requires_grad_(True)
    lp = torch.log_softmax(x, -1).gather(-1, ids.cpu().unsqueeze(-1)).squeeze(-1)
    (-(torch.exp(lp - lp.detach()) * adv_seq.double().cpu().unsqueeze(-1))).sum().backward()
    err = (dlogits.double().cpu() - x.grad).abs()
    assert (err <= 2.0 ** -8 * x.grad.abs() + 1e-6).all()
    with pytest.raises(ValueError):
        sampler.grpo_token_loss(logp, adv_seq[:3])
