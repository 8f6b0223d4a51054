"""Pins the loss-stage oracle with the reference's own known answers and with closed forms."""

import math

import pytest
import torch

from oracle import loss as O
from tests.golden.rejection_cases import BINARY_KL_CASES, CASES


def _t(x, dtype=torch.float32):
    return torch.tensor(x, dtype=dtype)


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_rejection_sampling_known_answers(case):
    cu = _t(case["cu"], torch.int32) if case["cu"] is not None else None
    r = O.rejection_sampling(_t(case["prox"]), _t(case["old"]), _t(case["mask"]), cu, **case["cfg"])
    assert torch.equal(r.loss_mask, _t(case["exp_mask"]))
    if case["exp_weight"] is not None:
        torch.testing.assert_close(r.behave_imp_weight, _t(case["exp_weight"]), rtol=1e-5, atol=1e-5)
    if case["exp_fraction"] is not None:
        assert r.filtered_fraction == pytest.approx(case["exp_fraction"])
    assert not torch.isnan(r.behave_imp_weight).any()


@pytest.mark.parametrize("case", BINARY_KL_CASES, ids=[c["name"] for c in BINARY_KL_CASES])
def test_binary_kl_cases(case):
    r = O.rejection_sampling(_t(case["prox"]), _t(case["old"]), _t(case["mask"]),
                             _t(case["cu"], torch.int32), **case["cfg"])
    assert torch.equal(r.loss_mask, _t(case["exp_mask"]))


def test_binary_kl_matches_float64_closed_form():
    torch.manual_seed(0)
    p = torch.rand(200, dtype=torch.float64) * 0.98 + 0.01
    q = torch.rand(200, dtype=torch.float64) * 0.98 + 0.01
    want = p * (p / q).log() + (1 - p) * ((1 - p) / (1 - q)).log()
    got = O.binary_kl(p.log().float(), q.log().float())
    torch.testing.assert_close(got.double(), want, rtol=2e-4, atol=2e-6)
    assert (got >= -1e-6).all()
    # symmetric in the sense used by the metric: max of both directions is symmetric
    a = torch.maximum(O.binary_kl(p.log().float(), q.log().float()), O.binary_kl(q.log().float(), p.log().float()))
    b = torch.maximum(O.binary_kl(q.log().float(), p.log().float()), O.binary_kl(p.log().float(), q.log().float()))
    assert torch.equal(a, b)


def test_binary_kl_matches_scipy_rel_entr_on_a_grid():
    """An independent routine for the same quantity: the Bernoulli KL is
    rel_entr(p, q) + rel_entr(1 - p, 1 - q) (scipy.special.rel_entr(x, y) = x log(x / y)).
    A dropped term, swapped arguments or a wrong sign fail here; the fp32 clamp quirk
    (p rounding to 1 -> NaN -> token rejected) is pinned by BINARY_KL_CASES above."""
    import numpy as np
    from scipy.special import rel_entr

    ps = np.concatenate([np.linspace(0.001, 0.999, 41), [1e-6, 0.5, 1 - 1e-4]])
    p, q = np.meshgrid(ps, ps, indexing="ij")
    want = rel_entr(p, q) + rel_entr(1.0 - p, 1.0 - q)
    got = O.binary_kl(torch.from_numpy(np.log(p)).float(), torch.from_numpy(np.log(q)).float())
    # fp32 evaluation of exp(log p): relative 1e-6 on p, amplified by 1/q and 1/(1-q) near the edges
    np.testing.assert_allclose(got.double().numpy(), want, rtol=5e-4, atol=2e-5)
    assert np.all(np.diag(got.numpy()) == 0.0)  # KL(p || p) = 0 exactly
    # asymmetry: the two directions differ, and the metric takes the larger
    i, j = 3, 30
    assert abs(want[i, j] - want[j, i]) > 1e-3
    both = torch.maximum(got, got.T)
    np.testing.assert_allclose(both.double().numpy(), np.maximum(want, want.T), rtol=5e-4, atol=2e-5)


def test_kl_estimators_closed_forms():
    d = _t([-1.0, -0.3, 0.0, 0.5, 2.0])
    z = torch.zeros_like(d)
    assert torch.equal(O.approx_kl(d, z, "k1"), d)
    torch.testing.assert_close(O.approx_kl(d, z, "k2"), d * d / 2)
    torch.testing.assert_close(O.approx_kl(d, z, "k3"), torch.exp(-d) - 1 + d)
    assert (O.approx_kl(d, z, "k3") >= 0).all()


def _cispo_inputs():
    # fixture of the reference's tests/test_cispo_loss.py:21-32
    log_ratio = _t([-2.0, -0.5, 0.0, 0.3, 1.5, 0.1])
    logprobs = _t([-1.0, -2.0, -0.3, -1.2, -0.7, -2.5]).requires_grad_(True)
    proximal = logprobs.detach() - log_ratio
    adv = _t([1.0, -2.0, 0.5, 3.0, -1.0, 2.0])
    mask = torch.tensor([1, 1, 1, 1, 1, 0], dtype=torch.bool)
    return logprobs, proximal, adv, mask, log_ratio


@pytest.mark.parametrize("eps,eps_hi", [(0.2, 0.28), (1.0, 4.0)])
def test_cispo_value_clip_mask_and_gradient(eps, eps_hi):
    lp, prox, adv, mask, lr = _cispo_inputs()
    loss, stat = O.cispo_loss(lp, prox, adv, eps, mask, eps_hi)
    ratio = lr.exp()
    rc = ratio.clamp(1 - eps, 1 + eps_hi)
    per = -rc * adv * lp.detach()
    torch.testing.assert_close(loss, torch.where(mask, per, 0.0).sum() / 5)
    torch.testing.assert_close(stat["importance_weight"], ratio)
    assert torch.equal(stat["clip_mask"], (ratio != rc) & mask)
    assert not stat["dual_clip_mask"].any()
    loss.backward()
    torch.testing.assert_close(lp.grad, torch.where(mask, -rc * adv / 5, 0.0))


def test_cispo_decoupled_weight():
    lp, prox, adv, mask, lr = _cispo_inputs()
    blr = _t([0.2, -0.4, 0.0, 0.1, -0.3, 0.5])
    old = prox - blr
    loss, stat = O.cispo_loss(lp, prox, adv, 1.0, mask, 4.0, old_logprobs=old,
                              rejection_sampling_cfg=dict(level="token", action="clamp", metric="ratio", upper=100.0))
    rc = lr.exp().clamp(0.0, 5.0)
    per = -rc * adv * lp.detach() * blr.exp()
    torch.testing.assert_close(loss, torch.where(mask, per, 0.0).sum() / 5)
    torch.testing.assert_close(stat["behave_imp_weight"][mask], blr.exp()[mask])
    loss.backward()
    torch.testing.assert_close(lp.grad, torch.where(mask, -rc * adv * blr.exp() / 5, 0.0))


def test_cispo_rejects_bad_eps_clip_higher():
    lp, prox, adv, mask, _ = _cispo_inputs()
    for bad in (None, 0.0, -1.0):
        with pytest.raises(ValueError, match="eps_clip_higher"):
            O.cispo_loss(lp, prox, adv, 1.0, mask, bad)


def test_gspo_geometric_mean_ratio_2d_and_packed():
    # reference tests/test_functional.py:89-177
    lp2 = _t([[1.0] * 4, [2.0] * 4])
    px2 = _t([[0.5] * 4, [1.0] * 4])
    ones = torch.ones(2, 4)
    m = torch.ones(2, 4, dtype=torch.bool)
    _, st = O.ppo_actor_loss(lp2, px2, torch.zeros(2, 4), ones, 0.2, m, importance_sampling_level="sequence")
    torch.testing.assert_close(st["importance_weight"][0], torch.full((4,), math.exp(0.5)), atol=1e-5, rtol=0)
    torch.testing.assert_close(st["importance_weight"][1], torch.full((4,), math.exp(1.0)), atol=1e-5, rtol=0)
    _, st = O.ppo_actor_loss(lp2.view(-1), px2.view(-1), torch.zeros(8), torch.ones(8), 0.2, m.view(-1),
                             importance_sampling_level="sequence", cu_seqlens=_t([0, 4, 8], torch.int32))
    torch.testing.assert_close(st["importance_weight"][:4], torch.full((4,), math.exp(0.5)), atol=1e-5, rtol=0)
    torch.testing.assert_close(st["importance_weight"][4:], torch.full((4,), math.exp(1.0)), atol=1e-5, rtol=0)


def test_gspo_advantage_average_loss_literal():
    # reference tests/test_functional.py:179-218: loss == -1.5
    adv = _t([[1.0, 2.0, 3.0, 4.0], [0.5] * 4])
    ones = torch.ones(2, 4)
    loss, _ = O.ppo_actor_loss(ones, ones, ones, adv, 0.2, torch.ones(2, 4, dtype=torch.bool),
                               importance_sampling_level="sequence")
    torch.testing.assert_close(loss, _t(-1.5))


def test_gspo_masked_advantages_do_not_contaminate():
    # reference tests/test_functional.py:261-296
    m = torch.tensor([[True, True, False, False]])
    z = torch.zeros(1, 4)
    l1, s1 = O.ppo_actor_loss(z, z, z, _t([[1.0, 1.0, 0.0, 0.0]]), 0.2, m, importance_sampling_level="sequence")
    l2, s2 = O.ppo_actor_loss(z, z, z, _t([[1.0, 1.0, 10.0, 10.0]]), 0.2, m, importance_sampling_level="sequence")
    torch.testing.assert_close(l1, l2)
    torch.testing.assert_close(s1["loss"][m], s2["loss"][m])
    assert (s2["loss"][~m] == 0).all()


def test_ppo_all_masked_gives_zero_loss():
    z = torch.randn(6)
    loss, st = O.ppo_actor_loss(z.clone().requires_grad_(True), z, z, torch.randn(6), 0.2,
                                torch.zeros(6, dtype=torch.bool))
    assert loss.item() == 0.0
    assert st["n_valid_tokens"] == 0.0 and st["masked_token_ratio"] == 1.0


def test_ppo_errors():
    z = torch.zeros(4)
    m = torch.ones(4, dtype=torch.bool)
    with pytest.raises(ValueError, match="cu_seqlens"):
        O.ppo_actor_loss(z, z, z, z, 0.2, m, importance_sampling_level="sequence")
    with pytest.raises(ValueError, match="importance_sampling_level"):
        O.ppo_actor_loss(z, z, z, z, 0.2, m, importance_sampling_level="bogus")
    with pytest.raises(AssertionError):
        O.ppo_actor_loss(z, z, z, z, 0.2, m, c_clip=0.5)


def test_ppo_gradient_five_cases():
    """In band -> -A r; r>hi,A>0 -> 0; r>hi,A<0 -> -A r; r<lo,A>0 -> -A r; r<lo,A<0 -> 0."""
    lr = _t([0.05, 0.5, 0.5, -0.5, -0.5, 0.0])
    adv = _t([2.0, 1.0, -1.0, 1.0, -1.0, 3.0])
    lp = _t([-1.0, -1.5, -0.2, -0.7, -2.0, -1.0]).requires_grad_(True)
    prox = lp.detach() - lr
    mask = torch.tensor([1, 1, 1, 1, 1, 0], dtype=torch.bool)
    loss, _ = O.ppo_actor_loss(lp, prox, prox, adv, 0.2, mask)
    loss.backward()
    r = lr.exp()
    want = _t([-2.0 * r[0].item(), 0.0, 1.0 * r[2].item(), -1.0 * r[3].item(), 0.0, 0.0]) / 5
    torch.testing.assert_close(lp.grad, want)
    torch.testing.assert_close(
        O.ppo_closed_form_grad(lp.detach(), prox, adv, mask, 5, 0.8, 1.2), want)


def test_closed_form_grad_matches_autograd_random():
    torch.manual_seed(3)
    n = 4000
    lp = (torch.randn(n) * 0.5 - 1).requires_grad_(True)
    prox = lp.detach() + torch.randn(n) * 0.2
    old = prox + torch.randn(n) * 0.3
    adv = torch.randn(n)
    adv[::17] = 0.0
    mask = torch.rand(n) > 0.2
    cfg = dict(level="token", action="mask", metric="ratio", upper=2.0, lower=0.5)
    loss, st = O.ppo_actor_loss(lp, prox, old, adv, 0.2, mask, eps_clip_higher=0.28, c_clip=3.0,
                                rejection_sampling_cfg=cfg)
    loss.backward()
    want = O.ppo_closed_form_grad(lp.detach(), prox, adv, st["new_mask"], mask.sum(), 0.8, 1.28, c_clip=3.0,
                                  weight=st["behave_imp_weight"])
    torch.testing.assert_close(lp.grad, want, rtol=1e-6, atol=1e-9)
