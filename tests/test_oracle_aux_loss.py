"""Pins of the CPU oracle for SAPO, the critic loss and the DPO sequence sums.

SAPO cases restate tests/test_functional.py:844-1224 of the reference (inputs and expected
values re-typed); the critic loss and DPO have no reference test and are pinned by hand-computed
values, closed forms and brute force."""

import math

import pytest
import torch

from oracle import aux_loss as A


# ---------------------------------------------------------------- SAPO
def test_sapo_known_value_at_ratio_one():
    # reference tests/test_functional.py:923-954
    lp = torch.tensor([[1.0, 1.0]])
    loss, stat = A.sapo_loss(lp, lp.clone(), torch.tensor([[1.0, 1.0]]), 1.0, 1.0, torch.ones(1, 2, dtype=torch.bool))
    assert torch.allclose(loss, torch.tensor(-2.0), atol=1e-5)
    assert torch.allclose(stat["sapo_soft_gate"], torch.tensor([[2.0, 2.0]]), atol=1e-5)


@pytest.mark.parametrize("adv,pick", [([1.0, 2.0], "pos"), ([-1.0, -2.0], "neg")])
def test_sapo_gate_selection(adv, pick):
    # reference :956-1004
    lp = torch.tensor([[0.5, 0.5]])
    _, stat = A.sapo_loss(lp, torch.zeros(1, 2), torch.tensor([adv]), 1.0, 2.0, torch.ones(1, 2, dtype=torch.bool))
    assert torch.allclose(stat["sapo_soft_gate"], stat[f"sapo_scaled_gate_{pick}"], atol=1e-6)
    # closed form of the selected gate at ratio e^0.5
    tau = 1.0 if pick == "pos" else 2.0
    want = 4.0 / tau / (1.0 + math.exp(-tau * (math.exp(0.5) - 1.0)))
    assert abs(stat["sapo_soft_gate"][0, 0].item() - want) < 1e-6


def test_sapo_mixed_signs_and_zero_advantage_uses_negative_gate():
    # reference :1006-1036; advantage 0 is "not positive"
    lp = torch.tensor([[0.5, 0.5, 0.5, 0.5]])
    _, stat = A.sapo_loss(lp, torch.zeros(1, 4), torch.tensor([[1.0, -1.0, 2.0, 0.0]]), 1.0, 2.0,
                          torch.ones(1, 4, dtype=torch.bool))
    g, gp, gn = stat["sapo_soft_gate"][0], stat["sapo_scaled_gate_pos"][0], stat["sapo_scaled_gate_neg"][0]
    assert g[0] == gp[0] and g[2] == gp[2] and g[1] == gn[1] and g[3] == gn[3]


def test_sapo_temperature_errors():
    x = torch.tensor([[1.0]])
    m = torch.ones(1, 1, dtype=torch.bool)
    with pytest.raises(ValueError, match="must be positive"):
        A.sapo_loss(x, x, x, 0.0, 1.0, m)
    with pytest.raises(ValueError, match="must be positive"):
        A.sapo_loss(x, x, x, 1.0, -1.0, m)


def test_sapo_gradient_is_tau_independent_at_ratio_one():
    # reference :1160-1195: the 4/tau factor makes d loss / d logprob = -A at ratio 1
    grads = []
    for tau in (1.0, 2.0):
        lp = torch.tensor([[0.0]], requires_grad=True)
        loss, _ = A.sapo_loss(lp, torch.tensor([[0.0]]), torch.tensor([[1.0]]), tau, tau, torch.ones(1, 1, dtype=torch.bool))
        loss.backward()
        grads.append(lp.grad.clone())
    assert torch.allclose(grads[0], grads[1], atol=1e-6)
    assert torch.allclose(grads[0], torch.tensor([[-1.0]]), atol=1e-6)


def test_sapo_loss_mask_formula_and_closed_form_gradient():
    # reference :1197-1224, then the gradient -4 g (1 - g) A r / N against autograd
    g = torch.Generator().manual_seed(0)
    lp = torch.randn(1, 4, generator=g).requires_grad_(True)
    old, adv = torch.randn(1, 4, generator=g), torch.randn(1, 4, generator=g)
    mask = torch.tensor([[True, True, False, False]])
    loss, _ = A.sapo_loss(lp, old, adv, 1.0, 1.0, mask)
    ratio = torch.exp(lp[:, :2] - old[:, :2])
    want = -(torch.sigmoid(ratio - 1.0) * 4.0 * adv[:, :2]).sum() / 2
    assert torch.allclose(loss, want, atol=1e-5)
    loss.backward()
    r = torch.exp(lp.detach() - old)
    s = torch.sigmoid(r - 1.0)
    closed = torch.where(mask, -4.0 * s * (1 - s) * adv * r / 2, torch.zeros(()))
    assert torch.allclose(lp.grad, closed, atol=1e-6)


def test_sapo_sequence_level_uses_geometric_mean_ratio_and_mean_advantage():
    cu = torch.tensor([0, 2, 5], dtype=torch.int32)
    lp = torch.tensor([0.2, 0.4, 0.0, 0.3, 0.6])
    old = torch.zeros(5)
    adv = torch.tensor([1.0, 3.0, -1.0, -2.0, 100.0])
    mask = torch.tensor([True, True, True, True, False])
    loss, stat = A.sapo_loss(lp, old, adv, 1.0, 1.5, mask, "sequence", cu)
    r0, r1 = math.exp(0.3), math.exp(0.15)
    torch.testing.assert_close(stat["importance_weight"], torch.tensor([r0, r0, r1, r1, 0.0]), rtol=1e-6, atol=0)
    g0 = 4.0 / (1 + math.exp(-(r0 - 1)))                 # advantage mean 2.0 > 0
    g1 = 4.0 / 1.5 / (1 + math.exp(-1.5 * (r1 - 1)))     # advantage mean -1.5
    want = (-(g0 * 2.0) * 2 - (g1 * -1.5) * 2) / 4
    assert abs(loss.item() - want) < 1e-6


# ---------------------------------------------------------------- critic loss
def test_critic_loss_hand_cases():
    # eps = 0.2, target 1.0. token 0: inside the band (both branches equal, no clip flag);
    # token 1: value moved towards the target beyond the band -> clipped branch is larger;
    # token 2: value moved away beyond the band -> original branch is larger.
    value = torch.tensor([0.6, 0.9, 0.1], requires_grad=True)
    old = torch.tensor([0.5, 0.5, 0.5])
    target = torch.tensor([1.0, 1.0, 1.0])
    loss, stat = A.critic_loss(value, old, target, 0.2)
    per = torch.tensor([0.5 * 0.4**2, 0.5 * 0.3**2, 0.5 * 0.9**2])
    torch.testing.assert_close(stat["loss"], per, rtol=1e-6, atol=0)
    assert stat["clip_mask"].tolist() == [False, True, False]
    assert abs(loss.item() - per.mean().item()) < 1e-7
    loss.backward()
    # ties split the gradient; the clipped branch outside the band has no gradient
    torch.testing.assert_close(value.grad, torch.tensor([(0.6 - 1.0) / 3, 0.0, (0.1 - 1.0) / 3]), rtol=1e-6, atol=1e-8)


def test_critic_loss_huber_and_mask():
    value = torch.tensor([0.0, 20.0, 3.0])
    old = value.clone()
    target = torch.tensor([1.0, 0.0, 3.0])
    mask = torch.tensor([True, True, False])
    loss, stat = A.critic_loss(value, old, target, 0.5, mask, "huber")
    # |diff| = 1 -> 0.5; |diff| = 20 >= 10 -> 10 * (20 - 5) = 150
    torch.testing.assert_close(stat["loss"], torch.tensor([0.5, 150.0, 0.0]))
    assert abs(loss.item() - 150.5 / 2) < 1e-5
    with pytest.raises(NotImplementedError):
        A.critic_loss(value, old, target, 0.5, mask, "l1")


# ---------------------------------------------------------------- DPO
def test_dpo_pair_logratios_brute_force():
    g = torch.Generator().manual_seed(1)
    lens = [5, 3, 1, 4, 6, 2]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    n = int(cu[-1])
    lp, ref = torch.randn(n, generator=g), torch.randn(n, generator=g)
    mask = torch.rand(n, generator=g) > 0.3
    valid = torch.tensor([True, False, True])
    pol, rf, ln = A.dpo_pair_logratios(lp, ref, cu, mask, valid)
    want_p, want_r, want_n = [], [], []
    for s in range(len(lens)):
        a, b = int(cu[s]), int(cu[s + 1])
        sp = sr = 0.0
        c = 0
        for t in range(a, b - 1):          # the last token of a sequence has no next token
            if mask[t + 1]:
                sp += float(lp[t]); sr += float(ref[t]); c += 1
        want_p.append(sp); want_r.append(sr); want_n.append(float(c))
    pick = lambda v: torch.tensor(v, dtype=torch.float64).view(-1, 2)[valid]
    torch.testing.assert_close(pol, pick(want_p), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(rf, pick(want_r), rtol=1e-12, atol=1e-12)
    assert torch.equal(ln, pick(want_n))
    assert pol.shape == (2, 2)


def test_dpo_preference_loss_closed_forms():
    x = torch.tensor([0.0, 2.0, -1.0])
    torch.testing.assert_close(A.dpo_preference_loss(x, beta=0.5),
                               torch.log1p(torch.exp(-0.5 * x)), rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(A.dpo_preference_loss(x, beta=0.5, loss_type="ipo"), (x - 1.0) ** 2)
    with pytest.raises(ValueError):
        A.dpo_preference_loss(x, beta=0.5, loss_type="hinge")


# ---------------------------------------------------------------- M2PO mask
def test_m2po_mask_hand_cases():
    old = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.0])
    prox = torch.tensor([1.0, 2.0, 3.0, 0.5, 9.0])   # m2 = 1, 4, 9, 0.25, 81
    mask = torch.tensor([True, True, True, True, False])
    # means of the suffixes (descending 9, 4, 1, 0.25): 3.5625, 1.75, 0.625, 0.25
    assert A.m2po_mask(old, prox, mask, 4.0).tolist() == [True, True, True, True, False]
    assert A.m2po_mask(old, prox, mask, 2.0).tolist() == [True, True, False, True, False]
    assert A.m2po_mask(old, prox, mask, 0.7).tolist() == [True, False, False, True, False]
    assert A.m2po_mask(old, prox, mask, 0.3).tolist() == [False, False, False, True, False]
    # no suffix mean below the threshold: all but the smallest are dropped
    assert A.m2po_mask(old, prox, mask, 0.1).tolist() == [False, False, False, True, False]
    none = torch.zeros(5, dtype=torch.bool)
    assert A.m2po_mask(old, prox, none, 1.0) is none


def test_m2po_mask_is_the_largest_prefix_with_mean_below_threshold():
    g = torch.Generator().manual_seed(2)
    for thr in (0.005, 0.02, 0.05, 1.0):
        old = torch.randn(4, 50, generator=g) * 0.2
        prox = old + torch.randn(4, 50, generator=g) * 0.15
        mask = torch.rand(4, 50, generator=g) > 0.3
        out = A.m2po_mask(old, prox, mask, thr)
        assert out.shape == mask.shape and not (out & ~mask).any()
        m2 = ((old - prox) ** 2)[mask].double().sort().values
        means = m2.cumsum(0) / torch.arange(1, m2.numel() + 1)
        ok = (means < thr).nonzero()
        want_kept = int(ok[-1]) + 1 if len(ok) else 1
        assert int(out.sum()) == want_kept
        kept = ((old - prox) ** 2)[out]
        dropped = ((old - prox) ** 2)[mask & ~out]
        assert dropped.numel() == 0 or kept.max() <= dropped.min()


# ---------------------------------------------------------------- proximal approximations
def test_prox_approximation_reference_literals():
    # reference tests/test_prox_approx.py:24-186
    old = torch.tensor([[-1.0, -2.0, -3.0]])
    new = torch.tensor([[-1.5, -2.5, -3.5]])
    a = A.prox_logp_approximations(old, new, torch.tensor([[0, 0, 0]], dtype=torch.int32), 2)
    torch.testing.assert_close(a["loglinear"], torch.tensor([[-1.25, -2.25, -3.25]]), rtol=1e-4, atol=1e-4)
    assert torch.equal(a["rollout"], old) and set(a) == {"loglinear", "linear", "rollout"}
    a = A.prox_logp_approximations(torch.tensor([[-1.0], [-2.0]]), torch.tensor([[-1.5], [-2.2]]),
                                   torch.tensor([[0], [2]], dtype=torch.int32), 4)
    torch.testing.assert_close(a["loglinear"], torch.tensor([[-1.375], [-2.1]]), rtol=1e-4, atol=1e-4)
    one = torch.tensor([[-1.0]])
    for ver, cur in ((4, 5), (3, 3)):   # behaviour == proximal; behaviour == current (0/0)
        a = A.prox_logp_approximations(one, torch.tensor([[-2.0]]), torch.tensor([[ver]], dtype=torch.int32), cur)
        torch.testing.assert_close(a["loglinear"], one, rtol=1e-4, atol=1e-4)
    a = A.prox_logp_approximations(torch.tensor([[-0.693]]), torch.tensor([[-1.386]]),
                                   torch.tensor([[0]], dtype=torch.int32), 2)
    torch.testing.assert_close(a["linear"], torch.log(torch.tensor([[0.375]])), rtol=1e-3, atol=1e-3)
    a = A.prox_logp_approximations(old, new, torch.tensor([[-1, 0, 1]], dtype=torch.int32), 3, "loglinear")
    assert a["loglinear"][0, 0] == old[0, 0] and torch.isfinite(a["loglinear"]).all() and list(a) == ["loglinear"]


def test_distill_loss_hand_cases():
    lp = torch.tensor([-1.0, -2.0, -0.5], requires_grad=True)
    old = torch.tensor([-1.0, -1.5, -0.5])
    teacher = torch.tensor([-0.5, -1.0, -9.0])
    mask = torch.tensor([True, True, False])
    base = (lp * torch.tensor([1.0, 0.0, 0.0])).sum()          # a stand-in RL loss: -1.0
    loss, stat = A.distill_loss(base, lp, old, teacher, mask, 2.0, 0.1)
    # penalty = ((-1 + 0.5) + (-2 + 1)) / 2 = -0.75; loss = 2 * (-1) + 0.1 * (-0.75)
    assert abs(loss.item() - (-2.075)) < 1e-6 and stat.tolist() == [-0.5, -1.0, 0.0]
    loss.backward()
    torch.testing.assert_close(lp.grad, torch.tensor([2.0 + 0.05, 0.05, 0.0]))
    lp.grad = None
    loss, stat = A.distill_loss(base, lp, old, teacher, mask, 0, 0.1)
    # term = exp(lp - old) * (teacher - lp): [1 * 0.5, exp(-0.5) * 1.0]
    t1 = math.exp(-0.5)
    assert abs(loss.item() - (-0.1 * (0.5 + t1) / 2)) < 1e-6
    torch.testing.assert_close(stat, torch.tensor([-0.5, -t1, 0.0]))
    loss.backward()
    torch.testing.assert_close(lp.grad, torch.tensor([-0.1 * 0.5 / 2, -0.1 * t1 / 2, 0.0]))
