"""Pins the GAE and normalisation oracles with the reference tests' literals and closed forms."""

import math

import pytest
import torch

from oracle import gae as G
from oracle import norm as N


def _t(x, dtype=torch.float32):
    return torch.tensor(x, dtype=dtype)


def test_gae_per_sample_lambda_literals():
    # reference tests/test_ppo_gae.py:196-221, atol = 0
    rewards = _t([[0.0, 0.0, 1.0, 0.0]] * 2)
    mask = _t([[1.0, 1.0, 1.0, 0.0]] * 2)
    adv, _ = G.gae_padded(rewards, torch.zeros_like(rewards), mask, torch.tensor([False, False]), 1.0,
                          _t([0.5, 0.0]))
    assert torch.equal(adv, _t([[0.25, 0.5, 1.0, 0.0], [0.0, 0.0, 1.0, 0.0]]))


def test_gae_closed_form_unmasked():
    """A_t = sum_k (gamma*lambda)^k delta_{t+k}, delta_t = r_t + gamma V_{t+1} - V_t."""
    torch.manual_seed(0)
    L, gamma, lam = 12, 0.9, 0.8
    r = torch.randn(1, L, dtype=torch.float64)
    v = torch.randn(1, L, dtype=torch.float64)
    adv, ret = G.gae_padded(r.float(), v.float(), torch.ones(1, L), torch.tensor([True]), gamma, lam)
    want = torch.zeros(L, dtype=torch.float64)
    for t in range(L - 1):
        acc = 0.0
        for k in range(L - 1 - t):
            nv = v[0, t + k + 1]
            acc += (gamma * lam) ** k * (r[0, t + k] + gamma * nv - v[0, t + k])
        want[t] = acc
    torch.testing.assert_close(adv[0].double(), want, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(ret, adv + v.float())


def test_gae_no_bootstrap_when_sequence_ended():
    r = _t([[0.0, 0.0, 1.0, 0.0]])
    v = _t([[0.5, 0.5, 0.5, 9.0]])
    a_eos, _ = G.gae_padded(r, v, torch.ones(1, 4), torch.tensor([False]), 1.0, 1.0)
    a_trunc, _ = G.gae_padded(r, v, torch.ones(1, 4), torch.tensor([True]), 1.0, 1.0)
    # with gamma = lambda = 1: A_t = sum r + V_boot - V_t
    assert torch.equal(a_eos, _t([[0.5, 0.5, 0.5, 0.0]]))
    assert torch.equal(a_trunc, _t([[9.5, 9.5, 9.5, 0.0]]))


def test_gae_masked_positions_carry_state():
    r = _t([[0.0, 5.0, 0.0, 2.0, 0.0]])
    v = _t([[0.1, 0.2, 0.3, 0.4, 0.0]])
    m = _t([[1.0, 0.0, 0.0, 1.0, 0.0]])
    adv, _ = G.gae_padded(r, v, m, torch.tensor([False]), 0.9, 0.8)
    assert adv[0, 1] == adv[0, 2] == adv[0, 3]  # masked tokens repeat the advantage to their right
    assert adv[0, 3].item() == pytest.approx(2.0 - 0.4)
    # the masked reward 5.0 never enters
    assert adv[0, 0].item() == pytest.approx((0.0 + 0.9 * 0.4 - 0.1) + 0.72 * 1.6, rel=1e-6)


def test_gae_packed_equals_padded():
    """The packed recurrence equals the reference's padded one on the same data, given what the
    reference's data guarantees: mask 0 on padding and on each sequence's last token (the loss
    mask is rolled by -1, actor.py:214-215)."""
    torch.manual_seed(1)
    lens = [5, 1, 9, 3]
    L = max(lens)
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    T = sum(lens)
    r, v = torch.randn(T), torch.randn(T)
    m = (torch.rand(T) > 0.3).float()
    m[cu[1:].long() - 1] = 0.0
    no_eos = torch.tensor([False, False, True, False])  # only the full-width row may bootstrap
    lam = _t([0.95, 0.5, 0.9, 1.0])
    adv_p, ret_p = G.gae_packed(r, v, m, cu, no_eos, 0.99, lam)
    rp, vp, mp = torch.zeros(4, L), torch.zeros(4, L), torch.zeros(4, L)
    for i, n in enumerate(lens):
        s = int(cu[i])
        rp[i, :n], vp[i, :n], mp[i, :n] = r[s:s + n], v[s:s + n], m[s:s + n]
    adv_d, ret_d = G.gae_padded(rp, vp, mp, no_eos, 0.99, lam)
    for i, n in enumerate(lens):
        s = int(cu[i])
        assert torch.equal(adv_p[s:s + n], adv_d[i, :n])
        assert torch.equal(ret_p[s:s + n], ret_d[i, :n])


def test_norm_leave_one_out_literals():
    # reference tests/test_adv_norm_config.py:730-749
    x = _t([[1.0], [2.0], [3.0], [4.0]])
    out = N.normalization(x, torch.ones_like(x), mean_level="batch", std_level=None, mean_leave1out=True)
    torch.testing.assert_close(out, _t([[-2.0], [-2.0 / 3], [2.0 / 3], [2.0]]), atol=1e-6, rtol=0)
    # :800-810
    x = _t([[0.0, 0.0], [1.0, 0.0], [0.0, 0.0]])
    out = N.normalization(x, torch.ones_like(x), mean_level="batch", std_level=None, mean_leave1out=True)
    torch.testing.assert_close(out, _t([[-0.2, -0.2], [1.0, -0.2], [-0.2, -0.2]]), atol=1e-4, rtol=0)


def test_norm_masked_batch_literals():
    # reference tests/test_adv_norm_config.py:1102-1152: mean 5.0, biased-sample std property
    x = _t([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0], [7.0, 8.0, 9.0]])
    m = _t([[1.0, 1.0, 0.0], [1.0, 0.0, 1.0], [0.0, 1.0, 1.0]])
    out = N.normalization(x, m, mean_level="batch", std_level="batch", group_size=1)
    assert out[0, 2] == 0 and out[1, 1] == 0 and out[2, 0] == 0
    vals = out[m.bool()]
    assert abs(vals.mean().item()) < 1e-5
    assert abs(vals.std().item() - 1.0) < 1e-5
    std = math.sqrt(52 / 5)  # unbiased (default) over the six active values
    torch.testing.assert_close(out[0, 0], _t((1 - 5) / (std + 1e-5)), rtol=1e-5, atol=1e-6)


def test_norm_masked_leave_one_out_literals():
    # reference tests/test_adv_norm_config.py:1209-1224
    x = _t([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]])
    m = _t([[1.0, 1.0], [1.0, 0.0], [0.0, 1.0]])
    out = N.normalization(x, m, mean_level="batch", std_level="batch", mean_leave1out=True, std_unbiased=True)
    for got, want in [(out[0, 0], -0.9258), (out[0, 1], -0.4629), (out[1, 0], 0.0), (out[2, 1], 1.3887)]:
        assert got.item() == pytest.approx(want, abs=1e-3)
    assert out[1, 1] == 0 and out[2, 0] == 0


def test_norm_unbiased_ratio():
    # reference tests/test_adv_norm_config.py:752-780
    x = _t([[1.0], [2.0], [3.0]])
    m = torch.ones_like(x)
    b = N.normalization(x, m, mean_level="batch", std_level="batch", std_unbiased=False)
    u = N.normalization(x, m, mean_level="batch", std_level="batch", std_unbiased=True)
    assert (b.std() / u.std()).item() == pytest.approx(math.sqrt(1.5), abs=1e-4)


def test_norm_variable_groups():
    # reference tests/test_reward_norm_variable_group.py:28-64
    x = _t([0.0, 3.0, 6.0, 10.0, 20.0, 1.0, 2.0, 3.0])
    sizes = [3, 2, 3]
    out = N.normalization(x, None, mean_level="group", std_level="group", group_size=2,
                          std_unbiased=False, eps=0.0, group_sizes=sizes)
    off = 0
    for s in sizes:
        c = x[off:off + s].double()
        want = (c - c.mean()) / c.std(unbiased=False)
        torch.testing.assert_close(out[off:off + s].double(), want, rtol=1e-5, atol=1e-5)
        off += s
    a = N.normalization(_t([0.0, 2.0, 10.0, 14.0]), None, mean_level="group", std_level="group", group_size=2,
                        std_unbiased=False, eps=0.0)
    b = N.normalization(_t([0.0, 2.0, 10.0, 14.0]), None, mean_level="group", std_level="group", group_size=2,
                        std_unbiased=False, eps=0.0, group_sizes=[2, 2])
    torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-6)


def test_norm_zero_variance_and_singleton():
    # reference tests/test_reward_norm_variable_group.py:78-127
    out = N.normalization(_t([0.0, 3.0, 6.0, 5.0, 5.0]), None, mean_level="group", std_level="group",
                          group_size=2, std_unbiased=False, eps=1e-5, group_sizes=[3, 2])
    assert torch.isfinite(out).all() and (out[3:] == 0).all()
    out = N.normalization(_t([7.0, 1.0, 5.0]), None, mean_level="group", std_level="group", group_size=1,
                          mean_leave1out=True, std_unbiased=True, eps=1e-5, group_sizes=[1, 2])
    assert torch.isfinite(out).all() and out[0].item() == 0.0


def test_norm_errors_and_all_masked():
    x = _t([0.0, 1.0, 2.0, 3.0])
    with pytest.raises(ValueError, match="must equal"):
        N.normalization(x, None, mean_level="group", std_level="group", group_size=2, group_sizes=[3, 2])
    with pytest.raises(ValueError, match="positive"):
        N.normalization(x, None, mean_level="group", std_level="group", group_size=2, group_sizes=[4, 0])
    out = N.normalization(x, torch.zeros(4))
    assert torch.equal(out, x)


def test_norm_tail_rows_divide_by_eps():
    # fixed group_size leaves bs % group_size rows with mean 0 / std 0 (data.py:1405-1410)
    x = _t([1.0, 3.0, 5.0])
    out = N.normalization(x, None, mean_level="group", std_level="group", group_size=2, eps=1e-5)
    assert out[2].item() == pytest.approx(5.0 / 1e-5, rel=1e-5)


def test_masked_normalization_closed_form():
    torch.manual_seed(0)
    x = torch.randn(50) * 3 + 2
    m = (torch.rand(50) > 0.4).float()
    out = N.masked_normalization(x, m, unbiased=False, eps=1e-5)
    act = x[m.bool()].double()
    want = ((x.double() * m.double()) - act.mean()) / (act.std(unbiased=False) + 1e-5)
    torch.testing.assert_close(out.double(), want, rtol=1e-5, atol=1e-6)


def test_masked_normalization_dim_is_per_slice():
    # dim = the reduced dimensions: each slice along the others is whitened by itself (brute force
    # per row / per column with torch's own mean and std of the active elements)
    torch.manual_seed(1)
    x = torch.randn(5, 40) * 2 + 1
    m = (torch.rand(5, 40) > 0.3).float()
    out = N.masked_normalization(x, m, unbiased=True, eps=1e-5, dim=-1)
    for r in range(5):
        act = x[r][m[r].bool()].double()
        want = (x[r].double() * m[r].double() - act.mean()) / (act.std(unbiased=True) + 1e-5)
        torch.testing.assert_close(out[r].double(), want, rtol=1e-5, atol=1e-6)
    out0 = N.masked_normalization(x, None, dim=(0,))
    for c in range(40):
        col = x[:, c].double()
        torch.testing.assert_close(out0[:, c].double(), (col - col.mean()) / (col.std(unbiased=False) + 1e-5),
                                   rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- turn-level GAE
def test_turn_level_gae_reference_literals():
    # reference tests/test_ppo_gae.py:81-151 (inputs and expected values re-typed)
    r = torch.tensor([[0.0, 1.0, 0.0, 2.0]])
    a, rt = G.gae_turn_level(r, torch.zeros_like(r), torch.ones_like(r), torch.tensor([[0, 0, 1, 1]], dtype=torch.int32),
                             torch.tensor([False]), 1.0, 0.5)
    assert torch.equal(a, torch.tensor([[2.0, 2.0, 2.0, 2.0]])) and torch.equal(rt, a)
    r = torch.tensor([[0.0, 3.0, 0.0, 0.0, 4.0]])
    v = torch.tensor([[1.0, 5.0, 9.0, 2.0, 8.0]])
    a, rt = G.gae_turn_level(r, v, torch.tensor([[1.0, 1.0, 0.0, 1.0, 1.0]]), torch.tensor([[0, 0, -1, 2, 2]]),
                             torch.tensor([True]), 0.5, 0.25)
    assert torch.equal(a, torch.tensor([[3.75, 3.75, 0.0, 6.0, 6.0]]))
    assert torch.equal(rt, torch.tensor([[4.75, 4.75, 9.0, 8.0, 8.0]]))
    r = torch.tensor([[0.0, 1.0, 0.0, 2.0], [0.0, 1.0, 0.0, 2.0]])
    a, _ = G.gae_turn_level(r, torch.zeros_like(r), torch.ones_like(r),
                            torch.tensor([[0, 0, 1, 1], [0, 0, 1, 1]], dtype=torch.int32),
                            torch.tensor([False, False]), 1.0, torch.tensor([0.5, 0.0]))
    assert torch.equal(a, torch.tensor([[2.0, 2.0, 2.0, 2.0], [1.0, 1.0, 2.0, 2.0]]))


@pytest.mark.parametrize("ids,message", [([-1, 0, 0, 1], "non-negative"), ([0, 0, 4, 4], "smaller than the sequence length"),
                                         ([0, 1, 0, 2], "temporally nondecreasing")])
def test_turn_level_gae_rejects_malformed_ids(ids, message):
    # reference tests/test_ppo_gae.py:511-532
    r = torch.zeros(1, 4)
    with pytest.raises(RuntimeError, match=message):
        G.gae_turn_level(r, r, torch.ones_like(r), torch.tensor([ids]), torch.tensor([False]), 1.0, 1.0)
    with pytest.raises(ValueError, match="integer dtype"):
        G.gae_turn_level(r, r, torch.ones_like(r), torch.zeros(1, 4), torch.tensor([False]), 1.0, 1.0)


def test_turn_level_gae_with_one_token_turns_is_token_level_gae():
    # every active token its own turn: the turn recurrence is the token recurrence over the
    # active tokens (value of the next ACTIVE token), which gae_padded computes as well
    g = torch.Generator().manual_seed(4)
    bs, L = 3, 40
    r, v = torch.randn(bs, L, generator=g), torch.randn(bs, L, generator=g)
    m = (torch.rand(bs, L, generator=g) > 0.3).float()
    m[:, -1] = 0
    ids = torch.arange(L).expand(bs, -1).clone()
    ne = torch.tensor([True, False, True])
    a, _ = G.gae_turn_level(r, v, m, ids, ne, 0.9, 0.8)
    want, _ = G.gae_padded(r, v, m, ne, 0.9, 0.8)
    torch.testing.assert_close(a, want * m, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- reward shaping before GAE
def test_kl_estimators_closed_forms():
    from oracle import advantages as ADV

    a = torch.tensor([-1.0, -2.0, -0.5, -30.0])
    b = torch.tensor([-1.5, -1.0, -0.5, -1.0])
    d = a - b  # 0.5, -1.0, 0.0, -29.0
    assert torch.equal(ADV.approx_kl(a, b, "k1"), torch.tensor([0.5, -1.0, 0.0, -10.0]))
    assert torch.equal(ADV.approx_kl(a, b, "k1", apply_clamp=False), d)
    assert torch.equal(ADV.approx_kl(a, b, "k2"), torch.tensor([0.125, 0.5, 0.0, 10.0]))
    k3 = ADV.approx_kl(a, b, "k3", apply_clamp=False)
    want = torch.tensor([math.exp(-0.5) - 1 + 0.5, math.e - 2.0, 0.0, math.exp(29.0) - 1 - 29.0])
    torch.testing.assert_close(k3, want, rtol=1e-6, atol=1e-7)
    with pytest.raises(ValueError, match="Invalid KL estimator"):
        ADV.approx_kl(a, b, "k4")


def test_shape_rewards_hand_computed():
    from oracle import advantages as ADV

    # row 0: 4 tokens then padding; row 1: full (no EOS); row 2: empty
    attn = torch.tensor([[1, 1, 1, 1, 0], [1, 1, 1, 1, 1], [0, 0, 0, 0, 0]])
    loss_mask = torch.tensor([[0, 1, 1, 1, 0], [0, 0, 1, 1, 1], [0, 0, 0, 0, 0]])
    logp = torch.tensor([[-1.0, -2.0, -3.0, -4.0, -5.0]] * 3)
    ref = torch.tensor([[-1.0, -1.0, -1.0, -1.0, -1.0]] * 3)
    score = torch.tensor([2.0, 3.0, 4.0])
    out = ADV.shape_rewards(loss_mask, attn, logp, ref, score, kl_ctl=0.5)
    # rolled mask: row 0 -> [1,1,1,0,0]; row 1 -> [0,1,1,1,0]
    assert out["loss_mask"].tolist() == [[1, 1, 1, 0, 0], [0, 1, 1, 1, 0], [0, 0, 0, 0, 0]]
    # old = roll(logp) * mask = [-2,-3,-4,0,0]; ref * mask = [-1,-1,-1,0,0]; kl = -0.5 * (old - ref)
    assert out["old_logp"][0].tolist() == [-2.0, -3.0, -4.0, 0.0, 0.0]
    assert out["kl_rewards"][0].tolist() == [0.5, 1.0, 1.5, 0.0, 0.0]
    # zero at seqlen - 1 = 3 (already 0), outcome at seqlen - 2 = 2
    assert out["tot_rewards"][0].tolist() == [0.5, 1.0, 3.5, 0.0, 0.0]
    # row 1: kl = [0, 1.0, 1.5, 2.0, 0]; zero at 4; outcome 3.0 at 3
    assert out["tot_rewards"][1].tolist() == [0.0, 1.0, 1.5, 5.0, 0.0]
    assert out["seq_no_eos_mask"].tolist() == [False, True, False]
    # empty row: index -1 zeroes the last slot, the outcome lands at 0
    assert out["tot_rewards"][2].tolist() == [4.0, 0.0, 0.0, 0.0, 0.0]
    out = ADV.shape_rewards(loss_mask, attn, logp, ref, score, kl_ctl=0.5, mask_no_eos_with_zero=True)
    assert out["tot_rewards"][1].tolist() == [0.0, 1.0, 1.5, 2.0, 0.0]  # truncated row: no outcome
    out = ADV.shape_rewards(loss_mask, attn, logp, None, score, kl_ctl=0.5, roll_logp=False)
    assert out["old_logp"][0].tolist() == [-1.0, -2.0, -3.0, 0.0, 0.0]  # not rolled, no reference
    assert out["kl_rewards"][0].tolist() == [0.5, 1.0, 1.5, 0.0, 0.0]

