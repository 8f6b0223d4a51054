"""HIP SAPO / critic / DPO kernels through the C ABI against the reference's literals and the
CPU oracle (loss <= 1e-4 rel, masks bit-exact, gradients against the oracle's autograd)."""

import pytest
import torch

from areal_amd.functional import (
    dpo_pair_logratios,
    dpo_preference_loss,
    ppo_critic_loss_fn,
    sapo_loss_fn,
)
from oracle import aux_loss as A

pytestmark = pytest.mark.gpu


def test_sapo_reference_literals(dev):
    # tests/test_functional.py:923-954 and :1160-1195 of the reference
    lp = torch.tensor([[1.0, 1.0]], device=dev)
    loss, stat = sapo_loss_fn(lp, lp.clone(), torch.ones(1, 2, device=dev), 1.0, 1.0,
                              torch.ones(1, 2, dtype=torch.bool, device=dev))
    assert loss.ndim == 0 and loss.dtype == torch.float32
    assert abs(loss.item() + 2.0) < 1e-5
    assert torch.allclose(stat["sapo_soft_gate"].cpu(), torch.tensor([[2.0, 2.0]]), atol=1e-5)
    grads = []
    for tau in (1.0, 2.0):
        x = torch.zeros(1, 1, device=dev, requires_grad=True)
        l, _ = sapo_loss_fn(x, torch.zeros(1, 1, device=dev), torch.ones(1, 1, device=dev), tau, tau,
                            torch.ones(1, 1, dtype=torch.bool, device=dev))
        l.backward()
        grads.append(x.grad.item())
    assert abs(grads[0] - grads[1]) < 1e-6 and abs(grads[0] + 1.0) < 1e-6
    with pytest.raises(ValueError, match="must be positive"):
        sapo_loss_fn(lp, lp, lp, 0.0, 1.0, torch.ones(1, 2, dtype=torch.bool, device=dev))
    with pytest.raises(ValueError, match="Invalid importance_sampling_level"):
        sapo_loss_fn(lp, lp, lp, 1.0, 1.0, torch.ones(1, 2, dtype=torch.bool, device=dev), "turn")
    with pytest.raises(ValueError, match="cu_seqlens is required"):
        sapo_loss_fn(lp[0], lp[0], lp[0], 1.0, 1.0, torch.ones(2, dtype=torch.bool, device=dev), "sequence")


@pytest.mark.parametrize("level", ["token", "sequence"])
@pytest.mark.parametrize("layout", ["packed", "padded"])
def test_sapo_matches_oracle(dev, level, layout):
    g = torch.Generator().manual_seed(11)
    if layout == "packed":
        lens = torch.randint(1, 400, (37,), generator=g)
        cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32)
        shape = (int(cu[-1]),)
    else:
        cu, shape = None, (24, 300)
    lp = (torch.randn(shape, generator=g) * 0.3 - 1.0)
    old = lp + torch.randn(shape, generator=g) * 0.2
    adv = torch.randn(shape, generator=g)
    adv.view(-1)[::17] = 0.0
    mask = torch.rand(shape, generator=g) > 0.25
    if layout == "padded":
        mask[3] = False  # an all-masked row
    lp_c = lp.clone().requires_grad_(True)
    want, ws = A.sapo_loss(lp_c, old, adv, 1.0, 1.05, mask, level, cu)
    want.backward()
    x = lp.to(dev).requires_grad_(True)
    loss, stat = sapo_loss_fn(x, old.to(dev), adv.to(dev), 1.0, 1.05, mask.to(dev), level,
                              cu.to(dev) if cu is not None else None)
    loss.backward()
    torch.testing.assert_close(loss.detach().cpu(), want.detach(), rtol=1e-4, atol=1e-7)
    for key, okey in (("loss", "loss"), ("importance_weight", "importance_weight"), ("approx_kl", "approx_kl"),
                      ("sapo_soft_gate", "sapo_soft_gate"), ("sapo_scaled_gate_pos", "sapo_scaled_gate_pos"),
                      ("sapo_scaled_gate_neg", "sapo_scaled_gate_neg")):
        assert stat[key].shape == shape
        torch.testing.assert_close(stat[key].cpu(), ws[okey], rtol=2e-5, atol=1e-6)
    assert not stat["clip_mask"].any() and not stat["dual_clip_mask"].any()
    torch.testing.assert_close(x.grad.cpu(), lp_c.grad, rtol=1e-4, atol=1e-8)


@pytest.mark.parametrize("n,level", [(70_001, "token"), (300_003, "token"), (70_001, "sequence")])
def test_sapo_reduced_stats_match_oracle_masked_stats(dev, n, level):
    """grpo_loss_fn(use_sapo_loss=True, stats_mode="reduced") writes no per-token statistic
    tensor; what it reports equals the oracle's per-token SAPO tensors (assembled as
    actor.py:662-741 hands them to the tracker) reduced by oracle.packing.masked_stats. The larger
    batch takes the four-tokens-per-thread form of the kernel."""
    from areal_amd.ppo.actor import grpo_loss_fn
    from oracle.packing import masked_stats as oracle_masked_stats

    g = torch.Generator().manual_seed(n)
    lens = torch.randint(1, n // 40, (40,), generator=g)
    lens[-1] = n - int(lens[:-1].sum())  # 40 sequences that cover the n tokens
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32)
    assert int(cu[-1]) == n
    lp = torch.randn(n, generator=g) * 0.3 - 1.0
    old = lp + torch.randn(n, generator=g) * 0.2
    adv = torch.randn(n, generator=g)
    mask = torch.rand(n, generator=g) > 0.25
    ent = torch.rand(n, generator=g) * 3
    vmin, vmax = -torch.rand(n, generator=g) * 9 - 3, torch.rand(n, generator=g) * 20
    lp_c = lp.clone().requires_grad_(True)
    want_loss, so = A.sapo_loss(lp_c, old, adv, 1.0, 1.05, mask, level, cu)
    want_loss.backward()
    lpd = lp_c.detach()
    diff = (old - lpd) * mask
    zeros = torch.zeros(n)
    vals = dict(importance_weight=so["importance_weight"], approx_kl=so["approx_kl"], new_logp=lpd, old_logp=old,
                entropy=ent, actor_loss=so["loss"], clip_ratio=zeros, dual_clip_ratio=zeros, logp_diff=diff,
                logp_abs_diff=diff.abs(), sapo_soft_gate=so["sapo_soft_gate"],
                sapo_scaled_gate_pos=so["sapo_scaled_gate_pos"], sapo_scaled_gate_neg=so["sapo_scaled_gate_neg"],
                vocab_min_logits=vmin, vocab_max_logits=vmax)
    den = {k: mask for k in vals}
    den["vocab_min_logits"] = den["vocab_max_logits"] = None
    want = oracle_masked_stats(vals, den)

    stats = {}
    x = lp.to(dev).requires_grad_(True)
    data = dict(logprobs=old.to(dev), advantages=adv.to(dev), loss_mask=mask.to(dev), cu_seqlens=cu.to(dev),
                prox_logp=old.to(dev))
    loss = grpo_loss_fn(x, ent.to(dev), data, 0.2, None, None, use_sapo_loss=True, sapo_tau_pos=1.0,
                        sapo_tau_neg=1.05, importance_sampling_level=level, vocab_min_logits=vmin.to(dev),
                        vocab_max_logits=vmax.to(dev), stats=stats, stats_mode="reduced")
    loss.backward()
    torch.testing.assert_close(loss.detach().cpu(), want_loss.detach(), rtol=1e-4, atol=1e-7)
    torch.testing.assert_close(x.grad.cpu(), lp_c.grad, rtol=1e-4, atol=1e-8)
    assert not any(torch.is_tensor(v) for v in stats.values())  # nothing of token shape comes back
    assert set(want) <= set(stats), sorted(set(want) - set(stats))
    for k, w in want.items():
        got = stats[k]
        assert got["count"] == w["count"], k
        assert got["sum"] == pytest.approx(w["sum"], rel=2e-5, abs=1e-7 * max(1.0, w["count"])), k
        assert got["min"] == pytest.approx(w["min"], rel=2e-6, abs=1e-6), k
        assert got["max"] == pytest.approx(w["max"], rel=2e-6, abs=1e-6), k
    assert stats["denominator/n_valid_tokens"] == float(mask.sum()) and stats["denominator/n_tokens"] == float(n)
    # the compute_logp diagnostics of the tensor mode, reduced under the same mask
    assert stats["compute_logp/prox_logp_gt"]["count"] == float(mask.sum())
    assert stats["compute_logp/prox_logp_gt"]["sum"] == pytest.approx(float(old[mask].double().sum()), rel=1e-6)


def test_reduced_mode_reduces_the_proximal_approximation_diagnostics(dev):
    """stats_mode="reduced" with versions: the compute_logp/... entries of the tensor mode come
    back as reduced values (sum, count, min, max under the behave mask), the staleness scalars
    as they are."""
    from areal_amd.config import RejectionSamplingConfig
    from areal_amd.ppo.actor import grpo_loss_fn
    from areal_amd.stats import masked_stats

    g = torch.Generator().manual_seed(17)
    n = 40_000
    lp = torch.randn(n, generator=g) * 0.3 - 1.0
    prox = lp + torch.randn(n, generator=g) * 0.05
    old = prox + torch.randn(n, generator=g) * 0.3
    ver = torch.randint(-1, 5, (n,), generator=g)
    data = dict(logprobs=old.to(dev), advantages=torch.randn(n, generator=g).to(dev),
                loss_mask=(torch.rand(n, generator=g) > 0.2).to(dev), prox_logp=prox.to(dev), versions=ver.to(dev))
    rs = RejectionSamplingConfig(level="token", action="mask", metric="ratio", lower=0.5, upper=2.0)
    out = {}
    for mode in ("tensors", "reduced"):
        st = {}
        grpo_loss_fn(lp.to(dev).requires_grad_(True), torch.zeros(n, device=dev), data, 0.2, None, None,
                     rejection_sampling=rs, current_version=5, prox_logp_method="metrics", stats=st, stats_mode=mode)
        out[mode] = st
    t, r = out["tensors"], out["reduced"]
    keys = [k for k in t if k.startswith("compute_logp/") and k != "compute_logp/n_valid_tokens"]
    assert "compute_logp/loglinear/abs_error" in keys and "compute_logp/kl_div_taylor" in keys
    want = masked_stats({k: t[k] for k in keys}, {k: t["compute_logp/n_valid_tokens"] for k in keys})
    assert not any(torch.is_tensor(v) for v in r.values())
    for k in keys:
        assert r[k]["count"] == want[k]["count"] == float(t["compute_logp/n_valid_tokens"].sum()), k
        assert r[k]["sum"] == pytest.approx(want[k]["sum"], rel=1e-12) and r[k]["max"] == want[k]["max"], k
    assert r["denominator/compute_logp/n_valid_tokens"] == float(t["unclipped_behave_tokens"].sum())
    for k in t:
        if k.startswith("scalar/version_stats/"):
            assert r[k] == t[k], k


@pytest.mark.parametrize("kind", ["mse", "huber"])
@pytest.mark.parametrize("masked", [True, False])
def test_critic_loss_matches_oracle(dev, kind, masked):
    g = torch.Generator().manual_seed(5)
    shape = (19, 257)
    old = torch.randn(shape, generator=g) * 3
    value = old + torch.randn(shape, generator=g) * 0.5
    target = old + torch.randn(shape, generator=g) * (15.0 if kind == "huber" else 1.0)
    value.view(-1)[:50] = old.view(-1)[:50]          # ties: zero step
    value.view(-1)[50:80] = old.view(-1)[50:80] + 0.2  # exactly on the clip bound
    mask = (torch.rand(shape, generator=g) > 0.3) if masked else None
    v_c = value.clone().requires_grad_(True)
    want, ws = A.critic_loss(v_c, old, target, 0.2, mask, kind)
    want.backward()
    v = value.to(dev).requires_grad_(True)
    loss, stat = ppo_critic_loss_fn(v, old.to(dev), target.to(dev), 0.2, mask.to(dev) if masked else None, kind)
    loss.backward()
    torch.testing.assert_close(loss.detach().cpu(), want.detach(), rtol=1e-4, atol=1e-7)
    assert torch.equal(stat["clip_mask"].cpu(), ws["clip_mask"])
    torch.testing.assert_close(stat["loss"].cpu(), ws["loss"], rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(v.grad.cpu(), v_c.grad, rtol=1e-4, atol=1e-9)
    with pytest.raises(NotImplementedError):
        ppo_critic_loss_fn(v, old.to(dev), target.to(dev), 0.2, None, "l1")
    with pytest.raises(AssertionError):
        ppo_critic_loss_fn(v.double(), old.to(dev), target.to(dev), 0.2)


def test_critic_loss_hand_cases(dev):
    value = torch.tensor([0.6, 0.9, 0.1], device=dev, requires_grad=True)
    loss, stat = ppo_critic_loss_fn(value, torch.full((3,), 0.5, device=dev), torch.ones(3, device=dev), 0.2)
    assert stat["clip_mask"].tolist() == [False, True, False]
    loss.backward()
    torch.testing.assert_close(value.grad.cpu(), torch.tensor([(0.6 - 1.0) / 3, 0.0, (0.1 - 1.0) / 3]),
                               rtol=1e-6, atol=1e-8)


def test_dpo_pair_logratios_matches_oracle(dev):
    g = torch.Generator().manual_seed(8)
    lens = torch.cat([torch.tensor([1, 2, 0, 5]), torch.randint(1, 3000, (36,), generator=g)])
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32)
    n = int(cu[-1])
    lp, ref = -torch.rand(n, generator=g) * 3, -torch.rand(n, generator=g) * 3
    mask = torch.rand(n, generator=g) > 0.4
    valid = torch.rand(20, generator=g) > 0.2
    lp_c = lp.clone().requires_grad_(True)
    wp, wr, wl = A.dpo_pair_logratios(lp_c, ref, cu, mask, valid)
    x = lp.to(dev).requires_grad_(True)
    p, r, l = dpo_pair_logratios(x, ref.to(dev), cu.to(dev), mask.to(dev), valid.to(dev))
    assert p.dtype == torch.float64 and p.shape == wp.shape
    torch.testing.assert_close(p.detach().cpu(), wp.detach(), rtol=1e-12, atol=1e-9)
    torch.testing.assert_close(r.cpu(), wr, rtol=1e-12, atol=1e-9)
    assert torch.equal(l.cpu(), wl)
    # sigmoid DPO loss on the pair deltas, backward to the log-probs
    def dpo(pp, rr):
        logits = (pp[:, 0] - pp[:, 1]) - (rr[:, 0] - rr[:, 1])
        return dpo_preference_loss(logits, beta=0.1).mean()
    dpo(wp, wr).backward()
    dpo(p, r).backward()
    torch.testing.assert_close(x.grad.cpu(), lp_c.grad, rtol=1e-5, atol=1e-9)


# ---------------------------------------------------------------- M2PO mask
def test_m2po_mask_hand_cases(dev):
    from areal_amd.ppo.actor import _apply_m2po_masking

    old = torch.zeros(5, device=dev)
    prox = torch.tensor([1.0, 2.0, 3.0, 0.5, 9.0], device=dev)
    mask = torch.tensor([True, True, True, True, False], device=dev)
    for thr, want in ((4.0, [1, 1, 1, 1, 0]), (2.0, [1, 1, 0, 1, 0]), (0.7, [1, 0, 0, 1, 0]),
                      (0.3, [0, 0, 0, 1, 0]), (0.1, [0, 0, 0, 1, 0])):
        out = _apply_m2po_masking(old, prox, mask, thr)
        assert out.dtype == torch.bool and out.tolist() == [bool(w) for w in want], thr
    none = torch.zeros(5, dtype=torch.bool, device=dev)
    assert not _apply_m2po_masking(old, prox, none, 1.0).any()


@pytest.mark.parametrize("n,thr", [(37, 0.02), (5000, 0.005), (300_000, 0.02), (300_000, 0.0001), (300_000, 5.0)])
def test_m2po_mask_matches_oracle(dev, n, thr):
    from areal_amd.ppo.actor import _apply_m2po_masking

    g = torch.Generator().manual_seed(n)
    old = torch.randn(n, generator=g) * 0.2
    prox = old + torch.randn(n, generator=g) * 0.15
    prox[::7] = old[::7]                       # many exact zeros of m2
    mask = torch.rand(n, generator=g) > 0.3
    want = A.m2po_mask(old, prox, mask, thr)
    got = _apply_m2po_masking(old.to(dev), prox.to(dev), mask.to(dev), thr).cpu()
    # the kept count may differ by the few tokens whose suffix mean is within rounding of the
    # threshold (the oracle accumulates in fp32, the kernel in fp64); the sets are nested
    assert not (got & ~mask).any()
    diff = int((got != want).sum())
    assert diff <= max(2, n // 100_000), diff
    m2 = (old - prox) ** 2
    if (mask & ~got).any():
        assert m2[got].max() <= m2[mask & ~got].min()
    kept_mean = m2[got].double().mean().item()
    assert kept_mean < thr or int(got.sum()) == 1


def test_m2po_ties_at_the_cut_are_kept_in_index_order(dev):
    from areal_amd.ppo.actor import _apply_m2po_masking

    # values 1 (x6) and 0 (x2): threshold 0.7 keeps the zeros and four of the ones
    old = torch.zeros(8, device=dev)
    prox = torch.tensor([1.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0, 1.0], device=dev)
    mask = torch.ones(8, dtype=torch.bool, device=dev)
    out = _apply_m2po_masking(old, prox, mask, 0.7)
    # kept sets of size j have mean (j - 2) / j: below 0.7 up to j = 6
    assert out.tolist() == [True, True, True, True, True, True, False, False]
    # 2-D shapes keep their shape
    out2 = _apply_m2po_masking(old.view(2, 4), prox.view(2, 4), mask.view(2, 4), 0.7)
    assert out2.shape == (2, 4) and out2.view(-1).tolist() == out.tolist()


# ---------------------------------------------------------------- proximal approximations, distillation
def test_prox_approximations_match_reference_literals_and_oracle(dev):
    from areal_amd.ppo.actor import compute_prox_logp_approximations

    old = torch.tensor([[-1.0, -2.0, -3.0]], device=dev)
    new = torch.tensor([[-1.5, -2.5, -3.5]], device=dev)
    a = compute_prox_logp_approximations(old, new, torch.tensor([[0, 0, 0]], dtype=torch.int32, device=dev), 2)
    torch.testing.assert_close(a["loglinear"].cpu(), torch.tensor([[-1.25, -2.25, -3.25]]), rtol=1e-4, atol=1e-4)
    assert torch.equal(a["rollout"], old) and a["linear"].shape == old.shape and a["linear"].dtype == torch.float32
    g = torch.Generator().manual_seed(1)
    o, n = torch.randn(40, 300, generator=g) - 1, torch.randn(40, 300, generator=g) - 1
    ver = torch.randint(-1, 12, (40, 300), generator=g)
    want = A.prox_logp_approximations(o, n, ver, 10)
    got = compute_prox_logp_approximations(o.to(dev), n.to(dev), ver.to(dev), 10)
    for k in want:
        torch.testing.assert_close(got[k].cpu(), want[k], rtol=2e-6, atol=1e-6)
    only = compute_prox_logp_approximations(o.to(dev), n.to(dev), ver.to(dev), 10, "loglinear")
    assert list(only) == ["loglinear"]


@pytest.mark.parametrize("rl_weight", [1.0, 0])
def test_grpo_loss_fn_optional_branches_match_oracle(dev, rl_weight):
    """grpo_loss_fn with the log-linear proximal approximation, M2PO masking and the distillation
    tail, against the same composition of oracle pieces."""
    from areal_amd.ppo.actor import grpo_loss_fn
    from oracle import loss as O

    g = torch.Generator().manual_seed(3)
    n = 5000
    lp = torch.randn(n, generator=g) * 0.3 - 1.0
    old = lp + torch.randn(n, generator=g) * 0.1
    ver = torch.randint(-1, 5, (n,), generator=g)
    adv = torch.randn(n, generator=g)
    mask = torch.rand(n, generator=g) > 0.2
    teacher = lp + torch.randn(n, generator=g) * 0.2
    data = dict(logprobs=old, advantages=adv, loss_mask=mask, prox_logp=None, versions=ver, teacher_logp=teacher,
                rl_loss_weight=rl_weight, distill_loss_weight=0.01)
    x = lp.to(dev).requires_grad_(True)
    stats = {}
    loss = grpo_loss_fn(x, torch.zeros(n, device=dev), {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in data.items()},
                        0.2, None, None, m2_threshold=0.02, current_version=5, prox_logp_method="loglinear", stats=stats)
    loss.backward()
    x_c = lp.clone().requires_grad_(True)
    prox = A.prox_logp_approximations(old, x_c.detach(), ver, 5, "loglinear")["loglinear"]
    m2 = A.m2po_mask(old, prox, mask, 0.02)
    base, _ = O.ppo_actor_loss(x_c, prox, old, adv, 0.2, m2)
    want, rkl = A.distill_loss(base, x_c, old, teacher, m2, rl_weight, 0.01)
    want.backward()
    torch.testing.assert_close(loss.detach().cpu(), want.detach(), rtol=1e-4, atol=1e-7)
    torch.testing.assert_close(x.grad.cpu(), x_c.grad, rtol=1e-4, atol=1e-9)
    torch.testing.assert_close(stats["rkl_loss"].cpu(), rkl.detach(), rtol=1e-5, atol=1e-7)
    assert "compute_logp/loglinear/approx_logp" in stats and "compute_logp/kl_div_dual" in stats
    assert stats["scalar/version_stats/v_proximal"] == 4
    with pytest.raises(ValueError, match="versions not available"):
        grpo_loss_fn(x, torch.zeros(n, device=dev), dict(logprobs=old.to(dev), advantages=adv.to(dev),
                     loss_mask=mask.to(dev), prox_logp=None), 0.2, None, None, prox_logp_method="loglinear")
    # a NaN or Inf among the proximal log-probs is an error, as in the reference (actor.py:924-928)
    bad = old.clone()
    bad[3] = float("inf")
    with pytest.raises(RuntimeError, match="prox_logp contains NaN or Inf"):
        grpo_loss_fn(x, torch.zeros(n, device=dev), dict(logprobs=old.to(dev), advantages=adv.to(dev),
                     loss_mask=mask.to(dev), prox_logp=bad.to(dev)), 0.2, None, None)

