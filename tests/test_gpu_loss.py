"""HIP actor-loss / rejection-sampling kernels against the reference's known answers and the
CPU oracle.  Masks and counts are compared bit-exact; loss within 1e-4 relative; gradients
within 1e-2 relative (measured: ~1e-6)."""

import pytest
import torch

from areal_amd.config import RejectionSamplingConfig
from areal_amd.functional import apply_rejection_sampling, cispo_loss_fn, ppo_actor_loss_fn
from oracle import loss as O
from tests.golden.rejection_cases import BINARY_KL_CASES, CASES

pytestmark = pytest.mark.gpu


def _t(x, dev, dtype=torch.float32):
    return torch.tensor(x, dtype=dtype, device=dev)


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_rejection_sampling_known_answers(dev, case):
    cu = _t(case["cu"], dev, torch.int32) if case["cu"] is not None else None
    r = apply_rejection_sampling(_t(case["prox"], dev), _t(case["old"], dev), _t(case["mask"], dev), cu,
                                 RejectionSamplingConfig(**case["cfg"]))
    assert r.loss_mask.dtype == torch.float32
    assert torch.equal(r.loss_mask.cpu(), torch.tensor(case["exp_mask"]))
    if case["exp_weight"] is not None:
        torch.testing.assert_close(r.behave_imp_weight.cpu(), torch.tensor(case["exp_weight"]), rtol=1e-5, atol=1e-5)
    if case["exp_fraction"] is not None:
        assert r.filtered_fraction == pytest.approx(case["exp_fraction"])
    assert not torch.isnan(r.behave_imp_weight).any()


@pytest.mark.parametrize("case", BINARY_KL_CASES, ids=[c["name"] for c in BINARY_KL_CASES])
def test_binary_kl_cases(dev, case):
    r = apply_rejection_sampling(_t(case["prox"], dev), _t(case["old"], dev), _t(case["mask"], dev),
                                 _t(case["cu"], dev, torch.int32), RejectionSamplingConfig(**case["cfg"]))
    assert torch.equal(r.loss_mask.cpu(), torch.tensor(case["exp_mask"]))


def _random_batch(n, n_seqs, seed, noise=0.3):
    g = torch.Generator().manual_seed(seed)
    torch.manual_seed(seed)
    lp = torch.randn(n, generator=g) * 0.7 - 1.5
    prox = lp + torch.randn(n, generator=g) * 0.2
    old = prox + torch.distributions.Laplace(0.0, noise).sample((n,))
    adv = torch.randn(n, generator=g)
    adv[::23] = 0.0
    mask = torch.rand(n, generator=g) > 0.25
    cuts = torch.sort(torch.randperm(n - 1, generator=g)[: n_seqs - 1] + 1).values
    cu = torch.cat([torch.tensor([0]), cuts, torch.tensor([n])]).to(torch.int32)
    return lp, prox, old, adv, mask, cu


def _guard_band(metric, bounds):
    """Tokens whose metric is within 2 ulp of a bound: where exp/log on CPU and GPU may differ."""
    n = 0
    for b in bounds:
        if b is None:
            continue
        bt = torch.tensor(b, dtype=torch.float32)
        ulp = torch.nextafter(bt, bt + 1) - bt
        n += int(((metric - bt).abs() <= 2 * ulp).sum())
    return n


RS_CONFIGS = [
    dict(level="token", action="mask", metric="ratio", upper=2.0, lower=0.5),
    dict(level="token", action="mask", metric="binary_kl", upper=0.05),
    dict(level="token", action="mask", metric="kl_k1", upper=0.4, lower=-0.4),
    dict(level="token", action="mask", metric="kl_k2", upper=0.1),
    dict(level="token", action="mask", metric="kl_k3", upper=0.1),
    dict(level="token", action="clamp", metric="ratio", upper=1.5, lower=0.7),
    dict(level="sequence", action="mask", metric="ratio", agg="mean", upper=1.05, lower=0.95),
    dict(level="sequence", action="mask", metric="kl_k2", agg="sum", upper=3.0),
    dict(level="sequence", action="mask", metric="kl_k3", agg="max", upper=0.8),
    dict(level="sequence", action="clamp", metric="ratio", agg="mean", upper=1.02),
]


@pytest.mark.parametrize("cfg", RS_CONFIGS, ids=[f'{c["level"]}-{c["action"]}-{c["metric"]}' for c in RS_CONFIGS])
@pytest.mark.parametrize("packed", [True, False], ids=["packed", "padded"])
def test_rejection_sampling_matches_oracle(dev, cfg, packed):
    n, n_seqs = 6000, 24
    lp, prox, old, adv, mask, cu = _random_batch(n, n_seqs, seed=11)
    if not packed:
        prox, old, mask = prox.view(24, 250), old.view(24, 250), mask.view(24, 250)
        cu = None
    maskf = mask.float()
    want = O.rejection_sampling(prox, old, maskf, cu, **cfg)
    got = apply_rejection_sampling(prox.to(dev), old.to(dev), maskf.to(dev), cu.to(dev) if cu is not None else None,
                                   RejectionSamplingConfig(**cfg))
    assert torch.equal(got.loss_mask.cpu(), want.loss_mask)
    torch.testing.assert_close(got.behave_imp_weight.cpu(), want.behave_imp_weight, rtol=2e-6, atol=1e-7)
    assert got.filtered_fraction == pytest.approx(want.filtered_fraction, abs=1e-12)


PPO_VARIANTS = [
    dict(),
    dict(eps_clip_higher=0.28, c_clip=3.0),
    dict(rs=RS_CONFIGS[0]),
    dict(rs=RS_CONFIGS[1], c_clip=2.0),
    dict(rs=RS_CONFIGS[5]),
    dict(rs=RS_CONFIGS[6]),
    dict(level="sequence"),
    dict(level="sequence", rs=RS_CONFIGS[0], eps_clip_higher=0.3),
    dict(level="sequence", rs=RS_CONFIGS[7]),
]


@pytest.mark.parametrize("var", PPO_VARIANTS, ids=[str(i) for i in range(len(PPO_VARIANTS))])
@pytest.mark.parametrize("packed", [True, False], ids=["packed", "padded"])
def test_ppo_loss_matches_oracle(dev, var, packed):
    n, n_seqs = 6000, 24
    lp, prox, old, adv, mask, cu = _random_batch(n, n_seqs, seed=5)
    if not packed:
        lp, prox, old, adv, mask = (t.view(24, 250) for t in (lp, prox, old, adv, mask))
        cu = None
    rs = var.get("rs")
    kw = dict(eps_clip=0.2, eps_clip_higher=var.get("eps_clip_higher"), c_clip=var.get("c_clip"),
              importance_sampling_level=var.get("level", "token"))
    lp_cpu = lp.clone().requires_grad_(True)
    want_loss, want = O.ppo_actor_loss(lp_cpu, prox, old, adv, loss_mask=mask, rejection_sampling_cfg=rs,
                                       cu_seqlens=cu, **kw)
    (want_loss * 1.7).backward()
    lp_gpu = lp.to(dev).requires_grad_(True)
    got_loss, got = ppo_actor_loss_fn(lp_gpu, prox.to(dev), old.to(dev), adv.to(dev), loss_mask=mask.to(dev),
                                      rejection_sampling=RejectionSamplingConfig(**rs) if rs else None,
                                      cu_seqlens=cu.to(dev) if cu is not None else None, **kw)
    (got_loss * 1.7).backward()
    assert got_loss.dtype == torch.float32 and got_loss.ndim == 0
    torch.testing.assert_close(got_loss.cpu(), want_loss.detach(), rtol=1e-4, atol=1e-7)
    for key in ("clip_mask", "dual_clip_mask"):
        assert got[key].dtype == torch.bool and got[key].shape == lp.shape
        assert torch.equal(got[key].cpu(), want[key]), key
    for key in ("loss", "importance_weight", "approx_kl"):
        assert got[key].dtype == torch.float32
        torch.testing.assert_close(got[key].cpu(), want[key], rtol=2e-5, atol=1e-6, msg=key)
    for key in ("n_total_tokens", "n_valid_tokens", "n_masked_tokens", "masked_token_ratio"):
        assert got[key] == want[key], key
    if rs:
        assert torch.equal(got["behave_mask"].cpu(), want["behave_mask"])
        torch.testing.assert_close(got["behave_imp_weight"].cpu(), want["behave_imp_weight"], rtol=2e-6, atol=1e-7)
        torch.testing.assert_close(got["behave_approx_kl"].cpu(), want["behave_approx_kl"], rtol=0, atol=0)
        assert got["filtered_fraction"] == pytest.approx(want["filtered_fraction"], abs=1e-12)
    g_want, g_got = lp_cpu.grad, lp_gpu.grad.cpu()
    assert (g_got[~want["new_mask"]] == 0).all()
    rel = (g_got - g_want).norm() / g_want.norm().clamp_min(1e-30)
    assert rel < 1e-4, f"gradient relative error {rel}"


def test_ppo_gradient_five_cases(dev):
    lr = torch.tensor([0.05, 0.5, 0.5, -0.5, -0.5, 0.0])
    adv = torch.tensor([2.0, 1.0, -1.0, 1.0, -1.0, 3.0])
    lp = torch.tensor([-1.0, -1.5, -0.2, -0.7, -2.0, -1.0])
    prox = lp - lr
    mask = torch.tensor([1, 1, 1, 1, 1, 0], dtype=torch.bool)
    x = lp.to(dev).requires_grad_(True)
    loss, _ = ppo_actor_loss_fn(x, prox.to(dev), prox.to(dev), adv.to(dev), 0.2, mask.to(dev))
    loss.backward()
    r = lr.exp()
    want = torch.tensor([-2.0 * r[0], 0.0, r[2], -r[3], 0.0, 0.0]) / 5
    torch.testing.assert_close(x.grad.cpu(), want, rtol=1e-6, atol=1e-8)


def _cispo_inputs():
    log_ratio = torch.tensor([-2.0, -0.5, 0.0, 0.3, 1.5, 0.1])
    logprobs = torch.tensor([-1.0, -2.0, -0.3, -1.2, -0.7, -2.5])
    adv = torch.tensor([1.0, -2.0, 0.5, 3.0, -1.0, 2.0])
    mask = torch.tensor([1, 1, 1, 1, 1, 0], dtype=torch.bool)
    return logprobs, logprobs - log_ratio, adv, mask, log_ratio


@pytest.mark.parametrize("eps,eps_hi", [(0.2, 0.28), (1.0, 4.0)])
def test_cispo_value_clip_mask_and_gradient(dev, eps, eps_hi):
    lp, prox, adv, mask, lr = _cispo_inputs()
    x = lp.to(dev).requires_grad_(True)
    pl = prox.to(dev).requires_grad_(True)
    loss, stat = cispo_loss_fn(x, pl, adv.to(dev), eps, mask.to(dev), eps_hi)
    ratio = lr.exp()
    rc = ratio.clamp(1 - eps, 1 + eps_hi)
    torch.testing.assert_close(loss.cpu(), torch.where(mask, -rc * adv * lp, 0.0).sum() / 5)
    torch.testing.assert_close(stat["importance_weight"].cpu(), ratio)
    assert torch.equal(stat["clip_mask"].cpu(), (ratio != rc) & mask)
    assert not stat["dual_clip_mask"].any()
    loss.backward()
    torch.testing.assert_close(x.grad.cpu(), torch.where(mask, -rc * adv / 5, 0.0))
    assert pl.grad is None


def test_cispo_decoupled_and_random(dev):
    lp, prox, adv, mask, lr = _cispo_inputs()
    blr = torch.tensor([0.2, -0.4, 0.0, 0.1, -0.3, 0.5])
    old = prox - blr
    x = lp.to(dev).requires_grad_(True)
    rs = RejectionSamplingConfig(level="token", action="clamp", metric="ratio", upper=100.0)
    loss, stat = cispo_loss_fn(x, prox.to(dev), adv.to(dev), 1.0, mask.to(dev), 4.0, old_logprobs=old.to(dev),
                               rejection_sampling=rs)
    rc = lr.exp().clamp(0.0, 5.0)
    torch.testing.assert_close(loss.cpu(), torch.where(mask, -rc * adv * lp * blr.exp(), 0.0).sum() / 5)
    torch.testing.assert_close(stat["behave_imp_weight"].cpu()[mask], blr.exp()[mask])
    assert "behave_mask" in stat and "behave_approx_kl" in stat
    loss.backward()
    torch.testing.assert_close(x.grad.cpu(), torch.where(mask, -rc * adv * blr.exp() / 5, 0.0))
    # random batch with sequence-level rejection (the "sequence-level mean" of config 5)
    lp, prox, old, adv, mask, cu = _random_batch(6000, 24, seed=9)
    cfg = dict(level="sequence", agg="mean", metric="ratio", action="mask", upper=1.05)
    a = lp.clone().requires_grad_(True)
    wl, w = O.cispo_loss(a, prox, adv, 1.0, mask, 4.0, old_logprobs=old, rejection_sampling_cfg=cfg, cu_seqlens=cu)
    wl.backward()
    b = lp.to(dev).requires_grad_(True)
    gl, g = cispo_loss_fn(b, prox.to(dev), adv.to(dev), 1.0, mask.to(dev), 4.0, old_logprobs=old.to(dev),
                          rejection_sampling=RejectionSamplingConfig(**cfg), cu_seqlens=cu.to(dev))
    gl.backward()
    torch.testing.assert_close(gl.cpu(), wl.detach(), rtol=1e-4, atol=1e-7)
    assert torch.equal(g["clip_mask"].cpu(), w["clip_mask"])
    assert torch.equal(g["behave_mask"].cpu(), w["behave_mask"])
    rel = (b.grad.cpu() - a.grad).norm() / a.grad.norm()
    assert rel < 1e-4


def test_all_masked_and_determinism(dev):
    z = torch.randn(512, device=dev)
    loss, st = ppo_actor_loss_fn(z.clone().requires_grad_(True), z, z, torch.randn(512, device=dev), 0.2,
                                 torch.zeros(512, dtype=torch.bool, device=dev))
    assert loss.item() == 0.0 and st["n_valid_tokens"] == 0.0 and st["masked_token_ratio"] == 1.0
    lp, prox, old, adv, mask, cu = (t.to(dev) for t in _random_batch(50000, 64, seed=2))
    rs = RejectionSamplingConfig(level="token", metric="ratio", upper=2.0, lower=0.5)
    outs = [ppo_actor_loss_fn(lp, prox, old, adv, 0.2, mask, rejection_sampling=rs) for _ in range(3)]
    for l, s in outs[1:]:
        assert torch.equal(l, outs[0][0])  # bit-identical repeat runs
        assert torch.equal(s["loss"], outs[0][1]["loss"])


# ---------------------------------------------------------------- statistics reduced in the loss pass
REDUCED_VARIANTS = [
    dict(),
    dict(eps_clip_higher=0.28, c_clip=1.5, rs=RS_CONFIGS[0]),
    dict(rs=RS_CONFIGS[5]),
    dict(level="sequence", rs=RS_CONFIGS[6]),
    dict(cispo=True, rs=RS_CONFIGS[0]),
]


@pytest.mark.parametrize("var", REDUCED_VARIANTS, ids=[str(i) for i in range(len(REDUCED_VARIANTS))])
def test_reduced_stats_match_oracle_masked_stats(dev, var):
    """grpo_loss_fn(stats_mode="reduced") writes no per-token statistic tensor; what it reports is
    compared with the oracle's per-token stat tensors (assembled as actor.py:662-733 hands them to
    the tracker) reduced by oracle.packing.masked_stats, the restatement of the tracker's masked
    sum / min / max (stats_tracker.py:455-560)."""
    from areal_amd.ppo.actor import grpo_loss_fn
    from oracle.packing import masked_stats as oracle_masked_stats

    n, n_seqs = 70_001, 24
    lp, prox, old, adv, mask, cu = _random_batch(n, n_seqs, seed=31)
    g = torch.Generator().manual_seed(32)
    ent = torch.rand(n, generator=g) * 3
    vmin, vmax = -torch.rand(n, generator=g) * 9 - 3, torch.rand(n, generator=g) * 20
    rs = var.get("rs")
    cispo = var.get("cispo", False)
    hi = 4.0 if cispo else var.get("eps_clip_higher")
    level = var.get("level", "token")

    # oracle: per-token tensors, then the tracker's reductions
    lp_o = lp.clone().requires_grad_(True)
    if cispo:
        lo, so = O.cispo_loss(lp_o, prox, adv, 0.2, mask, eps_clip_higher=hi, old_logprobs=old,
                              rejection_sampling_cfg=rs, cu_seqlens=cu)
        so["dual_clip_mask"] = torch.zeros(n, dtype=torch.bool)
    else:
        lo, so = O.ppo_actor_loss(lp_o, prox, old, adv, 0.2, mask, eps_clip_higher=hi, c_clip=var.get("c_clip"),
                                  rejection_sampling_cfg=rs, importance_sampling_level=level, cu_seqlens=cu)
    lo.backward()
    lpd = lp_o.detach()
    diff = (old - lpd) * mask
    vals = dict(importance_weight=so["importance_weight"], approx_kl=so["approx_kl"], new_logp=lpd, old_logp=old,
                entropy=ent, actor_loss=so["loss"], clip_ratio=so["clip_mask"].float(),
                dual_clip_ratio=so["dual_clip_mask"].float(), logp_diff=diff, logp_abs_diff=diff.abs(),
                clipped_new_logp=torch.where(so["clip_mask"], lpd, 0.0),
                clipped_old_logp=torch.where(so["clip_mask"], old, 0.0),
                vocab_min_logits=vmin, vocab_max_logits=vmax)
    den = {k: mask for k in vals}
    den["clipped_new_logp"] = den["clipped_old_logp"] = so["clip_mask"]
    den["vocab_min_logits"] = den["vocab_max_logits"] = None
    if rs is not None:
        vals.update(behave_imp_weight=so["behave_imp_weight"], behave_approx_kl=so["behave_approx_kl"],
                    behave_filtered_ratio=(mask & ~so["behave_mask"]).float())
        den.update(behave_imp_weight=so["behave_mask"], behave_approx_kl=so["behave_mask"], behave_filtered_ratio=mask)
    want = oracle_masked_stats(vals, den)

    stats = {}
    lp_g = lp.to(dev).requires_grad_(True)
    data = dict(logprobs=old.to(dev), advantages=adv.to(dev), loss_mask=mask.to(dev), prox_logp=prox.to(dev),
                cu_seqlens=cu.to(dev))
    loss = grpo_loss_fn(lp_g, ent.to(dev), data, 0.2, hi, var.get("c_clip"),
                        rejection_sampling=RejectionSamplingConfig(**rs) if rs else None,
                        importance_sampling_level=level, use_cispo_loss=cispo,
                        vocab_min_logits=vmin.to(dev), vocab_max_logits=vmax.to(dev),
                        stats=stats, stats_mode="reduced")
    loss.backward()
    torch.testing.assert_close(loss.detach().cpu(), lo.detach(), rtol=1e-4, atol=1e-7)
    rel = (lp_g.grad.cpu() - lp_o.grad).norm() / lp_o.grad.norm()
    assert rel < 1e-2
    assert not any(torch.is_tensor(v) for v in stats.values())  # nothing of token shape comes back
    assert set(want) <= set(stats), sorted(set(want) - set(stats))
    for k, w in want.items():
        got = stats[k]
        assert got["count"] == w["count"], k
        if w["count"] == 0:
            assert got["avg"] is None and got["min"] is None and got["max"] is None, k
            continue
        assert got["sum"] == pytest.approx(w["sum"], rel=2e-5, abs=1e-4 * max(1.0, w["count"]) * 1e-3), k
        assert got["min"] == pytest.approx(w["min"], rel=2e-6, abs=1e-6), k
        assert got["max"] == pytest.approx(w["max"], rel=2e-6, abs=1e-6), k
    assert stats["denominator/n_valid_tokens"] == float(mask.sum())
    assert stats["denominator/clipped_tokens"] == float(so["clip_mask"].sum())
    assert stats["denominator/n_tokens"] == float(n)
    if rs is not None:
        assert stats["denominator/unclipped_behave_tokens"] == float(so["behave_mask"].sum())
        assert stats["scalar/rs_filtered_fraction"] == pytest.approx(so["filtered_fraction"], abs=1e-12)


def test_reduced_stats_agree_with_the_tensor_mode_on_the_gpu(dev):
    """The same call in both modes: the reduced values equal masked_stats of the tensors the
    default mode returns, and the loss and gradient are bit-identical."""
    from areal_amd.ppo.actor import grpo_loss_fn
    from areal_amd.stats import masked_stats

    n = 200_000
    lp, prox, old, adv, mask, cu = _random_batch(n, 50, seed=41)
    rs = RejectionSamplingConfig(**RS_CONFIGS[1])
    data = dict(logprobs=old.to(dev), advantages=adv.to(dev), loss_mask=mask.to(dev), prox_logp=prox.to(dev))
    ent = torch.rand(n, device=dev)
    out = {}
    for mode in ("tensors", "reduced"):
        st = {}
        x = lp.to(dev).requires_grad_(True)
        loss = grpo_loss_fn(x, ent, data, 0.2, 0.28, 3.0, rejection_sampling=rs, stats=st, stats_mode=mode)
        loss.backward()
        out[mode] = (loss.detach(), x.grad, st)
    assert torch.equal(out["tensors"][0], out["reduced"][0]) and torch.equal(out["tensors"][1], out["reduced"][1])
    t, r = out["tensors"][2], out["reduced"][2]
    keys = ["importance_weight", "approx_kl", "new_logp", "old_logp", "entropy", "actor_loss", "clip_ratio",
            "logp_abs_diff"]
    want = masked_stats({k: t[k] for k in keys}, {k: t["n_valid_tokens"] for k in keys})
    want.update(masked_stats({"behave_imp_weight": t["behave_imp_weight"]},
                             {"behave_imp_weight": t["unclipped_behave_tokens"]}))
    for k, w in want.items():
        assert r[k]["count"] == w["count"]
        # a thread of the token pass adds its few tokens in fp32; from the wave level on sums are fp64
        assert r[k]["sum"] == pytest.approx(w["sum"], rel=1e-6, abs=1e-6), k
        assert r[k]["min"] == w["min"] and r[k]["max"] == w["max"], k
