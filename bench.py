"""Benchmark of the per-token RL training hot path on one MI355X.

One "step" = fused lm_head -> logprob/entropy forward, GRPO/PPO actor loss with IcePop
(ratio-bound) rejection sampling, and the backward pass to dHidden and dWeight, on one packed
micro-batch that is already resident in HBM.  Prints ONE JSON line.

    python bench.py --gpus 1 --steps 10 --warmup 3 [--workload qwen3-8b]
"""

from __future__ import annotations

import argparse
import functools
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

V_QWEN = 151936
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA peak used for the roofline fraction

# The contraction kernels of the default workload as rocprofv3 names them (checked against the
# loaded library before they are printed). gemm16_sweep<variant, epilogue>: variant 0 = both
# operands k-contiguous, 1 = both k-major, 2 = A k-major; Fwd16<edge, affine, moments, save>,
# Store16<edge, mode> with mode 0 = bf16, 3 = bf16 scaled per output row.
KERNEL_FWD_SAVE = "gemm16_sweep<0, Fwd16<false, false, false, true> >"
KERNEL_FWD = "gemm16_sweep<0, Fwd16<false, false, false, false> >"
KERNEL_RECOMPUTE = "gemm16_sweep<0, Bwd16<false, false> >"
KERNEL_DHIDDEN = "gemm16_sweep<2, Store16<false, 3> >"
KERNEL_DWEIGHT = "gemm16_sweep<1, Store16<false, 0> >"

WORKLOADS = {
    # name: (T, H, n_seqs, min_len, max_len, seed, description)
    "qwen3-8b": dict(T=32768, H=4096, n_seqs=32, lo=256, hi=2048, seed=3,
                     desc="BASELINE config 4: Qwen3-8B shape fwd+bwd, IcePop ratio bounds [0.5, 2.0]"),
    "qwen2.5-1.5b": dict(T=16384, H=1536, n_seqs=64, lo=32, hi=2048, seed=1,
                         desc="BASELINE config 2: Qwen2.5-1.5B shape fwd+bwd, decoupled PPO"),
    "qwen3-14b-128k": dict(T=131072, H=5120, n_seqs=4, lo=32768, hi=32768, seed=4,
                           desc="BASELINE config 5 shape: 4 x 32768 tokens, H=5120, fwd+bwd (39.8 GB of bf16 "
                                "exponentials kept for the backward)"),
    "qwen2.5-0.5b": dict(T=4096, H=896, n_seqs=16, lo=64, hi=512, seed=0,
                         desc="BASELINE config 1 shape (run fwd+bwd here)"),
}


def make_batch(name: str, device):
    """Synthetic packed micro-batch of the named shape (seeded, random-init weights)."""
    import torch

    w = WORKLOADS[name]
    T, H = w["T"], w["H"]
    g = torch.Generator().manual_seed(w["seed"])
    lens = torch.randint(w["lo"], w["hi"] + 1, (w["n_seqs"],), generator=g)
    if int(lens.sum()) > T:  # rescale proportionally so the sequences fit
        lens = torch.clamp((lens.double() * T / lens.sum()).floor().long(), min=w["lo"])
        while int(lens.sum()) > T:
            lens[lens.argmax()] -= 1
    pad = T - int(lens.sum())
    seg = lens.tolist() + ([pad] if pad > 0 else [])
    cu = torch.tensor([0] + torch.tensor(seg).cumsum(0).tolist(), dtype=torch.int32)
    loss_mask = torch.ones(T, dtype=torch.bool)
    loss_mask[cu[1 : w["n_seqs"] + 1].long() - 1] = False  # last token of a sequence has no label
    if pad > 0:
        loss_mask[T - pad :] = False
    hidden = torch.randn(T, H, generator=g, dtype=torch.float32).bfloat16()
    labels = torch.randint(0, V_QWEN, (T,), generator=g)
    weight = torch.empty(V_QWEN, H, dtype=torch.bfloat16)
    for i in range(0, V_QWEN, 16384):  # chunked to bound host memory
        n = min(16384, V_QWEN - i)
        weight[i : i + n] = (torch.randn(n, H, generator=g) * 0.02).bfloat16()
    adv_seq = torch.randn(len(seg), generator=g)
    advantages = adv_seq.repeat_interleave(torch.tensor(seg))
    return dict(
        hidden=hidden.to(device), weight=weight.to(device), labels=labels.to(device),
        cu_seqlens=cu.to(device), loss_mask=loss_mask.to(device), advantages=advantages.to(device),
        T=T, H=H, V=V_QWEN, seed=w["seed"],
    )


def make_batch_on_device(name: str, device):
    """The same shapes and distributions drawn with the device's generator (seeded): used for the
    secondary workloads, whose host-side generation would take longer than their timed steps."""
    import torch

    w = WORKLOADS[name]
    T, H = w["T"], w["H"]
    g = torch.Generator().manual_seed(w["seed"])
    lens = torch.randint(w["lo"], w["hi"] + 1, (w["n_seqs"],), generator=g)
    if int(lens.sum()) > T:
        lens = torch.clamp((lens.double() * T / lens.sum()).floor().long(), min=w["lo"])
        while int(lens.sum()) > T:
            lens[lens.argmax()] -= 1
    pad = T - int(lens.sum())
    seg = lens.tolist() + ([pad] if pad > 0 else [])
    cu = torch.tensor([0] + torch.tensor(seg).cumsum(0).tolist(), dtype=torch.int32)
    loss_mask = torch.ones(T, dtype=torch.bool)
    loss_mask[cu[1 : w["n_seqs"] + 1].long() - 1] = False
    if pad > 0:
        loss_mask[T - pad :] = False
    gd = torch.Generator(device=device).manual_seed(w["seed"])
    hidden = torch.randn(T, H, generator=gd, device=device, dtype=torch.float32).bfloat16()
    weight = torch.empty(V_QWEN, H, dtype=torch.bfloat16, device=device)
    for i in range(0, V_QWEN, 32768):  # chunked to bound the fp32 temporaries
        n = min(32768, V_QWEN - i)
        weight[i : i + n] = (torch.randn(n, H, generator=gd, device=device) * 0.02).bfloat16()
    labels = torch.randint(0, V_QWEN, (T,), generator=gd, device=device)
    adv_seq = torch.randn(len(seg), generator=g)
    advantages = adv_seq.repeat_interleave(torch.tensor(seg))
    return dict(hidden=hidden, weight=weight, labels=labels, cu_seqlens=cu.to(device),
                loss_mask=loss_mask.to(device), advantages=advantages.to(device), T=T, H=H, V=V_QWEN,
                seed=w["seed"])


def cpu_baseline(sample_tokens: int, H: int, seed: int, threads: int, repeats: int = 3):
    """The CPU oracle (plain PyTorch port of the reference's op sequence) on a token slice at
    full vocabulary: fp32 logits from bf16 operands, log-softmax + entropy, PPO loss with
    rejection sampling, autograd backward to hidden and weight. Returns (tokens/s of the median
    repeat, the repeats' seconds)."""
    import torch

    from oracle import logprob as olp
    from oracle import loss as oloss

    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(seed)
    n = sample_tokens
    hidden = torch.randn(n, H, generator=g).bfloat16()
    weight = (torch.randn(V_QWEN, H, generator=g) * 0.02).bfloat16()
    labels = torch.randint(0, V_QWEN, (n,), generator=g)
    adv = torch.randn(n, generator=g)
    mask = torch.ones(n, dtype=torch.bool)
    times = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        h32 = hidden.float().requires_grad_(True)
        w32 = weight.float().requires_grad_(True)
        logits = h32 @ w32.T
        lp, ent = olp.gather_logprobs_entropy(logits, labels, 1.0)
        old = lp.detach() + 0.05
        loss, _ = oloss.ppo_actor_loss(lp, lp.detach(), old, adv, 0.2, mask,
                                       rejection_sampling_cfg=dict(level="token", action="mask", metric="ratio",
                                                                   upper=2.0, lower=0.5))
        loss.backward()
        times.append(time.perf_counter() - t0)
        del h32, w32, logits, lp, ent, loss
    med = sorted(times)[len(times) // 2]
    return n / med, times


def cpu_baseline_advantages(threads: int):
    """The CPU oracle on BASELINE config 3 in full: the reference's padded GAE loop over
    [1024, 8192] slots and the group normalisation of the advantages (groups of 16 rows)."""
    import torch

    from oracle import gae as ogae
    from oracle import norm as onorm

    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(2)
    lens = torch.clamp((torch.randn(1024, generator=g) + 7.0).exp().long(), 16, 8192)
    pos = torch.arange(8192)[None, :]
    r = torch.zeros(1024, 8192)
    r[torch.arange(1024), (lens - 2).clamp(min=0)] = 1.0
    v = torch.randn(1024, 8192, generator=g)
    m = ((pos >= (lens // 4)[:, None]) & (pos < (lens - 1)[:, None])).float()
    no_eos = torch.zeros(1024, dtype=torch.bool)
    t0 = time.perf_counter()
    adv, _ = ogae.gae_padded(r, v, m, no_eos, 1.0, 0.95)
    t1 = time.perf_counter()
    onorm.normalization(adv, m, mean_level="group", std_level="group", group_size=16)
    t2 = time.perf_counter()
    return {"workload": "config 3 padded form in full: [1024, 8192] slots, PyTorch oracle",
            "gae_ms": (t1 - t0) * 1e3, "group_norm_ms": (t2 - t1) * 1e3, "cores": threads, "kind": "port"}


def hbm_rooflines(dev):
    """HBM-bound kernels of the path on their own workloads: algorithmic bytes / HIP-event time.
    GAE + group normalisation on BASELINE config 3 (1024 packed sequences, lognormal lengths),
    the actor-loss token kernel on 4 Mi tokens (forward + closed-form backward, full stat dict),
    and the logits-in row kernel on config 1's [4096, 151936] bf16 logits."""
    import torch

    from areal_amd.config import NormConfig, RejectionSamplingConfig
    from areal_amd.data import Normalization
    from areal_amd.functional import gather_logprobs_entropy, ppo_actor_loss_fn
    from areal_amd.ppo.gae import compute_gae_packed

    peak = 8000.0

    def timed(fn, iters=20, warm=3):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(iters):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / iters

    out = []

    def add(name, workload, nbytes, ms):
        gbs = nbytes / (ms * 1e-3) / 1e9
        out.append({"kernel": name, "workload": workload, "bound": "hbm", "algorithmic_bytes": nbytes,
                    "ms": ms, "achieved": gbs, "peak": peak, "unit": "GB/s", "frac": gbs / peak})

    g = torch.Generator().manual_seed(2)
    lens = torch.clamp((torch.randn(1024, generator=g) + 7.0).exp().long(), 16, 8192)
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32).to(dev)
    T = int(cu[-1])
    r = torch.zeros(T, device=dev)
    r[cu[1:].long() - 2] = 1.0
    v = torch.randn(T, device=dev)
    m = (torch.rand(T, device=dev) > 0.25).float()
    add("gae_tile_kernel", f"config 3: 1024 packed sequences, {T} tokens, 20 B/token",
        20 * T, timed(lambda: compute_gae_packed(r, v, m, cu, None, 1.0, 0.95)))
    # the same batch through the C ABI, launches back to back on the stream (no host work between
    # them): packed GAE, then group normalisation (groups of 16 sequences, mean and deviation at
    # group level) of the advantages under the same mask. 3 launches: gae_tile_kernel,
    # norm_stats5_kernel, norm_apply_cf_kernel.
    from areal_amd import _lib as L_

    lib_ = L_.load()
    adv_o, ret_o, nrm_o = torch.empty(T, device=dev), torch.empty(T, device=dev), torch.empty(T, device=dev)
    goff = cu[::16].to(torch.int64).contiguous()
    grow = torch.full((64,), 16, dtype=torch.int64, device=dev)
    max_glen = int((goff[1:] - goff[:-1]).max())
    gae_ws_n = lib_.areal_gae_workspace_bytes(T)
    nrm_ws_n = lib_.areal_group_norm_workspace_bytes(64, max_glen)
    gae_ws, nrm_ws = L_.workspace(gae_ws_n, dev), L_.workspace(nrm_ws_n, dev)
    strm = L_.stream_ptr(dev)

    def gae_then_norm():
        rc = lib_.areal_gae_packed(L_.ptr(r), L_.ptr(v), L_.ptr(m), L_.ptr(cu), None, None, T, 1024, 0, 1.0, 0.95,
                                   L_.ptr(adv_o), L_.ptr(ret_o), L_.ptr(gae_ws), gae_ws_n, strm)
        rc |= lib_.areal_group_norm(L_.ptr(adv_o), L_.ptr(m), T, L_.ptr(goff), L_.ptr(grow), 64, max_glen, -1, 2, 2,
                                    0, 1, 1e-5, L_.ptr(nrm_o), L_.ptr(nrm_ws), nrm_ws_n, strm)
        assert rc == 0

    add("gae_tile_kernel + norm_stats5_kernel + norm_apply_cf_kernel (C ABI)",
        f"config 3: 1024 packed sequences, {T} tokens, GAE then group normalisation of the advantages, "
        "launches back to back, 20 + 20 B/token", 40 * T, timed(gae_then_norm))
    # the same in two launches: the GAE kernel leaves the per-(tile, group) sums of its advantages,
    # the apply pass of the normalisation starts from them
    seg_n = lib_.areal_gae_segment_stats_bytes(T, 64)
    seg = torch.empty(seg_n // 8, dtype=torch.float64, device=dev)

    def gae_stats_then_apply():
        rc = lib_.areal_gae_packed_group_stats(L_.ptr(r), L_.ptr(v), L_.ptr(m), L_.ptr(cu), None, None, T, 1024, 1.0,
                                               0.95, L_.ptr(goff), 64, L_.ptr(adv_o), L_.ptr(ret_o), L_.ptr(seg), seg_n,
                                               strm)
        rc |= lib_.areal_group_norm_from_segment_stats(L_.ptr(adv_o), L_.ptr(m), T, L_.ptr(goff), L_.ptr(grow), 64,
                                                       max_glen, -1, 2, 2, 1, 1e-5, L_.ptr(seg), L_.ptr(nrm_o), strm)
        assert rc == 0

    add("gae_tile_kernel<stats> + norm_apply_cf_kernel (C ABI)",
        f"config 3: 1024 packed sequences, {T} tokens, GAE that leaves the normalisation's sums, then the apply "
        "pass: two launches, 20 + 20 B/token", 40 * T, timed(gae_stats_then_apply))
    del adv_o, ret_o, nrm_o, seg
    # the padded drop-in signature on the same batch: [1024, 8192] (8.39 M slots)
    from areal_amd.ppo.gae import _compute_token_level_gae

    rp = torch.zeros(1024, 8192, device=dev)
    rp[torch.arange(1024, device=dev), (lens.to(dev) - 2).clamp(min=0)] = 1.0
    vp = torch.randn(1024, 8192, device=dev)
    pos = torch.arange(8192, device=dev)[None, :]
    mp = ((pos >= (lens.to(dev) // 4)[:, None]) & (pos < (lens.to(dev) - 1)[:, None])).float()
    no_eos = torch.zeros(1024, dtype=torch.bool, device=dev)
    add("gae_owned_kernel", "config 3 padded form: [1024, 8192] slots, 20 B/slot",
        20 * rp.numel(), timed(lambda: _compute_token_level_gae(rp, vp, mp, no_eos, 1.0, 0.95)))
    # the whole advantage step on that padded batch: reward shaping (one pass), GAE, group
    # normalisation of rewards and advantages
    from areal_amd.data import KLEstimator
    from areal_amd.ppo.actor import compute_advantages

    attn = pos < lens.to(dev)[:, None]
    adv_data = dict(input_ids=torch.zeros(1024, 8192, dtype=torch.long, device=dev), attention_mask=attn,
                    loss_mask=(pos >= (lens.to(dev) // 4)[:, None]) & attn,
                    logprobs=torch.randn(1024, 8192, device=dev) * 0.1 - 1,
                    ref_logp=torch.randn(1024, 8192, device=dev) * 0.1 - 1, values=vp,
                    rewards=(torch.rand(1024, device=dev) > 0.5).float())
    gnorm = Normalization(NormConfig(mean_level="group", std_level="group", group_size=16))
    add("adv_prep_kernel + gae_owned_kernel<stats> + norm_apply_cf_kernel (compute_advantages, API level)",
        "config 3 padded form: [1024, 8192], KL-shaped rewards, GAE that also sums each row's advantages, "
        "group normalisation as its apply pass alone (plus the [1024] reward normalisation); "
        "26 + 20 + 20 B/slot",
        66 * rp.numel(),
        timed(lambda: compute_advantages(dict(adv_data), kl_ctl=0.01, kl_estimator=KLEstimator("k1"),
                                         reward_norm=gnorm, adv_norm=gnorm, discount=1.0, gae_lambda=0.95)))
    del rp, vp, mp, adv_data
    x = torch.randn(1024, 1600, device=dev)
    mk = (torch.rand(1024, 1600, device=dev) > 0.25).float()
    norm = Normalization(NormConfig(mean_level="group", std_level="group", group_size=16))
    add("norm_stats5_kernel + norm_apply_cf_kernel", "config 3: [1024, 1600] advantages, groups of 16 rows, 20 B/token",
        20 * x.numel(), timed(lambda: norm(x, mk)))
    # the same normalisation at the padded size, where launch latency no longer dominates
    xl_ = torch.randn(1024, 8192, device=dev)
    ml_ = (torch.rand(1024, 8192, device=dev) > 0.25).float()
    add("norm_stats5_kernel + norm_apply_cf_kernel", "[1024, 8192] advantages, groups of 16 rows, 20 B/token",
        20 * xl_.numel(), timed(lambda: norm(xl_, ml_)))
    del xl_, ml_
    Tl = 4 << 20
    lp = (torch.randn(Tl, device=dev) * 0.5 - 1).requires_grad_(True)
    prox = lp.detach() + torch.randn(Tl, device=dev) * 0.1
    old = prox + torch.randn(Tl, device=dev) * 0.1
    adv = torch.randn(Tl, device=dev)
    mask = torch.rand(Tl, device=dev) > 0.2
    rs = RejectionSamplingConfig(level="token", metric="ratio", upper=2.0, lower=0.5)

    def loss_step():
        lp.grad = None
        loss, _ = ppo_actor_loss_fn(lp, prox, old, adv, 0.2, mask, rejection_sampling=rs)
        loss.backward()

    add("ppo_actor_loss_fn + backward (API level)",
        "PPO + IcePop, 4 Mi tokens, fwd+bwd through the Python API: includes the one device-to-host copy "
        "of the counters per call (the reference has 1-3 .item() syncs), 47 B/token + 8 B/token grad scale",
        55 * Tl, timed(loss_step))

    # the same kernels through the C ABI without the host copy, back to back on the stream
    from areal_amd import _lib
    from areal_amd.functional import functional as F

    lib = _lib.load()
    cfg = _lib.LossConfig()
    cfg.loss_kind = F.LOSS_PPO
    cfg.clip_lo, cfg.clip_hi = 0.8, 1.2
    F._fill_rs(cfg, rs)
    lp32, mask_b = lp.detach(), mask.bool().contiguous()
    gout = torch.ones(1, device=dev)
    grad = torch.empty(Tl, device=dev)

    def loss_kernels():
        o = F._run_loss_kernel(cfg, lp32.shape, lp32, prox, old, adv, mask_b, None, True)
        rc = lib.areal_actor_loss_grad(_lib.ptr(o["dlp"]), _lib.ptr(gout), _lib.ptr(o["counters_dev"]),
                                       _lib.ptr(grad), Tl, _lib.stream_ptr(dev))
        _lib.check(rc, "areal_actor_loss_grad")

    add("loss_token+loss_finalize+loss_grad_scale", "PPO + IcePop, 4 Mi tokens, fwd+bwd kernels through the C ABI, "
        "47 B/token + 8 B/token grad scale", 55 * Tl, timed(loss_kernels, iters=50))
    # the same loss with every logged statistic reduced inside the token pass: no per-token
    # statistic tensor is written (17 B/token of inputs + 4 B entropy read, 4 B gradient written)
    ent = torch.rand(Tl, device=dev)
    both = torch.empty(8 + 4 * len(F.REDUCED_STAT_KEYS), dtype=torch.float64, device=dev)
    dlp = torch.empty(Tl, device=dev)
    loss_out = torch.empty((), device=dev)
    nb = lib.areal_actor_loss_stats_workspace_bytes(Tl, 0)
    ws_r = torch.empty(nb, dtype=torch.uint8, device=dev)
    import ctypes

    def loss_kernels_reduced():
        p = _lib.ptr
        rc = lib.areal_actor_loss_stats(
            p(lp32), p(prox), p(old), p(adv), p(mask_b), None, Tl, 0, 0, ctypes.byref(cfg), p(ent), None, None,
            p(loss_out), p(dlp), None, None, None, None, None, None, None, None, None,
            p(both[:8]), p(both[8:]), p(ws_r), nb, _lib.stream_ptr(dev))
        _lib.check(rc, "areal_actor_loss_stats")
        rc = lib.areal_actor_loss_grad(p(dlp), p(gout), p(both[:8]), p(grad), Tl, _lib.stream_ptr(dev))
        _lib.check(rc, "areal_actor_loss_grad")

    add("loss_token<stats>+loss_finalize+loss_grad_scale",
        "PPO + IcePop, 4 Mi tokens, fwd+bwd kernels through the C ABI with the 13 logged statistics reduced in "
        "the token pass instead of written as [T] tensors: 25 B/token + 8 B/token grad scale",
        33 * Tl, timed(loss_kernels_reduced, iters=50))
    from areal_amd.ppo.actor import grpo_loss_fn

    gdata = dict(logprobs=old, advantages=adv, loss_mask=mask, prox_logp=prox)

    def grpo_reduced():
        lp.grad = None
        st = {}
        grpo_loss_fn(lp, ent, gdata, 0.2, None, None, rejection_sampling=rs, stats=st, stats_mode="reduced").backward()

    def grpo_tensors():
        lp.grad = None
        st = {}
        grpo_loss_fn(lp, ent, gdata, 0.2, None, None, rejection_sampling=rs, stats=st).backward()
        masked_stats({k: st[k] for k in ("importance_weight", "approx_kl", "new_logp", "old_logp", "entropy",
                                          "actor_loss", "clip_ratio", "dual_clip_ratio", "logp_diff",
                                          "logp_abs_diff", "behave_filtered_ratio")},
                     {k: st["n_valid_tokens"] for k in st})

    from areal_amd.stats import masked_stats

    add("grpo_loss_fn(stats_mode='reduced') + backward (API level)",
        "PPO + IcePop with logging, 4 Mi tokens: statistics reduced in the loss pass, 25 + 8 B/token",
        33 * Tl, timed(grpo_reduced))
    add("grpo_loss_fn(stats_mode='tensors') + masked_stats + backward (API level)",
        "the same logging through per-token tensors and a separate reduction launch: 47 + 8 B/token written and "
        "read by the loss, 8 B of logp_diff tensors, then 11 x 5 B/token read by the reduction",
        (47 + 8 + 8 + 55) * Tl, timed(grpo_tensors))
    # kernels of the steps either side of the loss (API level: each call includes its own host work)
    from areal_amd.functional import ppo_critic_loss_fn, sapo_loss_fn
    from areal_amd.packing import pack_tensor_dict
    from areal_amd.ppo.actor import _apply_m2po_masking
    from areal_amd.ppo.gae import _compute_turn_level_gae
    from areal_amd.stats import masked_stats

    def sapo_step():
        lp.grad = None
        loss, _ = sapo_loss_fn(lp, old, adv, 1.0, 1.05, mask)
        loss.backward()

    add("sapo_token_kernel + backward (API level)", "SAPO, 4 Mi tokens, 7 output tensors, 41 B/token + 8 B/token grad scale",
        49 * Tl, timed(sapo_step))
    # the same kernels through the C ABI, back to back on the stream (no host work between them)
    p = _lib.ptr
    strm2 = _lib.stream_ptr(dev)
    aux_nb = lib.areal_aux_loss_workspace_bytes(Tl, 0)
    aux_ws = torch.empty(aux_nb, dtype=torch.uint8, device=dev)
    s_out = [torch.empty(Tl, device=dev) for _ in range(7)]  # dsum + 6 statistic tensors
    s_cnt = torch.empty(8 + 4 * 13, dtype=torch.float64, device=dev)

    def sapo_kernels(reduced):
        outs = [None] * 6 if reduced else [p(t) for t in s_out[1:]]
        rc = lib.areal_sapo_loss(p(lp32), p(old), p(adv), p(mask_b), None, Tl, 0, 0, 1.0, 1.05, 0, p(loss_out),
                                 p(s_out[0]), *outs, p(s_cnt[:8]), p(ent) if reduced else None, None, None,
                                 p(s_cnt[8:]) if reduced else None, p(aux_ws), aux_nb, strm2)
        _lib.check(rc, "areal_sapo_loss")
        rc = lib.areal_actor_loss_grad(p(s_out[0]), p(gout), p(s_cnt[:8]), p(grad), Tl, strm2)
        _lib.check(rc, "areal_actor_loss_grad")

    add("sapo_token+aux_finalize+loss_grad_scale (C ABI)", "SAPO, 4 Mi tokens, fwd+bwd kernels through the C ABI, "
        "41 B/token + 8 B/token grad scale", 49 * Tl, timed(lambda: sapo_kernels(False), iters=50))
    add("sapo_token<stats>+aux_finalize+loss_grad_scale (C ABI)", "SAPO, 4 Mi tokens, the 11 logged statistics reduced "
        "in the token pass instead of written as [T] tensors: 13 B/token in + 4 B entropy + 4 B gradient out + "
        "8 B/token grad scale", 29 * Tl, timed(lambda: sapo_kernels(True), iters=50))
    val = torch.randn(Tl, device=dev).requires_grad_(True)
    oldv, tgt = val.detach() + 0.1 * torch.randn(Tl, device=dev), torch.randn(Tl, device=dev)

    def critic_step():
        val.grad = None
        loss, _ = ppo_critic_loss_fn(val, oldv, tgt, 0.2, mask)
        loss.backward()

    add("critic_token_kernel + backward (API level)", "clipped value loss, 4 Mi tokens, 22 B/token + 8 B/token grad scale",
        30 * Tl, timed(critic_step))
    c_dv, c_sl, c_cm = torch.empty(Tl, device=dev), torch.empty(Tl, device=dev), torch.empty(Tl, dtype=torch.bool, device=dev)
    val32 = val.detach()

    def critic_kernels():
        rc = lib.areal_critic_loss(p(val32), p(oldv), p(tgt), p(mask_b), Tl, 0.2, 0, p(loss_out), p(c_dv), p(c_sl),
                                   p(c_cm), p(s_cnt[:8]), p(aux_ws), aux_nb, strm2)
        _lib.check(rc, "areal_critic_loss")
        rc = lib.areal_actor_loss_grad(p(c_dv), p(gout), p(s_cnt[:8]), p(grad), Tl, strm2)
        _lib.check(rc, "areal_actor_loss_grad")

    add("critic_token+aux_finalize+loss_grad_scale (C ABI)", "clipped value loss, 4 Mi tokens, fwd+bwd kernels through "
        "the C ABI, 22 B/token + 8 B/token grad scale", 30 * Tl, timed(critic_kernels, iters=50))
    add("m2_hist x4 + m2_select x4 + m2_tie_count + m2_apply (API level)",
        "M2PO mask by radix select, 4 Mi tokens, 6 passes x 9 B/token",
        54 * Tl, timed(lambda: _apply_m2po_masking(old, prox, mask, 0.04)))
    stat_vals = {f"s{i}": (adv if i % 2 else prox) for i in range(24)}
    stat_den = {f"s{i}": mask for i in range(24)}
    add("stats_partial_kernel + stats_final_kernel (API level)",
        "24 masked statistics (sum, count, min, max) over 4 Mi tokens, 5 B/token each",
        24 * 5 * Tl, timed(lambda: masked_stats(stat_vals, stat_den)))
    bsz, Lp = 1024, 8192
    plens = torch.clamp((torch.randn(bsz, generator=g) + 7.0).exp().long(), 16, Lp).to(dev)
    ppos = torch.arange(Lp, device=dev)[None, :]
    pattn = ppos < plens[:, None]
    pdata = dict(attention_mask=pattn, input_ids=torch.randint(0, 1000, (bsz, Lp), device=dev),
                 loss_mask=pattn & (ppos >= (plens // 4)[:, None]), logprobs=torch.randn(bsz, Lp, device=dev),
                 advantages=torch.randn(bsz, Lp, device=dev))
    n_packed = int(plens.sum())
    add("rowlens + cu_scan + pack_rows (API level)",
        f"pack_tensor_dict: [1024, 8192] padded -> {n_packed} packed tokens, 5 tensors (8+8+1+4+4 B), read + write",
        2 * 25 * n_packed + bsz * Lp, timed(lambda: pack_tensor_dict(dict(pdata))))
    # the same launches through the C ABI into preallocated outputs
    pk_mask = pattn.contiguous().view(torch.uint8)
    pk_lens = torch.empty(bsz, dtype=torch.int32, device=dev)
    pk_cu = torch.empty(bsz + 1, dtype=torch.int32, device=dev)
    pk_max = torch.empty(1, dtype=torch.int32, device=dev)
    pk_src = [pdata[k].contiguous() for k in ("input_ids", "loss_mask", "logprobs", "advantages")]
    pk_src.append(torch.zeros(bsz, Lp, dtype=torch.long, device=dev))  # a second 8-byte tensor (position ids)
    pk_dst = [torch.empty(n_packed, dtype=t.dtype, device=dev) for t in pk_src]

    import ctypes

    pk_srcs = (ctypes.c_void_p * 5)(*[t.data_ptr() for t in pk_src])
    pk_dsts = (ctypes.c_void_p * 5)(*[t.data_ptr() for t in pk_dst])
    pk_sizes = (ctypes.c_int64 * 5)(*[t.element_size() for t in pk_src])

    def pack_kernels():
        rc = lib.areal_seqlens_from_mask(p(pk_mask), bsz, Lp, p(pk_lens), p(pk_cu), p(pk_max), strm2)
        rc |= lib.areal_pack_padded_multi(pk_srcs, pk_dsts, pk_sizes, 5, p(pk_cu), bsz, Lp, n_packed, strm2)
        assert rc == 0

    add("rowlens + cu_scan + pack_rows (C ABI)",
        f"[1024, 8192] padded -> {n_packed} packed tokens, 5 tensors (8+8+1+4+4 B), read + write, and the "
        "attention mask read once", 2 * 25 * n_packed + bsz * Lp, timed(pack_kernels, iters=50))
    # back to the padded layout: five launches of the row-wise unpack kernel (pad value 0)
    pk_back = [torch.empty_like(t) for t in pk_src]

    def unpack_kernels():
        rc = 0
        for s_, d_ in zip(pk_dst, pk_back):
            rc |= lib.areal_unpack_to_padded(p(s_), p(d_), p(pk_cu), None, bsz, Lp, s_.element_size(), None, 0, strm2)
        assert rc == 0

    pack_kernels()
    add("unpack_kernel x5 (C ABI)",
        f"{n_packed} packed tokens -> [1024, 8192] padded, 5 tensors (8+8+1+4+4 B): packed read, every padded slot "
        "written", 25 * n_packed + 25 * bsz * Lp, timed(unpack_kernels, iters=50))
    del pk_back
    turn_ids = (torch.cumsum((torch.rand(bsz, Lp, device=dev) < 0.002).int(), dim=1)).to(torch.int32)
    tr = torch.zeros(bsz, Lp, device=dev)
    tr[torch.arange(bsz, device=dev), (plens - 2).clamp(min=0)] = 1.0
    tv, tm = torch.randn(bsz, Lp, device=dev), pdata["loss_mask"].float()
    tne = torch.zeros(bsz, dtype=torch.bool, device=dev)
    add("turn_gae_kernel (API level, with validation)", "turn-level GAE, [1024, 8192] slots, 2 x 16 B/slot read + 8 B/slot written",
        40 * bsz * Lp, timed(lambda: _compute_turn_level_gae(tr, tv, tm, turn_ids, tne, 1.0, 0.95)))
    del pdata, turn_ids, tr, tv, tm
    lg = torch.randn(4096, V_QWEN, device=dev).bfloat16()
    lab = torch.randint(0, V_QWEN, (4096,), device=dev)
    add("rows_fwd_kernel", "config 1: [4096, 151936] bf16 logits, logprob + entropy forward",
        lg.numel() * 2 + 16 * 4096, timed(lambda: gather_logprobs_entropy(lg, lab), iters=10))
    # its backward: logits read once more, dlogits written in the logits' dtype
    lg.requires_grad_(True)
    glp = torch.randn(4096, device=dev)

    def rows_fwd_bwd():
        lp, _ = gather_logprobs_entropy(lg, lab)
        lp.backward(glp)
        lg.grad = None

    t_fb = timed(rows_fwd_bwd, iters=10)
    add("rows_fwd_kernel + rows_bwd_kernel (API level)",
        "config 1: [4096, 151936] bf16 logits, forward + backward of the label log-probabilities: "
        "logits read twice, dlogits written once", lg.numel() * 6 + 32 * 4096, t_fb)
    return out


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="qwen3-8b", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-sample-tokens", type=int, default=2048)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-hbm-kernels", action="store_true")
    ap.add_argument("--no-library-gemm", action="store_true",
                    help="skip timing torch.mm (the vendor library's bf16 GEMM) at the forward's shape")
    ap.add_argument("--no-other-mode", action="store_true",
                    help="skip the short second leg that times the other backward mode")
    ap.add_argument("--only-hbm-kernels", action="store_true",
                    help="time only the HBM-bound kernels (prints {\"hbm_rooflines\": [...]})")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the short legs on the other BASELINE shapes (configs 1, 2 and 5)")
    ap.add_argument("--recompute", action="store_true",
                    help="backward recomputes the logits (save_probs=False) instead of using the "
                         "bf16 exponentials kept by the forward")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch

    from areal_amd import _lib
    from areal_amd.config import RejectionSamplingConfig
    from areal_amd.functional import fused_lm_head_logprobs_entropy
    from areal_amd.ppo.actor import grpo_loss_fn

    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X: the hot path has no CPU implementation")
    _lib.load()
    dev = torch.device("cuda:0")
    if args.only_hbm_kernels:
        print(json.dumps({"hbm_rooflines": hbm_rooflines(dev)}))
        return

    class Workload:
        """One packed micro-batch resident in HBM and the step that is timed on it: fused
        forward, GRPO loss with IcePop masking, backward to dHidden and dWeight."""

        def __init__(self, b):
            self.b = b
            self.T, self.H, self.V = b["T"], b["H"], b["V"]
            self.hidden = b["hidden"].requires_grad_(True)
            self.weight = b["weight"].requires_grad_(True)
            # rollout log-probs = train log-probs + Laplace(0, 0.1); proximal = train log-probs
            with torch.no_grad():
                logp0 = fused_lm_head_logprobs_entropy(self.hidden, self.weight, b["labels"], temperature=1.0).logprobs
            torch.manual_seed(b["seed"])
            old = logp0 + torch.distributions.Laplace(0.0, 0.1).sample((self.T,)).to(dev)
            self.input_data = dict(logprobs=old, advantages=b["advantages"], loss_mask=b["loss_mask"],
                                   prox_logp=logp0, cu_seqlens=b["cu_seqlens"])
            self.loss_fn = functools.partial(
                grpo_loss_fn, eps_clip=0.2, eps_clip_higher=None, c_clip=None,
                rejection_sampling=RejectionSamplingConfig(level="token", action="mask", metric="ratio",
                                                           lower=0.5, upper=2.0),
                # the step is queued without waiting for the GPU: the loss's host scalars are read
                # after the backward is queued (nothing is skipped on the device)
                defer_host_reads=True,
            )
            self.saved = False

        def step(self, record: bool, save_probs, accum=None):
            self.hidden.grad = None
            self.weight.grad = None
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)] if record else None
            if record:
                ev[0].record()
            out = fused_lm_head_logprobs_entropy(self.hidden, self.weight, self.b["labels"], temperature=1.0,
                                                 save_probs=save_probs, weight_grad_accum=accum)
            self.saved = out.logprobs.grad_fn.probs is not None
            if record:
                ev[1].record()
            loss = self.loss_fn(out.logprobs, out.entropy, self.input_data,
                                vocab_min_logits=out.vocab_min_logits, vocab_max_logits=out.vocab_max_logits)
            if record:
                ev[2].record()
            loss.backward()
            if record:
                ev[3].record()
            return loss, ev

        def run(self, n_steps: int, n_warm: int, save_probs, accum=None):
            """n_warm untimed steps, then n_steps timed ones between two synchronisations. The
            phase times come from HIP events recorded on the launch stream (read after the last
            step, so nothing waits on the host inside the timed region)."""
            evs = []
            for _ in range(n_warm):
                self.step(False, save_probs, accum)
            torch.cuda.synchronize()
            torch.cuda.reset_peak_memory_stats()
            t0 = time.perf_counter()
            for _ in range(n_steps):
                loss, ev = self.step(True, save_probs, accum)
                evs.append(ev)
            torch.cuda.synchronize()
            wall = time.perf_counter() - t0
            phases = [sum(e[i].elapsed_time(e[i + 1]) for e in evs) for i in range(3)]
            return wall, phases, loss, torch.cuda.max_memory_allocated() / 1e9

        def frac(self, ms_per_step: float) -> float:
            return 6.0 * self.T * self.H * self.V / (ms_per_step * 1e-3) / 1e12 / PEAK_BF16_TFLOPS

    wl = Workload(make_batch(args.workload, dev))
    b, T, H, V = wl.b, wl.T, wl.H, wl.V
    hidden, weight, input_data, loss_fn = wl.hidden, wl.weight, wl.input_data, wl.loss_fn

    # save_probs None: keep the exponentials if the bf16 [T, V] buffer fits the library's default limit
    wall, (t_fwd, t_loss, t_bwd), loss, peak_hbm_gb = wl.run(
        args.steps, args.warmup, False if args.recompute else None)
    saved = main_saved = wl.saved
    ms_per_step = wall * 1e3 / args.steps
    tokens_per_s = T * args.steps / wall

    # The other memory mode, a short leg of its own: the backward recomputes the logits chunk by
    # chunk and nothing of size [T, V] is kept between forward and backward (the reference's
    # memory behaviour, vocab_parallel_head.py:704-713). Same algorithmic flops, one more
    # contraction launch.
    other = None
    if not args.no_other_mode:
        n_other = max(1, min(args.steps, 5))
        o_wall, o_ph, _, o_peak = wl.run(n_other, 1, None if args.recompute else False)
        other = {
            "backward": "saved bf16 exponentials" if wl.saved else "recompute logits",
            "steps": n_other, "ms_per_step": o_wall * 1e3 / n_other,
            "frac": wl.frac(o_wall * 1e3 / n_other),
            "peak_hbm_gb": o_peak,
            "ms": {"lmhead_fwd": o_ph[0] / n_other, "loss_fwd": o_ph[1] / n_other,
                   "loss_bwd+lmhead_bwd": o_ph[2] / n_other},
        }
    saved = main_saved

    # The route an engine with fp32 master weights takes (FusedLMHeadAdapter's default, Megatron's
    # main_grad, vocab_parallel_head.py:870-876): dWeight is ADDED to an fp32 [V, H] buffer by the
    # contraction's epilogue instead of being stored as bf16.
    fp32_accum = None
    if not args.no_other_mode and not args.recompute:
        n_acc = max(1, min(args.steps, 5))
        acc = torch.zeros(V, H, dtype=torch.float32, device=dev)
        a_wall, a_ph, _, a_peak = wl.run(n_acc, 1, None, accum=acc)
        fp32_accum = {"steps": n_acc, "ms_per_step": a_wall * 1e3 / n_acc, "frac": wl.frac(a_wall * 1e3 / n_acc),
                      "peak_hbm_gb": a_peak,
                      "ms": {"lmhead_fwd": a_ph[0] / n_acc, "loss_fwd": a_ph[1] / n_acc,
                             "loss_bwd+lmhead_bwd": a_ph[2] / n_acc}}
        del acc

    # The two backward contractions on their own (median of three): a backward that asks for one
    # gradient launches one contraction, next to the loss backward and the operand preparation
    # (in recompute mode also the recompute pass), so these are upper bounds of the kernels' times.
    def backward_only(want_hidden):
        ts = []
        h_in = hidden.detach().requires_grad_(want_hidden)
        w_in = weight.detach().requires_grad_(not want_hidden)
        wrt = h_in if want_hidden else w_in
        for _ in range(3):
            out = fused_lm_head_logprobs_entropy(h_in, w_in, b["labels"], temperature=1.0,
                                                 save_probs=False if args.recompute else None)
            loss = loss_fn(out.logprobs, out.entropy, input_data,
                           vocab_min_logits=out.vocab_min_logits, vocab_max_logits=out.vocab_max_logits)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            torch.autograd.grad(loss, [wrt])
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1))
        return sorted(ts)[1]

    backward_split = {"dHidden launch sequence": backward_only(True),
                      "dWeight launch sequence": backward_only(False)}

    # Roofline of the MFMA contraction kernels (gemm_nt_sweep / gemm_tn_sweep): one step runs
    # 3 algorithmic GEMMs = 6*T*H*V flops (forward with the softmax epilogue, dHidden, dWeight);
    # with --recompute a fourth launch recomputes the logits and carries no algorithmic flops.
    # Durations are the HIP-event times of the forward and backward library calls on the
    # stream they are launched on (they also contain the merge, operand-prep, transpose and cast
    # kernels, which makes the figure slightly pessimistic).
    gemm_ms = (t_fwd + t_bwd) / args.steps
    algo_flops = 6.0 * T * H * V
    achieved = algo_flops / (gemm_ms * 1e-3) / 1e12
    fwd_tflops = 2.0 * T * H * V / (t_fwd / args.steps * 1e-3) / 1e12

    # The vendor library's plain bf16 GEMM of the forward's shape on this same box, right after
    # the timed steps: what a contraction without the softmax epilogue sustains here (boards are
    # power-limited under this load, so the figure moves from box to box with the kernels').
    lib_tflops = None
    lib_by_shape = None
    if not args.no_library_gemm:
        with torch.no_grad():
            hd, wt = hidden.detach(), weight.detach().t()
            logits = torch.empty(T, V, dtype=torch.bfloat16, device=dev)
            for _ in range(2):
                torch.mm(hd, wt, out=logits)
            a, c = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(5):
                torch.mm(hd, wt, out=logits)
            c.record()
            torch.cuda.synchronize()
            lib_tflops = 2.0 * T * H * V / (a.elapsed_time(c) / 5 * 1e-3) / 1e12
            # the same library at the two backward contractions' shapes and layouts
            lib_by_shape = {"forward [T,H] x [V,H]^T": lib_tflops}
            dh_out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
            dw_out = torch.empty(V, H, dtype=torch.bfloat16, device=dev)
            for name, fn in (("dHidden [T,V] x [V,H]", lambda: torch.mm(logits, weight.detach(), out=dh_out)),
                             ("dWeight [T,V]^T x [T,H]", lambda: torch.mm(logits.t(), hd, out=dw_out))):
                for _ in range(2):
                    fn()
                a.record()
                for _ in range(5):
                    fn()
                c.record()
                torch.cuda.synchronize()
                lib_by_shape[name] = 2.0 * T * H * V / (a.elapsed_time(c) / 5 * 1e-3) / 1e12
            del logits, dh_out, dw_out

    # L2<->fabric bytes per launch. Not measured by this run: constants from rocprofv3 --pmc
    # FETCH_SIZE / WRITE_SIZE runs of this command on this workload (KiB per dispatch, scaled by
    # the factors the same counters show for copy-like kernels of known size, the operand-prep
    # and the bf16 transpose: fetch x2.0, write x1.0); profiles/lmhead_contraction_qwen3-8b.md
    # has the commands and the table. The forward's fetch count moves by +-5 % from launch to
    # launch with L2 hit timing.
    traffic = None
    traffic_detail = None
    traffic_source = None
    if args.workload == "qwen3-8b" and saved:
        kib = 1024.0
        traffic_detail = {
            KERNEL_FWD_SAVE + " forward": 3.1562e7 * kib * 2.0 + 9.729e6 * kib,  # fetch: mean of 7 launches
            KERNEL_DHIDDEN + " dHidden": 2.9199e7 * kib * 2.0 + 2.6419e5 * kib,
            KERNEL_DWEIGHT + " dWeight": (2.9205e7 + 1.5956e5) * kib * 2.0 + 1.2219e6 * kib,  # with its 384-row tail
        }
        traffic = sum(traffic_detail.values()) / 3.0
        traffic_source = ("offline rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command "
                          "(profiles/lmhead_contraction_qwen3-8b.md), mean of the three contraction "
                          "launches; not re-measured by this run")
    final_loss = float(loss.detach().item())
    # The kernel names this line reports, checked against the loaded library (tests/test_bench_contract.py
    # makes the same check a hard failure); a box without a symbol demangler still gets its line.
    try:
        missing = [k for k in (KERNEL_FWD_SAVE, KERNEL_FWD, KERNEL_DHIDDEN, KERNEL_DWEIGHT, KERNEL_RECOMPUTE)
                   if not _lib.has_kernel(k)]
        kernel_names_checked = True
    except (OSError, subprocess.SubprocessError):
        missing, kernel_names_checked = [], False
    if missing:
        sys.exit(f"bench.py names kernels that the loaded library does not contain: {missing}")

    # The other BASELINE shapes, a short timed leg each (same step, saved-exponentials mode), after
    # the default workload's tensors are released. Drawn on the device; small shapes get more
    # warm-up steps (the caching allocator takes a few steps to stop re-splitting its blocks).
    other_workloads = []
    if not args.no_other_workloads and args.workload == "qwen3-8b":
        del wl, b, hidden, weight, input_data, loss_fn, loss
        torch.cuda.empty_cache()
        for name, n_steps, n_warm in (("qwen2.5-0.5b", 40, 20), ("qwen2.5-1.5b", 20, 10), ("qwen3-14b-128k", 3, 1)):
            w2 = Workload(make_batch_on_device(name, dev))
            w_wall, w_ph, _, w_peak = w2.run(n_steps, n_warm, None)
            ms = w_wall * 1e3 / n_steps
            other_workloads.append({
                "workload": f"{name}: {WORKLOADS[name]['desc']}", "tokens": w2.T, "hidden": w2.H, "vocab": w2.V,
                "steps": n_steps, "warmup": n_warm, "ms_per_step": ms, "value": w2.T / (ms * 1e-3),
                "unit": "tokens/s", "frac": w2.frac(ms),
                "backward": "saved bf16 exponentials" if w2.saved else "recompute logits", "peak_hbm_gb": w_peak,
                "ms": {"lmhead_fwd": w_ph[0] / n_steps, "loss_fwd": w_ph[1] / n_steps,
                       "loss_bwd+lmhead_bwd": w_ph[2] / n_steps},
            })
            del w2
            torch.cuda.empty_cache()
        wl = None

    result = {
        "metric": "packed tokens/sec, logprob+entropy+PPO loss fwd+bwd; % bf16 MFMA peak",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: {WORKLOADS[args.workload]['desc']}",
            "tokens": T, "hidden": H, "vocab": V,
            "loss": "PPO clip eps=0.2, rejection sampling ratio in [0.5, 2.0] (token, mask)",
            "final_loss": final_loss,
            "host_reads": "deferred (grpo_loss_fn(defer_host_reads=True): no host wait between the launches of a step)",
            "backward": "saved bf16 exponentials" if saved else "recompute logits",
            "peak_hbm_gb": peak_hbm_gb,
        },
        "pct_bf16_mfma_peak": 100.0 * (algo_flops / (ms_per_step * 1e-3) / 1e12) / PEAK_BF16_TFLOPS,
        "roofline": {
            "kernel": (f"{KERNEL_FWD_SAVE if saved else KERNEL_FWD} (forward), {KERNEL_DHIDDEN} (dHidden), "
                       f"{KERNEL_DWEIGHT} (dWeight)"
                       + ("" if saved else f", {KERNEL_RECOMPUTE} (recompute)")),
            "bound": "mfma",
            "achieved": achieved,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / PEAK_BF16_TFLOPS,
            "traffic": traffic,
            "traffic_source": traffic_source,
            "traffic_bytes_per_launch": traffic_detail,
            "forward_only_tflops": fwd_tflops,
            "library_gemm_same_box_tflops": lib_tflops,
            "library_gemm_by_shape_tflops": lib_by_shape,
            "ms": {"lmhead_fwd": t_fwd / args.steps, "loss_fwd": t_loss / args.steps,
                   "loss_bwd+lmhead_bwd": t_bwd / args.steps},
            "backward_split_ms": backward_split,
            "other_backward_mode": other,
            "recompute_mode_ms": (ms_per_step if not saved else (other["ms_per_step"] if other else None)),
            "fp32_wgrad_accum": fp32_accum,
            "fp32_wgrad_accum_ms": fp32_accum["ms_per_step"] if fp32_accum else None,
            "kernel_names_checked": kernel_names_checked,
        },
        "other_workloads": other_workloads,
    }
    if not args.no_hbm_kernels:
        wl = b = hidden = weight = input_data = loss_fn = loss = None
        torch.cuda.empty_cache()
        result["hbm_rooflines"] = hbm_rooflines(dev)
    if not args.no_cpu_baseline:
        # every core this process may run on (a GPU box grants a share of the host's cores)
        threads = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
        threads = min(threads, int(os.environ.get("OMP_NUM_THREADS", threads)) or threads)
        tps, times = cpu_baseline(args.cpu_sample_tokens, H, WORKLOADS[args.workload]["seed"], threads)
        result["cpu_baseline"] = {
            "value": tps, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"{args.cpu_sample_tokens}-token slice at full vocabulary, fwd+bwd with the "
                      f"PyTorch oracle, median of {len(times)} repeats ("
                      + ", ".join(f"{t:.1f}" for t in times)
                      + " s; the rate is per token, so it scales linearly in T)",
        }
        if not args.no_hbm_kernels:
            result["cpu_baseline_advantages"] = cpu_baseline_advantages(threads)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
