"""areal_actor_loss_static (scratch in a static device array, no allocation on the call path)
against areal_actor_loss (caller's workspace): bit-identical outputs, on two calls in a row, the
second with a smaller input, for token-level and sequence-level options."""

import ctypes

import pytest
import torch

from areal_amd import _lib

pytestmark = pytest.mark.gpu

_OUT_F32 = ("dlp", "stat_loss", "ratio", "approx_kl", "behave_w", "behave_kl")
_OUT_U8 = ("clip", "dual", "new_mask", "behave_mask")


def _inputs(n, n_seqs, seed, dev):
    g = torch.Generator().manual_seed(seed)
    lp = torch.randn(n, generator=g) * 0.7 - 1.5
    prox = lp + torch.randn(n, generator=g) * 0.2
    old = prox + torch.randn(n, generator=g) * 0.4
    adv = torch.randn(n, generator=g)
    mask = torch.rand(n, generator=g) > 0.25
    cuts = torch.sort(torch.randperm(n - 1, generator=g)[: n_seqs - 1] + 1).values
    cu = torch.cat([torch.tensor([0]), cuts, torch.tensor([n])]).to(torch.int32)
    longest = int((cu[1:] - cu[:-1]).argmax())
    old[cu[longest]:cu[longest + 1]] -= 1.5  # one sequence far off-policy: rejected at either level
    mask[cu[longest]] = True
    return [t.to(dev) for t in (lp, prox, old, adv, mask, cu)]


def _cfg(seq_level):
    c = _lib.LossConfig()
    c.loss_kind = 0
    c.clip_lo, c.clip_hi = 0.8, 1.28
    c.has_c_clip, c.c_clip = 1, 3.0
    c.seq_is = int(seq_level)
    c.rs_enabled = 1
    c.rs_seq_level = int(seq_level)
    c.rs_clamp = 0
    c.rs_metric = 0
    c.rs_agg = 1
    c.rs_upper, c.rs_has_lower, c.rs_lower = 2.0, 1, 0.5
    return c


def _call(lib, static, cfg, lp, prox, old, adv, mask, cu, dev):
    n, n_seqs = lp.numel(), cu.numel() - 1
    o = {k: torch.full((n,), -7.0, device=dev) for k in _OUT_F32}
    o.update({k: torch.full((n,), 9, dtype=torch.uint8, device=dev) for k in _OUT_U8})
    o["loss"] = torch.full((), -7.0, device=dev)
    o["counters"] = torch.full((8,), -7.0, dtype=torch.float64, device=dev)
    p = _lib.ptr
    args = [p(lp), p(prox), p(old), p(adv), p(mask), p(cu), n, n_seqs, 0, ctypes.byref(cfg),
            p(o["loss"]), p(o["dlp"]), p(o["stat_loss"]), p(o["ratio"]), p(o["approx_kl"]), p(o["clip"]),
            p(o["dual"]), p(o["new_mask"]), p(o["behave_w"]), p(o["behave_kl"]), p(o["behave_mask"]),
            p(o["counters"])]
    if static:
        rc = lib.areal_actor_loss_static(*args, _lib.stream_ptr(dev))
    else:
        nbytes = lib.areal_actor_loss_workspace_bytes(n, n_seqs)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        rc = lib.areal_actor_loss(*args, p(ws), nbytes, _lib.stream_ptr(dev))
    assert rc == 0, rc
    torch.cuda.synchronize()
    return o


@pytest.mark.parametrize("seq_level", [False, True], ids=["token", "sequence"])
def test_static_scratch_entry_point_matches_workspace_entry_point(dev, seq_level):
    lib = _lib.load()
    cfg = _cfg(seq_level)
    # two calls in a row on the shared scratch: a large batch, then a smaller one
    for n, n_seqs, seed in ((300_000, 700, 5), (4_099, 13, 6)):
        batch = _inputs(n, n_seqs, seed, dev)
        got = _call(lib, True, cfg, *batch, dev)
        want = _call(lib, False, cfg, *batch, dev)
        print("counters", n, want["counters"].tolist(), flush=True)
        for k in want:
            assert torch.equal(got[k], want[k]), (k, n)
        n_valid, n_filtered = float(want["counters"][1]), float(want["counters"][3])
        assert n_valid == float(batch[4].sum()) and 0 < n_filtered < n_valid


def test_static_scratch_entry_point_rejects_too_many_sequences(dev):
    lib = _lib.load()
    cfg = _cfg(True)
    n = 70_000
    lp, prox, old, adv, mask, _ = _inputs(n, 3, 7, dev)
    cu = torch.arange(n + 1, dtype=torch.int32, device=dev)  # 70000 sequences of one token
    p = _lib.ptr
    counters = torch.zeros(8, dtype=torch.float64, device=dev)
    new_mask = torch.zeros(n, dtype=torch.uint8, device=dev)
    w = torch.zeros(n, device=dev)
    null = ctypes.c_void_p(0)
    rc = lib.areal_actor_loss_static(p(lp), p(prox), p(old), p(adv), p(mask), p(cu), n, n, 0,
                                     ctypes.byref(cfg), null, null, null, null, null, null, null,
                                     p(new_mask), p(w), null, null, p(counters), _lib.stream_ptr(dev))
    assert rc == -5
