"""The engine shim on a toy causal LM: base model -> fused lm_head -> GRPO loss -> backward, with
fp32 master weights, the bf16 compute copy of ``lm_head.weight``, trailing pad tokens, a
zero-weight micro-batch, and gradients of two micro-batches accumulating in the fp32 ``.grad``
(``areal/engine/fsdp_engine.py:733-812, 1005-1008, 2147-2217``).  Expected values come from the
CPU oracle's closed-form lm_head backward pushed through a CPU copy of the toy base model."""

import copy
import functools
from types import SimpleNamespace

import pytest
import torch
from torch import nn

from areal_amd.config import RejectionSamplingConfig
from areal_amd.engine import FusedLMHeadAdapter
from areal_amd.ppo.actor import grpo_loss_fn
from oracle import logprob as L
from oracle import loss as O

pytestmark = pytest.mark.gpu

H, V = 64, 1536


class ToyBase(nn.Module):
    def __init__(self):
        super().__init__()
        self.embed = nn.Embedding(V, H)
        self.l1 = nn.Linear(H, H)
        self.l2 = nn.Linear(H, H)

    def forward(self, input_ids, **_):
        x = self.embed(input_ids)
        x = x + torch.tanh(self.l1(x))
        x = x + torch.tanh(self.l2(x))
        return SimpleNamespace(last_hidden_state=x * 2.0)


class ToyLM(nn.Module):
    def __init__(self):
        super().__init__()
        self.model = ToyBase()
        self.lm_head = nn.Linear(H, V, bias=False)


def _rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30)).item()


def _micro_batch(T, pad, seed, zero_weight=False):
    g = torch.Generator().manual_seed(seed)
    n = T - pad
    ids = torch.randint(0, V, (1, T), generator=g)
    mask = torch.rand(n, generator=g) > 0.3
    if zero_weight:
        mask[:] = False
    return dict(ids=ids, n=n, pad=pad, mask=mask, adv=torch.randn(n, generator=g),
                noise=torch.randn(n, generator=g) * 0.1)


def _weight_fn(d):
    return d["loss_mask"].count_nonzero()


@pytest.mark.parametrize("fused", [True, False], ids=["fused_fp32_accum", "autograd_cast"])
def test_adapter_two_micro_batches_accumulate_into_fp32_master_grad(dev, fused):
    torch.manual_seed(0)
    lm = ToyLM()  # fp32 parameters: the master weights
    cpu_lm = copy.deepcopy(lm)
    lm.to(dev)
    adapter = FusedLMHeadAdapter(lm, temperature=1.0, fuse_wgrad_accumulation=fused)
    rs = dict(level="token", action="mask", metric="ratio", upper=2.0, lower=0.5)
    loss_fn = functools.partial(grpo_loss_fn, eps_clip=0.2, eps_clip_higher=None, c_clip=None,
                                rejection_sampling=RejectionSamplingConfig(**rs))
    specs = [_micro_batch(320, 19, 1), _micro_batch(256, 40, 2, zero_weight=True), _micro_batch(200, 0, 3)]

    # forward-only pass first (the engine's compute_logp): proximal = behaviour log-probs + noise
    mbs = []
    for sp in specs:
        inputs = dict(input_ids=sp["ids"].to(dev))
        prox = adapter.compute_logprobs(inputs, pad_length=sp["pad"])
        assert prox.shape == (sp["n"],) and not prox.requires_grad
        sp["prox"] = prox.cpu()
        sp["old"] = sp["prox"] + sp["noise"]
        mbs.append(dict(model_inputs=inputs, pad_length=sp["pad"],
                        mb_input=dict(logprobs=sp["old"].to(dev), advantages=sp["adv"].to(dev),
                                      loss_mask=sp["mask"].to(dev), prox_logp=prox)))
    losses = adapter.forward_backward_batch(mbs, loss_fn, _weight_fn)
    assert losses[1].item() == 0.0  # the zero-weight micro-batch
    wg = lm.lm_head.weight.grad
    assert wg is not None and wg.dtype == torch.float32 and wg.shape == (V, H)

    # oracle: the same steps on the CPU copy
    total = float(sum(int(sp["mask"].sum()) for sp in specs))
    w_bf16 = cpu_lm.lm_head.weight.detach().bfloat16()
    dw_want = torch.zeros(V, H)
    want_losses = []
    for sp in specs:
        hidden = cpu_lm.model(sp["ids"]).last_hidden_state.squeeze(0)
        h_bf16 = hidden.detach().bfloat16()
        labels = torch.roll(sp["ids"], -1, -1)[0]
        n = sp["n"]
        lp = L.lm_head_logprobs_entropy(h_bf16, w_bf16, labels)[0][:n]
        # 2e-3 is the bound on identical bf16 inputs; here the toy base model ran in fp32 on two
        # devices, so an occasional hidden state rounds to the neighbouring bf16 value
        assert (sp["prox"] - lp).abs().max() < 4e-3
        if int(sp["mask"].sum()) == 0:
            want_losses.append(0.0)
            continue
        lp_o = lp.clone().requires_grad_(True)
        lo, _ = O.ppo_actor_loss(lp_o, sp["prox"], sp["old"], sp["adv"], 0.2, sp["mask"], rejection_sampling_cfg=rs)
        scale = float(sp["mask"].sum()) / total
        (lo * scale).backward()
        want_losses.append(float(lo.detach() * scale))
        g_full = torch.zeros(labels.numel())
        g_full[:n] = lp_o.grad
        dh, dw = L.lm_head_backward(h_bf16, w_bf16, labels, g_full)
        dw_want += dw
        hidden.backward(dh)  # through the toy base model: accumulates in cpu_lm's .grad
    for got, want in zip(losses, want_losses):
        assert got.item() == pytest.approx(want, rel=2e-3, abs=1e-5)
    assert _rel(wg.cpu(), dw_want) < 1e-2
    for name, p in lm.model.named_parameters():
        want = dict(cpu_lm.model.named_parameters())[name].grad
        assert p.grad is not None and p.grad.dtype == torch.float32
        assert _rel(p.grad.cpu(), want) < 1e-2, name


def test_adapter_zero_weight_micro_batch_reaches_every_parameter(dev):
    torch.manual_seed(1)
    lm = ToyLM().to(dev)
    adapter = FusedLMHeadAdapter(lm)
    sp = _micro_batch(128, 5, 9, zero_weight=True)
    loss_fn = functools.partial(grpo_loss_fn, eps_clip=0.2, eps_clip_higher=None, c_clip=None)
    n = sp["n"]
    mb = dict(logprobs=torch.zeros(n, device=dev), advantages=sp["adv"].to(dev), loss_mask=sp["mask"].to(dev),
              prox_logp=torch.zeros(n, device=dev))
    loss = adapter.compute_logprobs_and_loss(dict(input_ids=sp["ids"].to(dev)), mb, loss_fn, _weight_fn, 1.0,
                                             pad_length=sp["pad"])
    assert loss.item() == 0.0
    loss.backward()
    for name, p in lm.named_parameters():
        assert p.grad is not None and not p.grad.any(), name


def test_adapter_bf16_parameters_get_bf16_gradients_and_bad_modules_are_refused(dev):
    torch.manual_seed(2)
    lm = ToyLM().to(dev).bfloat16()
    adapter = FusedLMHeadAdapter(lm)
    sp = _micro_batch(192, 0, 4)
    inputs = dict(input_ids=sp["ids"].to(dev))
    prox = adapter.compute_logprobs(inputs)
    mb = dict(logprobs=prox + sp["noise"].to(dev), advantages=sp["adv"].to(dev), loss_mask=sp["mask"].to(dev),
              prox_logp=prox)
    loss_fn = functools.partial(grpo_loss_fn, eps_clip=0.2, eps_clip_higher=None, c_clip=None)
    adapter.forward_backward_batch([dict(model_inputs=inputs, mb_input=mb)], loss_fn, _weight_fn)
    assert lm.lm_head.weight.grad.dtype == torch.bfloat16 and lm.lm_head.weight.grad.any()
    with pytest.raises(TypeError):
        FusedLMHeadAdapter(nn.Linear(4, 4))


def test_adapter_reuses_the_bf16_compute_copy_until_the_master_weight_changes(dev):
    """The bf16 copy of an fp32 master lm_head.weight is made once per version of the parameter:
    micro-batches and forward-only calls share it; an in-place update (an optimizer step) makes
    the next call cast again, and the log-probabilities follow the new weights."""
    torch.manual_seed(3)
    lm = ToyLM().to(dev)
    adapter = FusedLMHeadAdapter(lm)
    sp = _micro_batch(192, 0, 4)
    inputs = dict(input_ids=sp["ids"].to(dev))
    lp0 = adapter.compute_logprobs(inputs)
    copy0 = adapter._compute_copy_value
    assert copy0.dtype == torch.bfloat16 and torch.equal(copy0, lm.lm_head.weight.detach().bfloat16())
    mb = dict(logprobs=lp0 + sp["noise"].to(dev), advantages=sp["adv"].to(dev), loss_mask=sp["mask"].to(dev),
              prox_logp=lp0)
    loss_fn = functools.partial(grpo_loss_fn, eps_clip=0.2, eps_clip_higher=None, c_clip=None)
    adapter.forward_backward_batch([dict(model_inputs=inputs, mb_input=mb)] * 2, loss_fn, _weight_fn)
    assert adapter._compute_copy_value is copy0  # forward-only call and both micro-batches: one cast
    assert torch.equal(adapter.compute_logprobs(inputs), lp0)
    with torch.no_grad():
        lm.lm_head.weight.mul_(1.5)  # what an optimizer step does: in place, the version counter moves
    lp1 = adapter.compute_logprobs(inputs)
    assert adapter._compute_copy_value is not copy0
    assert torch.equal(adapter._compute_copy_value, lm.lm_head.weight.detach().bfloat16())
    assert not torch.allclose(lp1, lp0)


def test_step_is_queued_without_waiting_for_the_gpu(dev):
    """Forward, loss and backward of one micro-batch with deferred host reads: no call of the
    step may synchronise with the device before its last launch is queued (the saved-mode
    backward is queued before the host looks at the forward's status; the loss's host scalars and
    reduced statistics are read afterwards).  Results equal those of the synchronising calls."""
    from areal_amd.functional import DeferredFloat, fused_lm_head_logprobs_entropy

    T, H, V = 1536, 256, 4096
    g = torch.Generator().manual_seed(11)
    hidden = torch.randn(T, H, generator=g).bfloat16().to(dev)
    weight = (torch.randn(V, H, generator=g) * 0.05).bfloat16().to(dev)
    labels = torch.randint(0, V, (T,), generator=g).to(dev)
    cu = torch.tensor([0, 500, 1100, 1536], dtype=torch.int32, device=dev)
    with torch.no_grad():
        logp0 = fused_lm_head_logprobs_entropy(hidden, weight, labels).logprobs
    old = logp0 + (torch.randn(T, generator=g) * 0.3).to(dev)
    data = dict(logprobs=old, advantages=torch.randn(T, generator=g).to(dev),
                loss_mask=(torch.rand(T, generator=g) > 0.2).to(dev), prox_logp=logp0, cu_seqlens=cu)
    rs = RejectionSamplingConfig(level="token", action="mask", metric="ratio", lower=0.5, upper=2.0)
    loss_fn = functools.partial(grpo_loss_fn, eps_clip=0.2, eps_clip_higher=None, c_clip=None,
                                rejection_sampling=rs, stats_mode="reduced")

    def step(defer):
        h = hidden.clone().requires_grad_(True)
        w = weight.clone().requires_grad_(True)
        stats = {}
        out = fused_lm_head_logprobs_entropy(h, w, labels, save_probs=True)
        loss = loss_fn(out.logprobs, out.entropy, data, stats=stats, defer_host_reads=defer)
        loss.backward()
        return loss, h.grad, w.grad, stats

    want_loss, want_dh, want_dw, want_stats = step(False)
    step(True)  # warm-up: allocator and pinned-memory pools
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("error")
    try:
        loss, dh, dw, stats = step(True)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    assert isinstance(stats["scalar/n_valid_tokens"], DeferredFloat)
    assert torch.equal(loss, want_loss) and torch.equal(dh, want_dh) and torch.equal(dw, want_dw)
    assert float(stats["scalar/n_valid_tokens"]) == want_stats["scalar/n_valid_tokens"]
    assert float(stats["scalar/rs_filtered_fraction"]) == want_stats["scalar/rs_filtered_fraction"]
    red = stats["reduction"]
    for key, val in red.results.items():
        assert want_stats[key] == val, key
    for name, count in red.denominators.items():
        assert want_stats["denominator/" + name] == count

    # a NaN in the proximal log-probs: the synchronising call raises, the deferred one poisons the loss
    bad = dict(data, prox_logp=logp0.clone().index_fill_(0, torch.tensor([7], device=dev), float("nan")))
    out = fused_lm_head_logprobs_entropy(hidden, weight, labels)
    with pytest.raises(RuntimeError, match="prox_logp contains NaN or Inf"):
        loss_fn(out.logprobs, out.entropy, bad)
    assert torch.isnan(loss_fn(out.logprobs, out.entropy, bad, defer_host_reads=True))
