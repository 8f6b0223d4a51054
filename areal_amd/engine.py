"""Engine-side glue: what ``FSDPEngine`` does between the model's last hidden states and the
scaled scalar loss (``areal/engine/fsdp_engine.py:2076-2217``), with the logits replaced by the
fused lm_head kernel.

The reference computes ``logits = model(...).logits`` and then reads them three times
(log-softmax, entropy, min/max). Here the caller passes the final hidden states and the
``lm_head`` weight; label roll, padding trim and loss scaling follow the reference.
"""

from __future__ import annotations

from collections.abc import Callable
from typing import Any

import torch

from areal_amd.functional.lm_head import fused_lm_head_logprobs_entropy


def _labels(inputs: dict[str, Any]) -> torch.Tensor:
    labels = inputs.get("rolled_input_ids")
    if labels is None:
        labels = torch.roll(inputs["input_ids"], shifts=-1, dims=-1)
    if labels.ndim == 2 and labels.shape[0] == 1:
        labels = labels.squeeze(0)
    return labels


def compute_logprobs(
    hidden: torch.Tensor,
    lm_head_weight: torch.Tensor,
    inputs: dict[str, Any],
    temperature: float = 1.0,
    pad_length: int = 0,
) -> torch.Tensor:
    """Forward-only label log-probabilities of a packed micro-batch
    (``fsdp_engine.py:2107-2134`` with the lm_head folded in)."""
    if hidden.ndim == 3 and hidden.shape[0] == 1:
        hidden = hidden.squeeze(0)
    with torch.no_grad():
        out = fused_lm_head_logprobs_entropy(
            hidden, lm_head_weight, _labels(inputs), temperature=temperature
        )
    logprobs = out.logprobs
    return logprobs[:-pad_length] if pad_length > 0 else logprobs


def compute_logprobs_and_loss(
    hidden: torch.Tensor,
    lm_head_weight: torch.Tensor,
    model_inputs: dict[str, Any],
    mb_input: dict[str, Any],
    loss_fn: Callable[..., torch.Tensor],
    loss_weight_fn: Callable[[dict[str, Any]], torch.Tensor],
    total_loss_weight: torch.Tensor | float,
    temperature: float = 1.0,
    pad_length: int = 0,
    loss_multiplier: float = 1.0,
    save_probs: bool | None = None,
    weight_grad_accum: torch.Tensor | None = None,
) -> torch.Tensor:
    """Scaled loss of one micro-batch (``fsdp_engine.py:2147-2217``).

    ``weight_grad_accum`` is handed to ``fused_lm_head_logprobs_entropy`` (an fp32 ``[V, H]``
    buffer the weight gradient is added to by the kernel; see ``FusedLMHeadAdapter``).

    ``save_probs`` is handed to ``fused_lm_head_logprobs_entropy`` (keep the bf16 softmax
    exponentials for the backward, or recompute the logits there).

    ``loss_fn(logprobs, entropy, mb_input, vocab_min_logits=..., vocab_max_logits=...)`` is
    the actor loss (normally a ``functools.partial`` of ``grpo_loss_fn``).  The per-token
    vocabulary min/max come out of the same kernel sweep instead of a second pass over logits.
    """
    local_weight = loss_weight_fn(mb_input)
    if local_weight == 0:
        # a zero that reaches both operands, as the reference's `logits.mean() * 0.0` does
        # (fsdp_engine.py:2158-2159): every parameter still receives a (zero) gradient
        return (hidden.float().mean() + lm_head_weight[:1].float().mean()) * 0.0
    if hidden.ndim == 3 and hidden.shape[0] == 1:
        hidden = hidden.squeeze(0)
    out = fused_lm_head_logprobs_entropy(
        hidden, lm_head_weight, _labels(model_inputs), temperature=temperature,
        save_probs=save_probs, weight_grad_accum=weight_grad_accum,
    )
    logprobs, entropy = out.logprobs, out.entropy
    vmin, vmax = out.vocab_min_logits, out.vocab_max_logits
    if pad_length > 0:
        logprobs, entropy = logprobs[:-pad_length], entropy[:-pad_length]
        vmin, vmax = vmin[:-pad_length], vmax[:-pad_length]
    loss = loss_fn(logprobs, entropy, mb_input, vocab_min_logits=vmin, vocab_max_logits=vmax)
    loss_scale = local_weight / total_loss_weight * loss_multiplier
    return loss * loss_scale


def _last_hidden_state(output) -> torch.Tensor:
    if torch.is_tensor(output):
        return output
    hidden = getattr(output, "last_hidden_state", None)
    if hidden is not None:
        return hidden
    if isinstance(output, (tuple, list)):
        return output[0]
    if isinstance(output, dict):
        return output["last_hidden_state"]
    raise TypeError(f"cannot find the last hidden states in a {type(output).__name__}")


class FusedLMHeadAdapter:
    """What ``FSDPEngine`` does with a causal LM per micro-batch (``fsdp_engine.py:733-772``,
    ``:2107-2217``), with the ``lm_head`` matmul folded into the fused kernel.

    ``module`` is a causal LM in the Hugging Face layout: ``module.model`` maps the model inputs
    to the final hidden states and ``module.lm_head`` is the output projection (only its
    ``weight`` and optional ``bias`` are read; its ``forward`` is never called, so no ``[T, V]``
    logits exist).

    Mixed precision follows the engine's arrangement (``fsdp_engine.py:1005-1008,1044-1046``):
    parameters are stored in the optimizer dtype (fp32 master weights) and computed with in
    ``compute_dtype`` (bf16).  The kernel gets a bf16 compute copy of ``lm_head.weight`` made
    per micro-batch.  Its gradient reaches the fp32 parameter in one of two ways:

    * ``fuse_wgrad_accumulation=True`` (default): the dWeight contraction adds into the fp32
      ``lm_head.weight.grad`` directly (created as zeros when missing), so gradients of several
      micro-batches accumulate in fp32 without a bf16 ``[V, H]`` intermediate, the arrangement
      of Megatron's fp32 ``main_grad`` (``vocab_parallel_head.py:873-879``);
    * otherwise autograd routes a bf16 ``dWeight`` through the cast back to fp32 and its
      ``AccumulateGrad`` adds it to ``.grad``.

    A bf16 ``lm_head.weight`` is used as it is and receives a bf16 gradient through autograd.
    """

    def __init__(
        self,
        module: torch.nn.Module,
        *,
        temperature: float = 1.0,
        compute_dtype: torch.dtype = torch.bfloat16,
        fuse_wgrad_accumulation: bool = True,
        save_probs: bool | None = None,
    ):
        if not hasattr(module, "model") or not hasattr(module, "lm_head"):
            raise TypeError("FusedLMHeadAdapter needs a module with `.model` and `.lm_head`")
        if compute_dtype != torch.bfloat16:
            raise ValueError(f"the fused LM head computes in bf16; got {compute_dtype}")
        self.module = module
        self.temperature = temperature
        self.compute_dtype = compute_dtype
        self.fuse_wgrad_accumulation = fuse_wgrad_accumulation
        self.save_probs = save_probs
        self._compute_copy_key = None
        self._compute_copy_value = None

    # -- pieces --------------------------------------------------------------------------
    def hidden_states(self, model_inputs: dict[str, Any]) -> torch.Tensor:
        """``[T, H]`` final hidden states in the compute dtype: the base model's forward, i.e.
        ``self.model(**inputs)`` of ``fsdp_engine.py:759-761`` stopped in front of ``lm_head``."""
        hidden = _last_hidden_state(self.module.model(**model_inputs))
        if hidden.ndim == 3 and hidden.shape[0] == 1:
            hidden = hidden.squeeze(0)
        return hidden.to(self.compute_dtype)

    def _compute_copy(self, param: torch.Tensor) -> torch.Tensor:
        """Detached compute-dtype copy of the master weight, made once per version of the
        parameter: the micro-batches of a step (and forward-only calls between optimizer steps)
        share it, and an in-place update of the parameter (the optimizer's) bumps its version
        counter and invalidates it.  At Qwen3-8B size the cast reads 2.5 GB and writes 1.2 GB."""
        key = (param.data_ptr(), param._version, tuple(param.shape), param.device)
        if self._compute_copy_key != key:
            self._compute_copy_value = param.detach().to(self.compute_dtype)
            self._compute_copy_key = key
        return self._compute_copy_value

    def _weight(self, hidden: torch.Tensor):
        """(compute copy of lm_head.weight, fp32 accumulator or None)."""
        param = self.module.lm_head.weight
        if param.dtype == self.compute_dtype:
            return param, None
        if not torch.is_grad_enabled():
            return self._compute_copy(param), None
        fused = (
            self.fuse_wgrad_accumulation
            and param.dtype == torch.float32
            and param.requires_grad
            and torch.is_grad_enabled()
            and hidden.requires_grad  # the backward is reached through the hidden states
        )
        if not fused:
            return param.to(self.compute_dtype), None  # autograd casts the gradient back
        if param.grad is None:
            param.grad = torch.zeros_like(param, memory_format=torch.contiguous_format)
        return self._compute_copy(param), param.grad

    def _bias(self):
        return getattr(self.module.lm_head, "bias", None)

    # -- the engine's two per-micro-batch computations -----------------------------------
    def compute_logprobs(self, model_inputs: dict[str, Any], pad_length: int = 0) -> torch.Tensor:
        """Forward-only label log-probabilities (``fsdp_engine.py:2107-2134, 2219-2249``)."""
        with torch.no_grad():
            hidden = self.hidden_states(model_inputs)
            weight, _ = self._weight(hidden)
            out = fused_lm_head_logprobs_entropy(
                hidden, weight, _labels(model_inputs), temperature=self.temperature, bias=self._bias()
            )
        logprobs = out.logprobs
        return logprobs[:-pad_length] if pad_length > 0 else logprobs

    def compute_logprobs_and_loss(
        self,
        model_inputs: dict[str, Any],
        mb_input: dict[str, Any],
        loss_fn: Callable[..., torch.Tensor],
        loss_weight_fn: Callable[[dict[str, Any]], torch.Tensor],
        total_loss_weight: torch.Tensor | float,
        pad_length: int = 0,
        loss_multiplier: float = 1.0,
    ) -> torch.Tensor:
        """Scaled loss of one micro-batch (``fsdp_engine.py:2147-2217``)."""
        hidden = self.hidden_states(model_inputs)
        local_weight = loss_weight_fn(mb_input)
        if local_weight == 0:
            # zero with a graph edge to the base model and to lm_head.weight
            # (fsdp_engine.py:2158-2159)
            return (hidden.float().mean() + self.module.lm_head.weight[:1].float().mean()) * 0.0
        weight, accum = self._weight(hidden)
        out = fused_lm_head_logprobs_entropy(
            hidden, weight, _labels(model_inputs), temperature=self.temperature, bias=self._bias(),
            save_probs=self.save_probs, weight_grad_accum=accum,
        )
        logprobs, entropy = out.logprobs, out.entropy
        vmin, vmax = out.vocab_min_logits, out.vocab_max_logits
        if pad_length > 0:
            logprobs, entropy = logprobs[:-pad_length], entropy[:-pad_length]
            vmin, vmax = vmin[:-pad_length], vmax[:-pad_length]
        loss = loss_fn(logprobs, entropy, mb_input, vocab_min_logits=vmin, vocab_max_logits=vmax)
        return loss * (local_weight / total_loss_weight * loss_multiplier)

    def forward_backward_batch(
        self,
        micro_batches: list[dict[str, Any]],
        loss_fn: Callable[..., torch.Tensor],
        loss_weight_fn: Callable[[dict[str, Any]], torch.Tensor],
        loss_multiplier: float = 1.0,
    ) -> list[torch.Tensor]:
        """``train_batch`` without the optimizer (``fsdp_engine.py:774-812``): the total loss
        weight over the micro-batches (``core/train_engine.py:30-65``, one rank), then forward
        and backward of each.  A micro-batch is ``dict(model_inputs=..., mb_input=...,
        pad_length=...)``.  Returns the detached scaled losses."""
        weights = [loss_weight_fn(mb["mb_input"]) for mb in micro_batches]
        dev = next((w.device for w in weights if torch.is_tensor(w)), None)
        total = torch.stack(
            [torch.as_tensor(w, device=dev).detach().to(torch.float32) for w in weights]
        ).sum().clone()
        assert total > 0, "Global total loss weight must be positive after all_reduce"
        losses = []
        for mb in micro_batches:
            loss = self.compute_logprobs_and_loss(
                mb["model_inputs"], mb["mb_input"], loss_fn, loss_weight_fn, total,
                pad_length=mb.get("pad_length", 0), loss_multiplier=loss_multiplier,
            )
            loss.backward()
            losses.append(loss.detach())
        return losses
