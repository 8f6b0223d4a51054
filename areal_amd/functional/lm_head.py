"""Fused lm_head -> log-softmax -> label log-prob + entropy on MI355X.

Host-side counterpart of the reference's chunked LM head
(``areal/models/mcore/vocab_parallel_head.py:560-938`` and its wrapper
``chunked_lm_head_logprobs_entropy`` at ``:941-982``): same outputs
(``ChunkedLMHeadOutput``), same error behaviour.  The arithmetic runs in the HIP kernels of
``csrc/lmhead.hip`` through the C ABI.

Two ways of carrying state to the backward:

* ``save_probs=False``: what the reference does -- row max and sum of exponentials per token,
  never a ``[T, V]`` tensor; the backward recomputes the logits chunk by chunk
  (``vocab_parallel_head.py:806-829``).
* ``save_probs=True``: the forward also writes the softmax exponentials as a bf16 ``[T, V]``
  tensor (2 bytes per logit), relative to a per-row reference estimated before the sweep; the
  backward contracts that buffer as it is (the per-row factor of dlogits goes to the output
  rows of dHidden and to the hidden states for dWeight) and skips the recomputation, a quarter
  of the step's matrix work.  The reference's logits-in path saves the same amount through
  autograd; 288 GB of HBM make it the default while it fits ``SAVE_PROBS_BYTES_LIMIT`` and
  60 % of the memory still available.  If some row's maximum logit lies more than 100 binades
  (69 nats at temperature 1) above its estimate, the kernel reports it, repeats the sweep
  without saving on the device (so the outputs are right without a host round trip), and the
  backward recomputes instead.
"""

from __future__ import annotations

import math
from typing import NamedTuple

import torch

from areal_amd import _lib

# Default budget for the backward workspace (bf16 dlogits of one token chunk in two layouts,
# plus transposed operands).  An MI355X has 288 GB of HBM, so one chunk normally covers the
# whole micro-batch.
DEFAULT_BWD_WORKSPACE_BYTES = 24 << 30

# save_probs=None keeps the exponentials when the bf16 [T, V] buffer is at most this large.
SAVE_PROBS_BYTES_LIMIT = 40 << 30


def _round_up(x: int, m: int) -> int:
    return (x + m - 1) // m * m


def _available_bytes(dev: torch.device) -> int:
    """Device memory the allocator can still hand out: free on the device plus what the caching
    allocator holds but has not given to a tensor."""
    free, _ = torch.cuda.mem_get_info(dev)
    return free + torch.cuda.memory_reserved(dev) - torch.cuda.memory_allocated(dev)


class ChunkedLMHeadOutput(NamedTuple):
    """Per-token outputs produced without materialising ``[T, V]`` logits.

    Field names and order follow ``vocab_parallel_head.py:497-506``.
    """

    logprobs: torch.Tensor
    entropy: torch.Tensor
    vocab_min_logits: torch.Tensor
    vocab_max_logits: torch.Tensor
    vocab_mean_logits: torch.Tensor
    vocab_norm_logits: torch.Tensor


def default_token_chunk(T: int, H: int, V: int, budget: int = DEFAULT_BWD_WORKSPACE_BYTES) -> int:
    """Largest token chunk (multiple of 256) whose backward workspace fits ``budget``: bf16
    dlogits of the chunk plus the transposed weight (and, when ``T`` is not a multiple of 64,
    transposed copies of the last chunk's hidden states and dlogits)."""
    ragged = T % 64 != 0
    per_token = 2 * V + 64 + (2 * (V + H) if ragged else 0)
    fixed = 2 * H * (V + 64)
    chunk = max((budget - fixed) // per_token, 256)
    chunk = (chunk // 256) * 256
    return int(min(max(chunk, 256), max(T, 1)))


class _FusedLMHead(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx, hidden, weight, bias, labels, temperature, logit_scale, token_chunk, save_probs,
        with_moments, weight_grad_accum,
    ):
        lib = _lib.load()
        dev = _lib.require_gpu(hidden, weight, labels, bias)
        H = hidden.size(-1)
        V = weight.size(0)
        hidden_2d = hidden.reshape(-1, H).contiguous()
        weight_c = weight.contiguous()
        labels_1d = labels.reshape(-1).to(torch.int64).contiguous()
        T = hidden_2d.size(0)
        bias_f = bias.detach().float().contiguous() if bias is not None else None

        # vocabulary mean / norm cost two more operations per logit in the sweep's epilogue: they
        # are computed only on request
        outs = [torch.empty(labels.shape, dtype=torch.float32, device=dev) for _ in range(4)]
        outs += [
            torch.empty(labels.shape, dtype=torch.float32, device=dev) if with_moments else None
            for _ in range(2)
        ]
        outs += [torch.empty(T, dtype=torch.float32, device=dev) for _ in range(2)]
        logprobs, entropy, vmin, vmax, vmean, vnorm, row_max, sum_exp = outs
        # the caller has ruled out no_grad mode
        needs_grad = any(ctx.needs_input_grad[:2]) or weight_grad_accum is not None
        if save_probs is None:
            need = 2 * _round_up(T, 128) * _round_up(V, 64)
            save_probs = need <= SAVE_PROBS_BYTES_LIMIT and need <= 0.6 * _available_bytes(dev)
        probs = probs_ref = probs_status = None
        if save_probs and needs_grad and T > 0:
            # rows padded to 128, columns to 64: areal_lmhead_probs_bytes(T, V)
            probs = torch.empty(
                (_round_up(T, 128), _round_up(V, 64)), dtype=torch.bfloat16, device=dev
            )
            probs_ref = torch.empty(T, dtype=torch.float32, device=dev)
            probs_status = torch.empty(1, dtype=torch.int32, device=dev)
        ctx.status_host = ctx.status_event = None
        if T > 0:
            nbytes = lib.areal_lmhead_fwd_workspace_bytes(T, H, V)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            rc = lib.areal_lmhead_fwd(
                _lib.ptr(hidden_2d), _lib.ptr(weight_c), _lib.ptr(bias_f), _lib.ptr(labels_1d),
                T, H, V, 1.0 / temperature, logit_scale,
                *[_lib.ptr(o) for o in outs],
                _lib.ptr(probs), probs.numel() * 2 if probs is not None else 0,
                _lib.ptr(probs_ref), _lib.ptr(probs_status),
                _lib.ptr(ws), nbytes, _lib.stream_ptr(dev),
            )
            _lib.check(rc, "areal_lmhead_fwd")
            if probs_status is not None:
                # Whether every row's saved exponentials are in range travels to pinned host
                # memory behind the forward, so the backward reads it without a device-to-host
                # copy of its own between the loss and its first launch.
                ctx.status_host = torch.empty(1, dtype=torch.int32, pin_memory=True)
                ctx.status_host.copy_(probs_status, non_blocking=True)
                ctx.status_event = torch.cuda.Event()
                ctx.status_event.record(torch.cuda.current_stream(dev))

        ctx.save_for_backward(hidden_2d, weight_c, labels_1d, row_max, sum_exp)
        # Plain attributes, not saved tensors: the backward rewrites entries of probs in place.
        ctx.probs = probs
        ctx.probs_ref = probs_ref
        ctx.probs_status = probs_status
        ctx.label_logprobs = logprobs.detach().reshape(-1).clone() if probs is not None else None
        ctx.bias_f = bias_f
        ctx.temperature = temperature
        ctx.logit_scale = logit_scale
        ctx.token_chunk = token_chunk
        ctx.hidden_shape = hidden.shape
        ctx.weight_dtype = weight.dtype
        ctx.bias_dtype = bias.dtype if bias is not None else None
        ctx.weight_grad_accum = weight_grad_accum
        ctx.set_materialize_grads(False)
        ctx.mark_non_differentiable(*[o for o in (entropy, vmin, vmax, vmean, vnorm) if o is not None])
        return tuple(outs[:6])

    @staticmethod
    def backward(ctx, grad_logprobs, *unused):
        hidden_2d, weight_c, labels_1d, row_max, sum_exp = ctx.saved_tensors
        need_h, need_w, need_b = ctx.needs_input_grad[:3]
        want_h = need_h
        # dWeight goes straight into the caller's fp32 accumulator when one was given (the master
        # weight's .grad): the contraction's epilogue adds to it, nothing of size [V, H] is
        # allocated and no gradient is returned for the weight
        accum = ctx.weight_grad_accum
        if accum is not None:
            need_w = True
        if grad_logprobs is None or not (need_h or need_w or need_b):
            return (None,) * 10
        lib = _lib.load()
        dev = hidden_2d.device
        T, H = hidden_2d.shape
        V = weight_c.size(0)
        g = grad_logprobs.reshape(-1).to(torch.float32).contiguous()
        # the kernels need one of dHidden / dWeight as an output; a bias-only request computes dHidden
        need_h = need_h or (need_b and not need_w)
        dh = torch.empty_like(hidden_2d) if need_h else None
        # (zeroed when the kernels add to it, which they do together with the weight accumulator)
        db32 = None
        if need_b:
            db32 = (torch.zeros if accum is not None else torch.empty)(V, dtype=torch.float32, device=dev)
        probs, probs_ref, probs_status = ctx.probs, ctx.probs_ref, ctx.probs_status
        # A contraction over the whole batch can store dWeight in bf16 itself: the saved mode always,
        # the recompute mode when one token chunk covers the batch. Several chunks accumulate in
        # fp32 and cast at the end.
        chunk = (ctx.token_chunk or default_token_chunk(T, H, V)) if T > 0 else 1
        bf16_out = accum is None and T > 0 and ctx.weight_dtype == torch.bfloat16
        direct = bf16_out and (probs is not None or chunk >= T)
        dw_direct = torch.empty((V, H), dtype=torch.bfloat16, device=dev) if (need_w and direct) else None
        dw32 = accum
        if accum is None and need_w and not direct:
            dw32 = torch.empty((V, H), dtype=torch.float32, device=dev)
        ctx.probs = ctx.probs_ref = ctx.probs_status = None  # consumed; a second backward recomputes
        recompute = probs is None
        if T == 0:
            recompute = False
            if dw32 is not None and accum is None:
                dw32.zero_()
            if db32 is not None:
                db32.zero_()
        elif probs is not None:
            # Queued before the host knows whether every row's saved exponentials were in range:
            # the kernels read that status on the device and return at once if it is set.
            nbytes = lib.areal_lmhead_bwd_saved_workspace_bytes(T, H, V)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            rc = lib.areal_lmhead_bwd_saved(
                _lib.ptr(hidden_2d), _lib.ptr(weight_c), _lib.ptr(labels_1d),
                _lib.ptr(row_max), _lib.ptr(sum_exp), _lib.ptr(ctx.label_logprobs), _lib.ptr(g),
                T, H, V, 1.0 / ctx.temperature, ctx.logit_scale,
                _lib.ptr(probs), probs.numel() * 2, _lib.ptr(probs_ref), _lib.ptr(probs_status),
                _lib.ptr(dh), _lib.ptr(dw_direct if direct else dw32),
                2 if direct else (1 if accum is not None else 0),
                _lib.ptr(db32), _lib.ptr(ws), nbytes, _lib.stream_ptr(dev),
            )
            _lib.check(rc, "areal_lmhead_bwd_saved")
            # The status travelled to pinned memory behind the forward. Looking at it now, with
            # the launches above already queued, idles nothing; if it was set (a row's maximum
            # far above its estimate) those launches did nothing and the recompute mode runs.
            ctx.status_event.synchronize()
            if int(ctx.status_host[0]) != 0:
                recompute = True
                if need_w and direct and chunk < T:
                    direct, dw_direct = False, None
                    dw32 = torch.empty((V, H), dtype=torch.float32, device=dev)
            del probs, probs_ref
        if recompute:
            nbytes = lib.areal_lmhead_bwd_workspace_bytes(T, H, V, chunk)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            rc = lib.areal_lmhead_bwd(
                _lib.ptr(hidden_2d), _lib.ptr(weight_c), _lib.ptr(ctx.bias_f),
                _lib.ptr(labels_1d), _lib.ptr(row_max), _lib.ptr(sum_exp), _lib.ptr(g),
                T, H, V, 1.0 / ctx.temperature, ctx.logit_scale,
                _lib.ptr(dh), _lib.ptr(dw_direct if direct else dw32), _lib.ptr(db32),
                2 if direct else (1 if accum is not None else 0), chunk,
                _lib.ptr(ws), nbytes, _lib.stream_ptr(dev),
            )
            _lib.check(rc, "areal_lmhead_bwd")
        dw = dw_direct
        if dw32 is not None and accum is None:
            if ctx.weight_dtype == torch.float32:
                dw = dw32
            else:
                dw = torch.empty((V, H), dtype=ctx.weight_dtype, device=dev)
                rc = lib.areal_cast_f32_to_bf16(
                    _lib.ptr(dw32), _lib.ptr(dw), dw32.numel(), _lib.stream_ptr(dev)
                )
                _lib.check(rc, "areal_cast_f32_to_bf16")
        dh = dh.view(ctx.hidden_shape) if (dh is not None and want_h) else None
        db = db32.to(ctx.bias_dtype) if db32 is not None else None
        return dh, dw, db, None, None, None, None, None, None, None


def fused_lm_head_logprobs_entropy(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    *,
    temperature: float = 1.0,
    vocab_chunk: int | None = None,
    logit_scale: float = 1.0,
    bias: torch.Tensor | None = None,
    token_chunk: int | None = None,
    save_probs: bool | None = None,
    with_moments: bool = False,
    weight_grad_accum: torch.Tensor | None = None,
) -> ChunkedLMHeadOutput:
    """Label log-probabilities, entropy and vocabulary statistics of ``hidden @ weight.T``.

    Args:
        hidden: ``[..., H]`` bf16 final hidden states (packed tokens).
        weight: ``[V, H]`` bf16 lm_head weight (row = vocabulary id).
        labels: ``[...]`` integer labels, leading dimensions matching ``hidden``.
        temperature: softmax temperature (> 0).
        vocab_chunk: accepted for signature compatibility; the kernel sweeps the vocabulary
            in 256-row tiles whatever its value.
        logit_scale: multiplier applied to the logits before the softmax (> 0).
        bias: optional ``[V]`` bias added to the logits.
        token_chunk: tokens per backward chunk (bounds the bf16 dlogits workspace);
            ``None`` picks the largest chunk within ``DEFAULT_BWD_WORKSPACE_BYTES``.
        save_probs: keep the bf16 softmax exponentials for the backward instead of recomputing
            the logits; ``None`` decides by ``SAVE_PROBS_BYTES_LIMIT``.
        with_moments: also return ``vocab_mean_logits`` and ``vocab_norm_logits`` (two more
            operations per logit in the sweep); without it those two fields are ``None``.
        weight_grad_accum: an fp32 ``[V, H]`` tensor (normally the ``.grad`` of an fp32 master
            copy of ``weight``) that the weight gradient is ADDED to by the dWeight contraction
            itself, as Megatron's fp32 ``main_grad`` accumulation does
            (``vocab_parallel_head.py:873-879``); no gradient is then returned for ``weight``.
            The bias gradient, if any, is added in the same way only through autograd.

    Gradient flows through ``logprobs`` only (to ``hidden`` and ``weight``), as in the
    reference (``vocab_parallel_head.py:732-734``).
    """
    del vocab_chunk
    if not math.isfinite(temperature) or temperature <= 0:
        raise ValueError(f"temperature must be positive, got {temperature}")
    if not math.isfinite(logit_scale) or logit_scale <= 0:
        raise ValueError(f"logit_scale must be positive, got {logit_scale}")
    if token_chunk is not None and token_chunk <= 0:
        raise ValueError(f"chunk_size must be positive, got {token_chunk}")
    if hidden.dtype != weight.dtype:
        raise ValueError(
            "chunked LM Head requires matching hidden and weight dtypes, got "
            f"{hidden.dtype} and {weight.dtype}"
        )
    if weight.ndim != 2 or hidden.size(-1) != weight.size(1):
        raise ValueError(
            f"weight must be [V, H] with H == hidden.size(-1); got {tuple(weight.shape)} "
            f"and {tuple(hidden.shape)}"
        )
    if hidden.numel() // max(hidden.size(-1), 1) != labels.numel():
        raise ValueError(
            "LM Head hidden leading dimensions must match labels: "
            f"got {tuple(hidden.shape)} and {tuple(labels.shape)}"
        )
    if hidden.dtype != torch.bfloat16:
        raise ValueError(f"the fused LM head computes in bf16; got {hidden.dtype}")
    if hidden.size(-1) % 8 != 0:
        raise ValueError(f"hidden size must be a multiple of 8, got {hidden.size(-1)}")
    if bias is not None and bias.shape != (weight.size(0),):
        raise ValueError(f"bias must have shape ({weight.size(0)},), got {tuple(bias.shape)}")
    if weight_grad_accum is not None:
        if weight_grad_accum.dtype != torch.float32 or weight_grad_accum.shape != weight.shape:
            raise ValueError(
                "weight_grad_accum must be an fp32 tensor of the weight's shape, got "
                f"{weight_grad_accum.dtype} {tuple(weight_grad_accum.shape)}"
            )
        if not weight_grad_accum.is_contiguous():
            raise ValueError("weight_grad_accum must be contiguous")
    if not torch.is_grad_enabled():
        save_probs = False  # no backward will come: keep nothing
        weight_grad_accum = None
    values = _FusedLMHead.apply(
        hidden, weight, bias, labels, float(temperature), float(logit_scale), token_chunk,
        save_probs, bool(with_moments), weight_grad_accum,
    )
    return ChunkedLMHeadOutput(*values)


def chunked_lm_head_logprobs_entropy(
    output_layer,
    hidden_states: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    *,
    temperature: float,
    chunk_size: int,
    logit_scale: float = 1.0,
) -> ChunkedLMHeadOutput:
    """The reference's entry point of the same name (``vocab_parallel_head.py:941-982``), for
    callers that hold an output layer object: the bias comes from ``output_layer.bias`` unless
    ``output_layer.skip_bias_add`` is set, ``chunk_size`` is validated and otherwise unused (the
    kernels hold no fp32 logits, so there is nothing to bound by it), and the layer options the
    fused path cannot honour are refused with the reference's errors. Tensor-parallel layers (a ``tp_group`` of more than one rank) are
    outside the one-GPU scope."""
    if not getattr(output_layer, "chunked_loss_supported", True):
        raise NotImplementedError(
            "chunked LM Head loss does not support this output-layer forward override"
        )
    config = getattr(output_layer, "config", None)
    if getattr(config, "defer_embedding_wgrad_compute", False):
        raise NotImplementedError(
            "chunked LM Head loss is incompatible with defer_embedding_wgrad_compute"
        )
    if getattr(output_layer, "gather_output", False):
        raise NotImplementedError(
            "chunked LM Head loss requires vocab-parallel (ungathered) output"
        )
    tp_group = getattr(output_layer, "tp_group", None)
    if tp_group is not None:
        import torch.distributed as dist

        if dist.is_initialized() and dist.get_world_size(tp_group) > 1:
            raise NotImplementedError("vocab-parallel LM heads over several GPUs are not built here")
    bias = None
    if not getattr(output_layer, "skip_bias_add", False):
        bias = getattr(output_layer, "bias", None)
    if chunk_size <= 0:
        raise ValueError(f"chunk_size must be positive, got {chunk_size}")
    return fused_lm_head_logprobs_entropy(
        hidden_states, weight, labels, temperature=temperature, logit_scale=logit_scale, bias=bias,
        with_moments=True,
    )

