"""Oracle: label log-probabilities, entropy and the lm_head contraction (CPU, test-only).

Follows
  * ``areal/utils/functional/vocab_parallel.py:16-30`` (log_softmax of ``logits.float()/T``,
    gather, ``-sum p log p``) and ``:42-82`` (row chunking, which does not change values);
  * ``areal/models/mcore/vocab_parallel_head.py:538-557`` (fp32 logits of a bf16 contraction,
    ``+bias``, ``*logit_scale``), ``:647-700`` (vocab min/max/mean/norm, row max,
    ``pred - log sum_exp``, ``log sum_exp - sum(shifted*e)/sum_exp``);
  * ``areal/utils/functional/vocab_parallel_kernels.py:99-137`` (backward:
    ``(onehot - p) * g * invT * logit_scale``) and ``vocab_parallel_head.py:830-879``
    (dlogits rounded to the weight dtype, then ``dH = dlogits @ W``, ``dW = dlogits^T @ hidden``).

Pinned by: float64 ``torch.log_softmax`` on tiny shapes, sum(softmax) == 1, entropy in
[0, log V], brute force at V <= 8, and autograd of the textbook form for the backward
(``tests/test_oracle_logprob.py``).
"""

from __future__ import annotations

import torch


def gather_logprobs(logits: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0):
    lsm = torch.log_softmax(logits.float() / temperature, dim=-1)
    return lsm.gather(-1, labels.unsqueeze(-1)).squeeze(-1)


def gather_logprobs_entropy(logits: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0):
    lsm = torch.log_softmax(logits.float() / temperature, dim=-1)
    entropy = -(lsm.exp() * lsm).sum(-1)
    return lsm.gather(-1, labels.unsqueeze(-1)).squeeze(-1), entropy


def lm_head_logits(hidden, weight, bias=None, logit_scale: float = 1.0, row_chunk: int = 2048):
    """fp32 logits of the (bf16-valued) operands, accumulated in fp32."""
    out = []
    w = weight.float()
    for i in range(0, hidden.shape[0], row_chunk):
        x = hidden[i : i + row_chunk].float() @ w.T
        if bias is not None:
            x = x + bias.float()
        if logit_scale != 1.0:
            x = x * logit_scale
        out.append(x)
    if not out:
        return torch.empty((0, weight.shape[0]), dtype=torch.float32)
    return torch.cat(out)


def lm_head_logprobs_entropy(
    hidden, weight, labels, temperature=1.0, logit_scale=1.0, bias=None, row_chunk: int = 1024
):
    """Six per-token outputs of the chunked LM head, one row chunk at a time."""
    res = [[] for _ in range(6)]
    inv_t = 1.0 / temperature
    for i in range(0, hidden.shape[0], row_chunk):
        x = lm_head_logits(hidden[i : i + row_chunk], weight, bias, logit_scale)
        lab = labels[i : i + row_chunk]
        row_max = x.max(-1).values
        shifted = (x - row_max[:, None]) * inv_t
        e = shifted.exp()
        sum_e = e.sum(-1)
        pred = shifted.gather(-1, lab[:, None]).squeeze(-1)
        log_sum = sum_e.log()
        res[0].append(pred - log_sum)
        res[1].append(log_sum - (shifted * e).sum(-1) / sum_e)
        res[2].append(x.min(-1).values)
        res[3].append(row_max)
        res[4].append(x.mean(-1))
        res[5].append(torch.linalg.vector_norm(x, dim=-1))
    return tuple(torch.cat(r) if r else torch.empty(0) for r in res)


def lm_head_backward(
    hidden, weight, labels, grad_logprobs, temperature=1.0, logit_scale=1.0, bias=None,
    round_dlogits_to=torch.bfloat16, row_chunk: int = 1024, with_bias_grad: bool = False,
):
    """Closed-form dHidden [T,H] and dWeight [V,H] (fp32) for upstream dLoss/dlogprobs; with
    ``with_bias_grad`` also dBias [V] = column sums of dlogits (vocab_parallel_head.py:862-863)."""
    inv_t = 1.0 / temperature
    w = weight.float()
    d_hidden = torch.zeros(hidden.shape, dtype=torch.float32)
    d_weight = torch.zeros(weight.shape, dtype=torch.float32)
    d_bias = torch.zeros(weight.shape[0], dtype=torch.float32)
    for i in range(0, hidden.shape[0], row_chunk):
        h = hidden[i : i + row_chunk].float()
        x = lm_head_logits(hidden[i : i + row_chunk], weight, bias, logit_scale)
        p = torch.softmax(x * inv_t, dim=-1)
        g = grad_logprobs[i : i + row_chunk].float()[:, None]
        d = -p * g
        d.scatter_add_(1, labels[i : i + row_chunk, None], g)
        d = d * (inv_t * logit_scale)
        if round_dlogits_to is not None:
            d = d.to(round_dlogits_to).float()
        d_hidden[i : i + row_chunk] = d @ w
        d_weight += d.T @ h
        d_bias += d.sum(dim=0)
    if with_bias_grad:
        return d_hidden, d_weight, d_bias
    return d_hidden, d_weight


def logits_backward(logits, labels, grad_logprobs, grad_entropy=None, temperature=1.0):
    """dLoss/dlogits for the logits-in API: closed forms
    d lp_label / d x_j = (1[j==label] - p_j)/T and d ent / d x_j = -p_j (log p_j + ent)/T."""
    z = logits.float() / temperature
    lsm = torch.log_softmax(z, dim=-1)
    p = lsm.exp()
    grad = torch.zeros_like(p)
    if grad_logprobs is not None:
        g = grad_logprobs.float()[:, None]
        grad = grad - p * g
        grad.scatter_add_(1, labels[:, None], g.expand(-1, 1).contiguous())
    if grad_entropy is not None:
        ent = -(p * lsm).sum(-1, keepdim=True)
        grad = grad - grad_entropy.float()[:, None] * p * (lsm + ent)
    return grad / temperature
