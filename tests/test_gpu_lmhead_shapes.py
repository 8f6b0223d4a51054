"""Shape sweep of the fused lm_head kernels: ragged and aligned token counts, hidden sizes and
vocabularies around every boundary the launch plan has (256-wide tiles, 64- and 128-deep
contraction steps, split contraction ranges, the split of dWeight's last round), both backward
modes, against a plain fp32 torch evaluation of the same operator on the GPU
(areal/utils/functional/vocab_parallel.py:24-30 restated with torch ops; an implementation
independent of the kernels under test: the library GEMM in fp32).

Tolerances as in test_gpu_lmhead.py: logprobs / entropy 2e-3 absolute, gradients 1e-2 relative L2."""

import pytest
import torch

from areal_amd.functional import fused_lm_head_logprobs_entropy

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30)).item()


def _reference(hidden, weight, labels, grad, temp, scale):
    h = hidden.detach().float().requires_grad_(True)
    w = weight.detach().float().requires_grad_(True)
    logits = (h @ w.t()) * scale / temp
    logp = torch.log_softmax(logits, dim=-1)
    lp = logp.gather(-1, labels[:, None])[:, 0]
    ent = -(logp.exp() * logp).sum(-1)
    (lp * grad).sum().backward()
    return lp.detach(), ent.detach(), logits.detach().min(-1).values * temp, logits.detach().max(-1).values * temp, h.grad, w.grad


def _case_list():
    g = torch.Generator().manual_seed(20240607)
    tokens = [64, 128, 192, 200, 256, 257, 320, 448, 1000, 1088]
    hiddens = [128, 256, 384, 640, 896, 1024]
    vocabs = [640, 1000, 1536, 2176, 4160, 5000, 8192 + 128]
    cases = []
    for _ in range(28):
        t = tokens[int(torch.randint(len(tokens), (1,), generator=g))]
        h = hiddens[int(torch.randint(len(hiddens), (1,), generator=g))]
        v = vocabs[int(torch.randint(len(vocabs), (1,), generator=g))]
        cases.append((t, h, v))
    # dWeight's last partial round of super-blocks with a ragged hidden size (2.5 tiles) and a
    # ragged vocabulary: 80 x 3 tiles
    cases.append((2048, 640, 20403))
    # token count 64 short of a multiple of 128 with a contraction long enough to split
    cases.append((1984, 256, 9000))
    # contraction lengths that are an odd number of 64-deep steps (the main loop's last pair of
    # k-tiles then has a dead second k-tile): hidden size (forward, recompute), vocabulary
    # (dHidden: 31, 65, 575 steps, the last one split over copies of the schedule), token count
    # (dWeight in recompute mode: 3 and 7 steps)
    cases += [(192, 192, 1984), (448, 320, 4160), (1000, 960, 5000), (320, 448, 1536), (2048, 192, 36764),
              (256, 128 + 64, 640)]
    return sorted(set(cases))


@pytest.mark.parametrize("save_probs", [True, False], ids=["saved", "recompute"])
@pytest.mark.parametrize("T,H,V", _case_list())
def test_shapes_against_fp32_torch(dev, T, H, V, save_probs):
    g = torch.Generator(device="cpu").manual_seed(T * 31 + H * 7 + V)
    temp, scale = (1.0, 1.0) if (T + V) % 3 else (0.7, 1.5)
    hidden = torch.randn(T, H, generator=g).bfloat16().to(dev)
    weight = (torch.randn(V, H, generator=g) * (2.0 / H ** 0.5)).bfloat16().to(dev)
    labels = torch.randint(0, V, (T,), generator=g).to(dev)
    grad = torch.randn(T, generator=g)
    grad[::5] = 0
    grad = grad.to(dev)
    h = hidden.clone().requires_grad_(True)
    w = weight.clone().requires_grad_(True)
    out = fused_lm_head_logprobs_entropy(h, w, labels, temperature=temp, logit_scale=scale,
                                         save_probs=save_probs)
    (out.logprobs * grad).sum().backward()
    lp, ent, vmin, vmax, dh, dw = _reference(hidden, weight, labels, grad, temp, scale)
    assert (out.logprobs.detach() - lp).abs().max().item() < 2e-3
    assert (out.entropy - ent).abs().max().item() < 2e-3
    # the vocabulary extremes are those of the unscaled-by-temperature logits
    # (areal/engine/fsdp_engine.py:2061-2105 takes them before the temperature division)
    span = max(1.0, vmax.abs().max().item(), vmin.abs().max().item())
    assert (out.vocab_max_logits - vmax).abs().max().item() < 2e-3 * span
    assert (out.vocab_min_logits - vmin).abs().max().item() < 2e-3 * span
    assert h.grad.dtype == torch.bfloat16 and w.grad.dtype == torch.bfloat16
    assert _rel(h.grad.float(), dh) < 1e-2
    assert _rel(w.grad.float(), dw) < 1e-2
    assert (h.grad[::5] == 0).all()


@pytest.mark.parametrize("accumulate", [False, True], ids=["bf16", "fp32_accumulate"])
@pytest.mark.parametrize("save_probs", [True, False], ids=["saved", "recompute"])
@pytest.mark.parametrize("H", [136, 640, 896, 1344])
def test_hidden_sizes_tiled_224_wide_elementwise(dev, H, save_probs, accumulate):
    """Hidden sizes that fill their 256-wide output tiles to 7/8 at most run dHidden and dWeight on
    224-wide tiles (896 = 4 x 224; 640 = 224 + 224 + 192; 136 in one; 1344 = 6 x 224). Every
    gradient element is compared, so a misplaced or missing block of 16 columns cannot hide in a
    norm: |error| <= 2 % of the gradient's largest magnitude (bf16 outputs of bf16 operands)."""
    T, V = 512, 2112
    g = torch.Generator(device="cpu").manual_seed(H)
    hidden = torch.randn(T, H, generator=g).bfloat16().to(dev)
    weight = (torch.randn(V, H, generator=g) * (2.0 / H ** 0.5)).bfloat16().to(dev)
    labels = torch.randint(0, V, (T,), generator=g).to(dev)
    grad = torch.randn(T, generator=g).to(dev)
    h = hidden.clone().requires_grad_(True)
    w = weight.clone().requires_grad_(True)
    main_grad = torch.full((V, H), 0.25, dtype=torch.float32, device=dev) if accumulate else None
    out = fused_lm_head_logprobs_entropy(h, w, labels, save_probs=save_probs, weight_grad_accum=main_grad)
    (out.logprobs * grad).sum().backward()
    lp, _, _, _, dh, dw = _reference(hidden, weight, labels, grad, 1.0, 1.0)
    assert (out.logprobs.detach() - lp).abs().max().item() < 2e-3
    got_dw = main_grad - 0.25 if accumulate else w.grad.float()
    for got, want in ((h.grad.float(), dh), (got_dw, dw)):
        err = (got - want).abs()
        assert err.max().item() <= 2e-2 * want.abs().max().item(), (int(err.argmax()) % H, err.max().item())


# (hidden size, vocabulary) of published model families, at a ragged 1.5 token tiles.
MODEL_SHAPES = [
    (1024, 151936),   # Qwen3-0.6B
    (2048, 151936),   # Qwen3-1.7B
    (2560, 151936),   # Qwen3-4B
    (3584, 152064),   # Qwen2.5-7B
    (5120, 152064),   # Qwen2.5-14B / 32B
    (4096, 128256),   # Llama-3-8B
    (8192, 128256),   # Llama-3-70B
]


@pytest.mark.parametrize("save_probs", [True, False], ids=["saved", "recompute"])
@pytest.mark.parametrize("H,V", MODEL_SHAPES)
def test_model_family_shapes(dev, H, V, save_probs):
    """Hidden sizes and vocabularies of common model families run and agree with fp32 torch (the
    launch plan depends on both: tile counts, splits of the contraction, the last partial round)."""
    T = 384
    g = torch.Generator(device=dev).manual_seed(H + V)  # on the device: the weight has up to 1 G entries
    hidden = torch.randn(T, H, generator=g, device=dev).bfloat16()
    weight = (torch.randn(V, H, generator=g, device=dev) * (2.0 / H ** 0.5)).bfloat16()
    labels = torch.randint(0, V, (T,), generator=g, device=dev)
    grad = torch.randn(T, generator=g, device=dev)
    h = hidden.clone().requires_grad_(True)
    w = weight.clone().requires_grad_(True)
    out = fused_lm_head_logprobs_entropy(h, w, labels, save_probs=save_probs)
    (out.logprobs * grad).sum().backward()
    lp, ent, _, _, dh, dw = _reference(hidden, weight, labels, grad, 1.0, 1.0)
    assert (out.logprobs.detach() - lp).abs().max().item() < 2e-3
    assert (out.entropy - ent).abs().max().item() < 2e-3
    assert _rel(h.grad.float(), dh) < 1e-2
    assert _rel(w.grad.float(), dw) < 1e-2
