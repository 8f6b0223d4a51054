"""Fused lm_head -> logprob/entropy kernels against the CPU oracle.

Tolerances: bf16-input logprobs within 2e-3 absolute of the fp32 oracle (measured ~1e-5);
gradients within 1e-2 relative (relative L2, as the reference compares dW in
tests/test_megatron_lm_head.py:190-199; measured ~2.5e-3, the bf16 rounding of dlogits)."""

import pytest
import torch

from areal_amd import _lib
from areal_amd.functional import fused_lm_head_logprobs_entropy
from oracle import logprob as L

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30)).item()


@pytest.mark.parametrize("M,N,K", [(32, 32, 16), (256, 256, 64), (300, 200, 72), (1000, 520, 8), (96, 13, 32),
                                   (260, 513, 200),
                                   # K a multiple of 128: the hand-scheduled main loop (one pair of
                                   # k-tiles, several, ragged M and N, M not a multiple of 8)
                                   (256, 256, 128), (512, 256, 1024), (300, 200, 256), (520, 1000, 384),
                                   (96, 13, 128), (264, 513, 1280),
                                   # an odd number of k-tiles (3, 5, 7, 21): the last pair's second k-tile is dead
                                   (256, 256, 192), (520, 300, 320), (512, 1000, 448), (264, 513, 1344)])
@pytest.mark.parametrize("mode", [0, 1, 2])
def test_gemm_nt(dev, M, N, K, mode):
    lib = _lib.load()
    g = torch.Generator().manual_seed(M + N + K)
    A = torch.randn(M, K, generator=g).bfloat16().to(dev)
    B = torch.randn(N, K, generator=g).bfloat16().to(dev)
    ref = (B.float() @ A.float().T)
    if mode == 0:
        out = torch.empty((N, M), dtype=torch.bfloat16, device=dev)
    else:
        out = torch.ones((N, M), dtype=torch.float32, device=dev)
    rc = lib.areal_gemm_nt_bf16(_lib.ptr(A), K, _lib.ptr(B), K, _lib.ptr(out), M, M, N, K, mode,
                                _lib.stream_ptr(dev))
    assert rc == 0
    if mode == 0:
        assert torch.equal(out, ref.bfloat16()) or _rel(out.float(), ref) < 4e-3
    else:
        torch.testing.assert_close(out, ref + (1.0 if mode == 2 else 0.0), rtol=1e-5, atol=1e-4)


SHAPES = [
    # T, H, V, temperature, logit_scale, bias, token_chunk
    (13, 32, 96, 0.7, 0.5, True, 5),       # the reference's test shape, chunk 5, scale 0.5, bias
    (13, 32, 96, 1.0, 1.0, False, None),
    (2, 8, 3, 1.0, 1.0, False, None),
    (300, 64, 1000, 1.5, 1.0, False, 128),
    (700, 128, 5000, 1.0, 2.0, True, None),
    (515, 896, 151936, 1.0, 1.0, False, 256),
    # V a multiple of 64: dHidden reads the [V, H] weight in place (no transposed copy)
    (260, 200, 1088, 0.7, 1.0, True, 128),
    (700, 512, 4096, 1.0, 1.0, False, None),
    # every contraction length (H, round_up(V, 64), the token chunk) a multiple of 128: all five
    # contractions take the hand-scheduled main loop
    (768, 256, 1536, 1.0, 1.0, False, None),
    (384, 384, 2000, 0.8, 1.5, True, 128),
    (1024, 128, 640, 1.0, 1.0, False, 256),
    # T = 6.5 x 128: the saved buffer's rows are padded to 896 so that dWeight's token range is whole
    # pairs of k-tiles
    (832, 256, 1536, 1.0, 1.0, False, None),
    # 144 x 2 dWeight tiles = 9 super-blocks of 32 workgroups: the last one is contracted by a second
    # launch with the token range split over 8 copies (saved mode)
    (2048, 512, 36764, 1.0, 1.0, False, None),
]


@pytest.mark.parametrize("save_probs", [False, True], ids=["recompute", "saved"])
@pytest.mark.parametrize("T,H,V,temp,scale,use_bias,chunk", SHAPES)
def test_forward_backward_against_oracle(dev, T, H, V, temp, scale, use_bias, chunk, save_probs):
    g = torch.Generator().manual_seed(T * 7 + V)
    hidden = torch.randn(T, H, generator=g).bfloat16()
    # logits / temperature of standard deviation sqrt(H) / 2 at most (up to 10 nats here): a row's
    # maximum then stays within the 69 nats above its sampled estimate that the saved mode allows
    w_std = (0.5 if V < 10000 else 0.02) / max(1.0, scale / temp)
    weight = (torch.randn(V, H, generator=g) * w_std).bfloat16()
    bias = (torch.randn(V, generator=g) * 0.1).bfloat16() if use_bias else None
    b_dev = bias.to(dev).requires_grad_(True) if use_bias else None
    labels = torch.randint(0, V, (T,), generator=g)
    grad = torch.randn(T, generator=g)
    grad[::3] = 0
    h = hidden.to(dev).requires_grad_(True)
    w = weight.to(dev).requires_grad_(True)
    # vocabulary mean / norm are opt-in (half of the shapes ask for them)
    with_moments = (T + V) % 2 == 1
    out = fused_lm_head_logprobs_entropy(h, w, labels.to(dev), temperature=temp, logit_scale=scale,
                                         bias=b_dev, token_chunk=chunk, save_probs=save_probs,
                                         with_moments=with_moments)
    want = L.lm_head_logprobs_entropy(hidden, weight, labels, temp, scale, bias)
    names = ["logprobs", "entropy", "vocab_min", "vocab_max", "vocab_mean", "vocab_norm"]
    for name, a, b in zip(names, out, want):
        if name in ("vocab_mean", "vocab_norm") and not with_moments:
            assert a is None
            continue
        assert a.dtype == torch.float32 and a.shape == (T,)
        tol = 2e-3 if name in ("logprobs", "entropy") else 2e-3 * max(1.0, b.abs().max().item())
        err = (a.cpu() - b).abs().max().item()
        assert err < tol, f"{name}: max abs err {err}"
    assert out.logprobs.requires_grad and not out.entropy.requires_grad
    if save_probs:  # ordinary logits: the saved exponentials are in range, no recompute fallback
        assert int(out.logprobs.grad_fn.probs_status.item()) == 0
    (out.logprobs * grad.to(dev)).sum().backward()
    dh_want, dw_want, db_want = L.lm_head_backward(hidden, weight, labels, grad, temp, scale, bias,
                                                   with_bias_grad=True)
    if use_bias:  # column sums of the bf16 dlogits (vocab_parallel_head.py:862-863)
        assert b_dev.grad.dtype == torch.bfloat16
        assert _rel(b_dev.grad.cpu().float(), db_want) < 1e-2
    assert h.grad.dtype == torch.bfloat16 and w.grad.dtype == torch.bfloat16
    assert _rel(h.grad.cpu().float(), dh_want) < 1e-2
    assert _rel(w.grad.cpu().float(), dw_want) < 1e-2
    assert (h.grad[::3] == 0).all()  # rows with zero upstream gradient get exactly zero
    cos = torch.nn.functional.cosine_similarity(w.grad.cpu().float().view(-1), dw_want.view(-1), dim=0)
    assert cos > 0.9999


def test_no_vocab_sized_tensor_is_saved(dev):
    # as the reference checks in tests/test_megatron_lm_head.py:738-741
    T, H, V = 48, 64, 4096
    h = torch.randn(T, H, device=dev).bfloat16().requires_grad_(True)
    w = torch.randn(V, H, device=dev).bfloat16().requires_grad_(True)
    y = torch.randint(0, V, (T,), device=dev)
    out = fused_lm_head_logprobs_entropy(h, w, y, save_probs=False)
    for t in out.logprobs.grad_fn.saved_tensors:
        assert tuple(t.shape) != (T, V) and t.numel() <= max(T * H, V * H)


def test_saved_exponentials_are_bf16_and_used_once(dev):
    # save_probs=True keeps one bf16 [T, V] buffer (padded to 64), consumed by the first
    # backward; a second backward over a retained graph recomputes the logits instead.
    T, H, V = 100, 64, 1000
    g = torch.Generator().manual_seed(5)
    hidden = torch.randn(T, H, generator=g).bfloat16().to(dev)
    weight = (torch.randn(V, H, generator=g) * 0.3).bfloat16().to(dev)
    y = torch.randint(0, V, (T,), generator=g).to(dev)
    grad = torch.randn(T, generator=g).to(dev)
    h, w = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
    out = fused_lm_head_logprobs_entropy(h, w, y, save_probs=True)
    fn = out.logprobs.grad_fn
    assert fn.probs.dtype == torch.bfloat16 and tuple(fn.probs.shape) == (128, 1024)
    assert tuple(fn.probs_ref.shape) == (T,) and int(fn.probs_status.item()) == 0
    loss = (out.logprobs * grad).sum()
    loss.backward(retain_graph=True)
    assert fn.probs is None
    g1h, g1w = h.grad.clone(), w.grad.clone()
    h.grad = None
    w.grad = None
    loss.backward()
    assert _rel(h.grad.float(), g1h.float()) < 1e-2 and _rel(w.grad.float(), g1w.float()) < 1e-2
    with torch.no_grad():  # nothing is kept when no gradient can flow
        out = fused_lm_head_logprobs_entropy(h, w, y, save_probs=True)
    assert out.logprobs.grad_fn is None


@pytest.mark.parametrize("H", [64, 128, 256])
def test_saved_path_falls_back_when_a_row_exceeds_the_exponent_window(dev, H):
    # The saved exponentials are relative to a per-row reference estimated from the label's
    # logit and 7 sampled vocabulary entries. A row whose maximum logit lies more than 100
    # binades above all of those is reported by the forward, and the backward recomputes the
    # logits instead of using the buffer: gradients still match the oracle. With H a multiple of
    # 128 the forward's own sums are relative to that reference too, and the log-probabilities
    # come from the sweep that the forward repeats on the device when a row is out of range.
    T, V = 96, 1000
    g = torch.Generator().manual_seed(21)
    weight = (torch.randn(V, H, generator=g) * 0.3).bfloat16()
    hot = 777  # not one of the sampled ids k * V / 8 and not a label
    labels = torch.randint(0, 700, (T,), generator=g)
    hidden = (torch.randn(T, H, generator=g) * 0.5).bfloat16()
    hidden[5] = (weight[hot].float() * (40.0 * 64 / H)).bfloat16()  # logit of `hot` ~ 230 nats above the rest
    grad = torch.randn(T, generator=g)
    h = hidden.to(dev).requires_grad_(True)
    w = weight.to(dev).requires_grad_(True)
    out = fused_lm_head_logprobs_entropy(h, w, labels.to(dev), save_probs=True)
    assert int(out.logprobs.grad_fn.probs_status.item()) == 1
    want = L.lm_head_logprobs_entropy(hidden, weight, labels, 1.0, 1.0, None)
    # the label log-probability of the hot row is about -200: compare relatively
    torch.testing.assert_close(out.logprobs.cpu(), want[0], rtol=2e-3, atol=2e-3)
    (out.logprobs * grad.to(dev)).sum().backward()
    dh_want, dw_want = L.lm_head_backward(hidden, weight, labels, grad, 1.0, 1.0, None)
    assert _rel(h.grad.cpu().float(), dh_want) < 1e-2
    assert _rel(w.grad.cpu().float(), dw_want) < 1e-2


@pytest.mark.parametrize("temp,scale", [(0.7, 2.0), (0.35, 1.0), (1.0, 1.0)])
def test_logprob_of_saturated_rows_keeps_fp32_resolution(dev, temp, scale):
    # Logits of magnitude ~65 whose label holds all the probability: c2 * max is ~130, where one
    # fp32 ulp is 1.5e-5. The kernels keep every softmax sum relative to the rounded product
    # fl(c2 * max) and merge with that same value, so this rounding cancels: the log-probability
    # is right to fp32 resolution (not to ulp(c2 * max)) and never positive.
    T, H, V = 2, 16, 3
    g = torch.Generator().manual_seed(297)
    hidden = torch.randn(T, H, generator=g).bfloat16()
    weight = (torch.randn(V, H, generator=g) * (25.0 * 2.0 / H ** 0.5)).bfloat16()
    logits = (hidden.double() @ weight.double().T) * scale / temp
    labels = logits.argmax(dim=1)
    want = torch.log_softmax(logits, dim=1).gather(1, labels[:, None])[:, 0]
    for Hp in (16, 64):  # generic kernel and the K % 64 == 0 kernel
        hd = torch.zeros(T, Hp, dtype=torch.bfloat16)
        hd[:, :H] = hidden
        wt = torch.zeros(V, Hp, dtype=torch.bfloat16)
        wt[:, :H] = weight
        out = fused_lm_head_logprobs_entropy(hd.to(dev), wt.to(dev), labels.to(dev), temperature=temp,
                                             logit_scale=scale)
        lp = out.logprobs.cpu().double()
        assert (lp <= 0).all()
        assert (lp - want).abs().max() < 3e-7, (lp, want)


def test_saved_path_confident_tokens_and_invalid_labels(dev):
    # Tokens whose label probability is ~1: 1 - p must not be lost to the bf16 rounding of p
    # (the label's dlogit comes from the fp32 log-probability). Labels outside [0, V) get no
    # one-hot term, as in the recompute path.
    T, H, V = 192, 64, 777
    g = torch.Generator().manual_seed(9)
    weight = (torch.randn(V, H, generator=g) * 0.3).bfloat16()
    labels = torch.randint(0, V, (T,), generator=g)
    hidden = (weight[labels].float() * 4.0).bfloat16()  # logit of the label dominates
    grad = torch.randn(T, generator=g)
    h = hidden.to(dev).requires_grad_(True)
    w = weight.to(dev).requires_grad_(True)
    out = fused_lm_head_logprobs_entropy(h, w, labels.to(dev), save_probs=True)
    assert out.logprobs.max().item() > -1e-3
    (out.logprobs * grad.to(dev)).sum().backward()
    dh_want, dw_want = L.lm_head_backward(hidden, weight, labels, grad)
    assert _rel(h.grad.cpu().float(), dh_want) < 1e-2
    assert _rel(w.grad.cpu().float(), dw_want) < 1e-2
    bad = labels.clone()
    bad[::2] = -100
    bad[1::4] = V + 3
    res = []
    for save in (False, True):
        h2 = hidden.to(dev).requires_grad_(True)
        w2 = weight.to(dev).requires_grad_(True)
        o = fused_lm_head_logprobs_entropy(h2, w2, bad.to(dev), save_probs=save)
        (o.logprobs * grad.to(dev)).sum().backward()
        res.append((o.logprobs.detach(), h2.grad.float(), w2.grad.float()))
    torch.testing.assert_close(res[0][0], res[1][0], rtol=0, atol=1e-4)
    assert _rel(res[1][1], res[0][1]) < 1e-2 and _rel(res[1][2], res[0][2]) < 1e-2


def test_chunking_and_repeat_runs_are_bit_identical(dev):
    T, H, V = 600, 128, 3000
    g = torch.Generator().manual_seed(0)
    hidden = torch.randn(T, H, generator=g).bfloat16().to(dev)
    weight = (torch.randn(V, H, generator=g) * 0.3).bfloat16().to(dev)
    y = torch.randint(0, V, (T,), generator=g).to(dev)
    grad = torch.randn(T, generator=g).to(dev)
    res = []
    for chunk in (None, None, 256):
        h, w = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
        out = fused_lm_head_logprobs_entropy(h, w, y, token_chunk=chunk, save_probs=False)
        (out.logprobs * grad).sum().backward()
        res.append((out.logprobs.detach(), out.entropy, h.grad, w.grad))
    for a, b in zip(res[0], res[1]):
        assert torch.equal(a, b)
    assert torch.equal(res[0][0], res[2][0]) and torch.equal(res[0][2], res[2][2])
    assert _rel(res[2][3].float(), res[0][3].float()) < 1e-2  # dW: different accumulation split


def test_large_logits_are_stable(dev):
    T, H, V = 64, 64, 2048
    h = (torch.randn(T, H, device=dev) * 30).bfloat16()
    w = (torch.randn(V, H, device=dev) * 3).bfloat16()
    y = torch.randint(0, V, (T,), device=dev)
    out = fused_lm_head_logprobs_entropy(h, w, y)
    want = L.lm_head_logprobs_entropy(h.cpu(), w.cpu(), y.cpu())
    assert torch.isfinite(out.logprobs).all() and torch.isfinite(out.entropy).all()
    torch.testing.assert_close(out.logprobs.cpu(), want[0], rtol=1e-4, atol=2e-3)


def test_empty_and_3d_inputs(dev):
    w = torch.randn(100, 16, device=dev).bfloat16()
    out = fused_lm_head_logprobs_entropy(torch.empty(0, 16, device=dev).bfloat16(), w,
                                         torch.empty(0, dtype=torch.long, device=dev))
    assert out.logprobs.shape == (0,)
    h = torch.randn(2, 5, 16, device=dev).bfloat16()
    y = torch.randint(0, 100, (2, 5), device=dev)
    out = fused_lm_head_logprobs_entropy(h, w, y)
    want = L.lm_head_logprobs_entropy(h.cpu().view(10, 16), w.cpu(), y.cpu().view(-1))
    assert out.logprobs.shape == (2, 5)
    torch.testing.assert_close(out.logprobs.cpu().view(-1), want[0], rtol=1e-4, atol=2e-3)


def test_chunked_lm_head_wrapper_uses_the_layer_bias(dev):
    from types import SimpleNamespace

    from areal_amd.functional import chunked_lm_head_logprobs_entropy

    T, H, V = 40, 32, 200
    g = torch.Generator().manual_seed(3)
    hidden = torch.randn(T, H, generator=g).bfloat16()
    weight = (torch.randn(V, H, generator=g) * 0.3).bfloat16()
    bias = (torch.randn(V, generator=g) * 0.2).bfloat16()
    labels = torch.randint(0, V, (T,), generator=g)
    layer = SimpleNamespace(bias=bias.to(dev), skip_bias_add=False, gather_output=False, tp_group=None)
    out = chunked_lm_head_logprobs_entropy(layer, hidden.to(dev), weight.to(dev), labels.to(dev),
                                           temperature=0.7, chunk_size=16, logit_scale=0.5)
    want = L.lm_head_logprobs_entropy(hidden, weight, labels, 0.7, 0.5, bias)
    torch.testing.assert_close(out.logprobs.cpu(), want[0], rtol=0, atol=2e-3)
    layer.skip_bias_add = True
    out = chunked_lm_head_logprobs_entropy(layer, hidden.to(dev), weight.to(dev), labels.to(dev),
                                           temperature=0.7, chunk_size=16, logit_scale=0.5)
    want = L.lm_head_logprobs_entropy(hidden, weight, labels, 0.7, 0.5, None)
    torch.testing.assert_close(out.logprobs.cpu(), want[0], rtol=0, atol=2e-3)

