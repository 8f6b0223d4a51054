"""Pins the logprob / entropy / lm_head oracle with float64 textbook forms and brute force."""

import math

import pytest
import torch

from oracle import logprob as L


@pytest.mark.parametrize("shape", [(7, 31), (17, 1537)])
@pytest.mark.parametrize("temp", [0.7, 1.0, 1.5])
def test_logits_path_against_float64(shape, temp):
    # shapes and temperatures of the reference's tests/test_vocab_parallel_inplace.py:51-58,95,102
    torch.manual_seed(0)
    x = torch.randn(*shape)
    y = torch.randint(0, shape[1], (shape[0],))
    lp, ent = L.gather_logprobs_entropy(x, y, temp)
    lsm = torch.log_softmax(x.double() / temp, -1)
    torch.testing.assert_close(lp.double(), lsm.gather(-1, y[:, None])[:, 0], rtol=1e-5, atol=2e-5)
    torch.testing.assert_close(ent.double(), -(lsm.exp() * lsm).sum(-1), rtol=1e-5, atol=2e-5)
    assert (lp <= 0).all() and (ent >= 0).all() and (ent <= math.log(shape[1]) + 1e-5).all()
    torch.testing.assert_close(L.gather_logprobs(x, y, temp), lp)


def test_brute_force_tiny_vocab():
    x = torch.tensor([[0.0, 1.0, 2.0], [5.0, 5.0, 5.0]])
    y = torch.tensor([2, 0])
    lp, ent = L.gather_logprobs_entropy(x, y)
    z0 = sum(math.exp(v) for v in (0.0, 1.0, 2.0))
    p0 = [math.exp(v) / z0 for v in (0.0, 1.0, 2.0)]
    assert lp[0].item() == pytest.approx(math.log(p0[2]), abs=1e-6)
    assert ent[0].item() == pytest.approx(-sum(p * math.log(p) for p in p0), abs=1e-6)
    assert lp[1].item() == pytest.approx(-math.log(3), abs=1e-6)
    assert ent[1].item() == pytest.approx(math.log(3), abs=1e-6)


def test_large_logits_are_stable():
    torch.manual_seed(1)
    x = torch.randn(5, 64) * 100
    y = torch.randint(0, 64, (5,))
    lp, ent = L.gather_logprobs_entropy(x, y)
    assert torch.isfinite(lp).all() and torch.isfinite(ent).all()


@pytest.mark.parametrize("temp,scale,use_bias", [(0.7, 0.5, True), (1.0, 1.0, False)])
def test_lm_head_against_float64_and_autograd(temp, scale, use_bias):
    # shape (13, 32, 96), logit_scale 0.5, bias, temperatures 0.7 / 1.0 as in the reference's
    # tests/test_megatron_lm_head.py:665-692
    torch.manual_seed(2)
    T, H, V = 13, 32, 96
    h = torch.randn(T, H).bfloat16()
    w = (torch.randn(V, H) * 0.3).bfloat16()
    b = (torch.randn(V) * 0.1).bfloat16() if use_bias else None
    y = torch.randint(0, V, (T,))
    out = L.lm_head_logprobs_entropy(h, w, y, temp, scale, b)
    hd, wd = h.double().requires_grad_(True), w.double().requires_grad_(True)
    bd = b.double().requires_grad_(True) if b is not None else None
    logits = hd @ wd.T
    if b is not None:
        logits = logits + bd
    logits = logits * scale
    lsm = torch.log_softmax(logits / temp, -1)
    lp = lsm.gather(-1, y[:, None])[:, 0]
    torch.testing.assert_close(out[0].double(), lp.detach(), rtol=1e-5, atol=2e-5)
    torch.testing.assert_close(out[1].double(), -(lsm.exp() * lsm).sum(-1).detach(), rtol=1e-5, atol=2e-5)
    torch.testing.assert_close(out[2].double(), logits.min(-1).values.detach(), rtol=1e-5, atol=2e-5)
    torch.testing.assert_close(out[3].double(), logits.max(-1).values.detach(), rtol=1e-5, atol=2e-5)
    torch.testing.assert_close(out[4].double(), logits.mean(-1).detach(), rtol=1e-5, atol=2e-5)
    torch.testing.assert_close(out[5].double(), logits.norm(dim=-1).detach(), rtol=1e-5, atol=2e-5)
    g = torch.randn(T)
    g[::3] = 0
    (lp * g.double()).sum().backward()
    dh, dw, db = L.lm_head_backward(h, w, y, g, temp, scale, b, round_dlogits_to=None, with_bias_grad=True)
    if b is not None:
        torch.testing.assert_close(db.double(), bd.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(dh.double(), hd.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(dw.double(), wd.grad, rtol=1e-4, atol=1e-5)
    assert (dh[::3] == 0).all()  # zero upstream gradient -> exactly zero rows


def test_logits_backward_closed_form_matches_autograd():
    torch.manual_seed(3)
    x = torch.randn(9, 40, requires_grad=True)
    y = torch.randint(0, 40, (9,))
    lp, ent = L.gather_logprobs_entropy(x, y, 0.8)
    glp, gen = torch.randn(9), torch.randn(9)
    ((lp * glp).sum() + (ent * gen).sum()).backward()
    got = L.logits_backward(x.detach(), y, glp, gen, 0.8)
    torch.testing.assert_close(got, x.grad, rtol=1e-5, atol=2e-5)
