"""Logits-in gather_logprobs / gather_logprobs_entropy kernels against the CPU oracle
(shapes, temperatures and tolerances of the reference's tests/test_vocab_parallel_inplace.py)."""

import pytest
import torch

from areal_amd.functional import gather_logprobs, gather_logprobs_entropy
from oracle import logprob as L

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(7, 31), (17, 1537), (33, 4096), (5, 151936)])
@pytest.mark.parametrize("temp", [0.7, 1.0, 1.5])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_forward_backward(dev, shape, temp, dtype):
    g = torch.Generator().manual_seed(shape[1])
    x = (torch.randn(*shape, generator=g) * 2).to(dtype)
    y = torch.randint(0, shape[1], (shape[0],), generator=g)
    w_lp = torch.randn(shape[0], generator=g)
    w_lp[::2] = 0
    w_ent = torch.randn(shape[0], generator=g)
    xg = x.to(dev).requires_grad_(True)
    lp, ent = gather_logprobs_entropy(xg, y.to(dev), temp)
    want_lp, want_ent = L.gather_logprobs_entropy(x, y, temp)
    torch.testing.assert_close(lp.cpu(), want_lp, rtol=1e-5, atol=2e-5)
    torch.testing.assert_close(ent.cpu(), want_ent, rtol=1e-5, atol=2e-5)
    torch.testing.assert_close(gather_logprobs(xg, y.to(dev), temp).cpu(), want_lp, rtol=1e-5, atol=2e-5)
    ((lp * w_lp.to(dev)).sum() + (ent * w_ent.to(dev)).sum()).backward()
    want_g = L.logits_backward(x, y, w_lp, w_ent, temp)
    assert xg.grad.dtype == dtype
    if dtype == torch.float32:
        torch.testing.assert_close(xg.grad.cpu(), want_g, rtol=1e-5, atol=2e-5)
    else:
        torch.testing.assert_close(xg.grad.cpu().float(), want_g, rtol=1e-2, atol=1e-4)
    # logprob-only gradient: rows with zero upstream weight get exactly zero
    xg2 = x.to(dev).requires_grad_(True)
    (gather_logprobs(xg2, y.to(dev), temp) * w_lp.to(dev)).sum().backward()
    assert (xg2.grad[::2] == 0).all()
    torch.testing.assert_close(xg2.grad.cpu().float(), L.logits_backward(x, y, w_lp, None, temp),
                               rtol=1e-2 if dtype == torch.bfloat16 else 1e-5, atol=1e-4)


def test_large_logits_and_leading_dims(dev):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 3, 64, generator=g) * 100
    y = torch.randint(0, 64, (2, 3), generator=g)
    lp, ent = gather_logprobs_entropy(x.to(dev), y.to(dev))
    want_lp, want_ent = L.gather_logprobs_entropy(x, y)
    assert lp.shape == (2, 3) and torch.isfinite(lp).all() and torch.isfinite(ent).all()
    torch.testing.assert_close(lp.cpu(), want_lp, rtol=1e-5, atol=1e-4)
    torch.testing.assert_close(ent.cpu(), want_ent, rtol=1e-5, atol=1e-4)


def test_repeat_runs_bit_identical(dev):
    x = torch.randn(64, 32000, device=dev).bfloat16()
    y = torch.randint(0, 32000, (64,), device=dev)
    a = gather_logprobs_entropy(x, y)
    b = gather_logprobs_entropy(x, y)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
