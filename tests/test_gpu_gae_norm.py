"""HIP GAE scan and normalisation kernels against the reference's literals and the CPU oracle."""

import math

import pytest
import torch

from areal_amd.config import NormConfig
from areal_amd.data import Normalization
from areal_amd.functional import masked_normalization
from areal_amd.ppo.gae import _compute_token_level_gae, compute_gae_packed
from oracle import gae as G
from oracle import norm as N

pytestmark = pytest.mark.gpu


def _t(x, dev, dtype=torch.float32):
    return torch.tensor(x, dtype=dtype, device=dev)


def test_gae_per_sample_lambda_literals(dev):
    rewards = _t([[0.0, 0.0, 1.0, 0.0]] * 2, dev)
    mask = _t([[1.0, 1.0, 1.0, 0.0]] * 2, dev)
    adv, ret = _compute_token_level_gae(rewards, torch.zeros_like(rewards), mask,
                                        torch.tensor([False, False], device=dev), 1.0, _t([0.5, 0.0], dev))
    assert torch.equal(adv.cpu(), torch.tensor([[0.25, 0.5, 1.0, 0.0], [0.0, 0.0, 1.0, 0.0]]))
    assert torch.equal(ret, adv)


def test_gae_legacy_recurrence_case(dev):
    # inputs of the reference's tests/test_ppo_gae.py:154-193
    r = torch.tensor([[0.0, 0.5, 0.0, 2.0], [0.0, 1.0, 0.0, 0.0]])
    v = torch.tensor([[0.1, 0.2, 0.3, 0.4], [0.2, 0.1, 0.0, 0.5]])
    m = torch.tensor([[1.0, 1.0, 0.0, 1.0], [0.0, 1.0, 1.0, 1.0]])
    ne = torch.tensor([False, True])
    want_a, want_r = G.gae_padded(r, v, m, ne, 0.9, 0.8)
    a, rt = _compute_token_level_gae(r.to(dev), v.to(dev), m.to(dev), ne.to(dev), 0.9, 0.8)
    torch.testing.assert_close(a.cpu(), want_a, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(rt.cpu(), want_r, rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("bs,L", [(3, 7), (64, 1000), (5, 5000)])
def test_gae_padded_matches_oracle(dev, bs, L):
    g = torch.Generator().manual_seed(bs * 31 + L)
    r = torch.randn(bs, L, generator=g) * (torch.rand(bs, L, generator=g) > 0.9)
    v = torch.randn(bs, L, generator=g)
    lens = torch.randint(1, L + 1, (bs,), generator=g)
    lens[0] = L
    m = ((torch.arange(L)[None] < (lens[:, None] - 1)) & (torch.rand(bs, L, generator=g) > 0.2)).float()
    ne = lens == L
    lam = torch.rand(bs, generator=g) * 0.3 + 0.7
    for lam_arg in (0.95, lam):
        want_a, want_r = G.gae_padded(r, v, m, ne, 0.99, lam_arg)
        a, rt = _compute_token_level_gae(r.to(dev), v.to(dev), m.to(dev), ne.to(dev), 0.99,
                                         lam_arg.to(dev) if isinstance(lam_arg, torch.Tensor) else lam_arg)
        scale = want_a.abs().max().item()
        torch.testing.assert_close(a.cpu(), want_a, rtol=1e-4, atol=1e-5 * scale)
        torch.testing.assert_close(rt.cpu(), want_r, rtol=1e-4, atol=1e-5 * scale)


def test_gae_packed_matches_oracle_and_edge_cases(dev):
    g = torch.Generator().manual_seed(7)
    lens = torch.cat([torch.tensor([1, 2, 1]), torch.randint(1, 3000, (40,), generator=g), torch.tensor([1])])
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32)
    T = int(cu[-1])
    r, v = torch.randn(T, generator=g), torch.randn(T, generator=g)
    m = (torch.rand(T, generator=g) > 0.3).float()
    ne = torch.rand(lens.numel(), generator=g) > 0.5
    want_a, want_r = G.gae_packed(r, v, m, cu, ne, 1.0, 0.95)
    a, rt = compute_gae_packed(r.to(dev), v.to(dev), m.to(dev), cu.to(dev), ne.to(dev), 1.0, 0.95)
    scale = want_a.abs().max().item()
    torch.testing.assert_close(a.cpu(), want_a, rtol=1e-4, atol=1e-5 * scale)
    torch.testing.assert_close(rt.cpu(), want_r, rtol=1e-4, atol=1e-5 * scale)
    assert (a.cpu()[cu[1:].long() - 1] == 0).all()  # last token of every sequence
    # repeat runs are bit-identical
    a2, _ = compute_gae_packed(r.to(dev), v.to(dev), m.to(dev), cu.to(dev), ne.to(dev), 1.0, 0.95)
    assert torch.equal(a, a2)
    # empty input
    e = torch.empty(0, device=dev)
    a0, r0 = compute_gae_packed(e, e, e, torch.zeros(1, dtype=torch.int32, device=dev), None, 1.0, 0.95)
    assert a0.numel() == 0 and r0.numel() == 0


@pytest.mark.parametrize("lens", [
    [140_000],                                   # one very long sequence: the reduce-then-scan launches
    [1] * 5000,                                  # one-token sequences: thousands of ends per tile
    [0, 3, 0, 0, 2500, 0, 7, 0],                 # empty sequences between real ones
    [5, 70_000, 1, 2049, 2047, 4096, 1, 30_000], # ends on and around tile edges, long next to short (34 tiles
                                                 # of one sequence to the right of a tile)
    [2048] * 9,                                  # every end exactly on a tile edge
    [40_000, 3, 50_000],                         # long on average: the reduce-then-scan launches again
    [0, 0, 9000, 0, 8192, 0],                    # empty sequences at both ends and on a tile edge
], ids=["one-long", "unit", "empty", "mixed", "tile-aligned", "long-average", "empty-ends"])
def test_gae_packed_sequence_layouts(dev, lens):
    g = torch.Generator().manual_seed(len(lens) * 13 + lens[0])
    lens = torch.tensor(lens)
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32)
    T = int(cu[-1])
    r = torch.randn(T, generator=g) * (torch.rand(T, generator=g) > 0.8)
    v = torch.randn(T, generator=g)
    m = (torch.rand(T, generator=g) > 0.3).float()
    ne = torch.rand(lens.numel(), generator=g) > 0.5
    lam = torch.rand(lens.numel(), generator=g) * 0.2 + 0.8
    for lam_arg in (0.95, lam):
        want_a, want_r = G.gae_packed(r, v, m, cu, ne, 0.999, lam_arg)
        a, rt = compute_gae_packed(r.to(dev), v.to(dev), m.to(dev), cu.to(dev), ne.to(dev), 0.999,
                                   lam_arg.to(dev) if isinstance(lam_arg, torch.Tensor) else lam_arg)
        scale = max(want_a.abs().max().item(), 1.0)
        torch.testing.assert_close(a.cpu(), want_a, rtol=1e-4, atol=1e-5 * scale)
        torch.testing.assert_close(rt.cpu(), want_r, rtol=1e-4, atol=1e-5 * scale)


def test_gae_padded_long_rows(dev):
    # rows longer than a tile, and far longer (takes the reduce-then-scan launches)
    for bs, L in ((7, 8192), (3, 20_000), (300, 10_000), (2, 140_000)):
        g = torch.Generator().manual_seed(L)
        r = torch.randn(bs, L, generator=g) * (torch.rand(bs, L, generator=g) > 0.95)
        v = torch.randn(bs, L, generator=g)
        m = (torch.rand(bs, L, generator=g) > 0.1).float()
        m[:, -1] = 0
        ne = torch.tensor([i % 2 == 0 for i in range(bs)])
        want_a, want_r = G.gae_padded(r, v, m, ne, 1.0, 0.95)
        a, rt = _compute_token_level_gae(r.to(dev), v.to(dev), m.to(dev), ne.to(dev), 1.0, 0.95)
        scale = max(want_a.abs().max().item(), 1.0)
        torch.testing.assert_close(a.cpu(), want_a, rtol=1e-4, atol=1e-5 * scale)
        torch.testing.assert_close(rt.cpu(), want_r, rtol=1e-4, atol=1e-5 * scale)


def test_gae_sequences_are_independent(dev):
    """Changing one sequence must not change any other (the scan's reset maps)."""
    g = torch.Generator().manual_seed(3)
    lens = torch.randint(1, 5000, (30,), generator=g)
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32).to(dev)
    T = int(cu[-1])
    r, v = torch.randn(T, generator=g).to(dev), torch.randn(T, generator=g).to(dev)
    m = torch.ones(T, device=dev)
    a1, _ = compute_gae_packed(r, v, m, cu, None, 1.0, 0.95)
    s, e = int(cu[10]), int(cu[11])
    r2 = r.clone()
    r2[s:e] += 100.0
    a2, _ = compute_gae_packed(r2, v, m, cu, None, 1.0, 0.95)
    assert torch.equal(a1[:s], a2[:s]) and torch.equal(a1[e:], a2[e:])


NORM_CASES = [
    dict(mean_level="batch", std_level="batch"),
    dict(mean_level="batch", std_level="batch", std_unbiased=False),
    dict(mean_level="batch", std_level=None, mean_leave1out=True),
    dict(mean_level="batch", std_level="batch", mean_leave1out=True),
    dict(mean_level="group", std_level="group", group_size=4),
    dict(mean_level="group", std_level="group", group_size=4, std_unbiased=False, eps=0.0),
    dict(mean_level="group", std_level="batch", group_size=4),
    dict(mean_level="batch", std_level="group", group_size=4),
    dict(mean_level="group", std_level=None, group_size=4, mean_leave1out=True),
    dict(mean_level=None, std_level="batch"),
    dict(mean_level="group", std_level="group", group_size=5),  # 2 tail rows
    dict(mean_level="group", std_level="group", group_size=1, mean_leave1out=True),
]


@pytest.mark.parametrize("cfg", NORM_CASES, ids=[str(i) for i in range(len(NORM_CASES))])
@pytest.mark.parametrize("shape,masked", [((12, 40), True), ((12,), False), ((12, 700), True)])
def test_normalization_matches_oracle(dev, cfg, shape, masked):
    g = torch.Generator().manual_seed(len(shape) * 100 + shape[-1])
    x = torch.randn(*shape, generator=g) * 2 + 0.5
    m = (torch.rand(*shape, generator=g) > 0.35).float() if masked else None
    if masked:
        m[1] = 0  # a fully masked row
    want = N.normalization(x, m, **cfg)
    got = Normalization(NormConfig(**cfg))(x.to(dev), m.to(dev) if masked else None)
    assert got.dtype == torch.float32 and got.shape == x.shape
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-6 * want.abs().max().item())


def test_normalization_reference_literals(dev):
    x = _t([[1.0], [2.0], [3.0], [4.0]], dev)
    out = Normalization(NormConfig(mean_level="batch", std_level=None, mean_leave1out=True))(x, torch.ones_like(x))
    torch.testing.assert_close(out.cpu(), torch.tensor([[-2.0], [-2.0 / 3], [2.0 / 3], [2.0]]), atol=1e-6, rtol=0)
    x = _t([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]], dev)
    m = _t([[1.0, 1.0], [1.0, 0.0], [0.0, 1.0]], dev)
    out = Normalization(NormConfig(mean_level="batch", std_level="batch", mean_leave1out=True))(x, m).cpu()
    for got, want in [(out[0, 0], -0.9258), (out[0, 1], -0.4629), (out[1, 0], 0.0), (out[2, 1], 1.3887)]:
        assert got.item() == pytest.approx(want, abs=1e-3)
    x = _t([0.0, 3.0, 6.0, 10.0, 20.0, 1.0, 2.0, 3.0], dev)
    norm = Normalization(NormConfig(mean_level="group", std_level="group", group_size=2, std_unbiased=False, eps=0.0))
    out = norm(x, group_sizes=[3, 2, 3]).cpu().double()
    off = 0
    for s in [3, 2, 3]:
        c = x.cpu()[off:off + s].double()
        torch.testing.assert_close(out[off:off + s], (c - c.mean()) / c.std(unbiased=False), rtol=1e-5, atol=1e-5)
        off += s
    cfg = NormConfig(mean_level="group", std_level="group", group_size=2, std_unbiased=False, eps=1e-5)
    out = Normalization(cfg)(_t([0.0, 3.0, 6.0, 5.0, 5.0], dev), group_sizes=[3, 2])
    assert torch.isfinite(out).all() and (out[3:] == 0).all()
    cfg = NormConfig(mean_level="group", std_level="group", group_size=1, mean_leave1out=True)
    out = Normalization(cfg)(_t([7.0, 1.0, 5.0], dev), group_sizes=[1, 2])
    assert out[0].item() == 0.0
    # all-masked input comes back unchanged
    x = _t([1.0, 2.0, 3.0], dev)
    assert torch.equal(Normalization(NormConfig())(x, torch.zeros_like(x)), x)


def test_masked_normalization_matches_oracle(dev):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 300, generator=g) * 3 + 2
    m = (torch.rand(64, 300, generator=g) > 0.4).float()
    for unbiased in (False, True):
        want = N.masked_normalization(x, m, unbiased=unbiased)
        got = masked_normalization(x.to(dev), m.to(dev), unbiased=unbiased)
        torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-6)
    want = N.masked_normalization(x, None)
    torch.testing.assert_close(masked_normalization(x.to(dev)).cpu(), want, rtol=1e-5, atol=1e-6)
    # statistics per slice: trailing dimension, leading dimension, and a middle one of a 3-D tensor
    for dim in (-1, (0,), 1):
        want = N.masked_normalization(x, m, unbiased=True, dim=dim)
        got = masked_normalization(x.to(dev), m.to(dev), dim=dim, unbiased=True)
        torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-6)
    x3 = torch.randn(6, 50, 7, generator=g)
    m3 = (torch.rand(6, 50, 7, generator=g) > 0.2).float()
    for dim in ((1,), (0, 2), (0, 1, 2)):
        want = N.masked_normalization(x3, m3, dim=dim)
        got = masked_normalization(x3.to(dev), m3.to(dev), dim=dim)
        assert got.shape == x3.shape
        torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-6)
    want = N.masked_normalization(x3, None, dim=(2,))
    torch.testing.assert_close(masked_normalization(x3.to(dev), dim=(2,)).cpu(), want, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- turn-level GAE
def test_turn_level_gae_reference_literals(dev):
    from areal_amd.ppo.gae import _compute_turn_level_gae

    r = _t([[0.0, 1.0, 0.0, 2.0]], dev)
    a, rt = _compute_turn_level_gae(r, torch.zeros_like(r), torch.ones_like(r),
                                    torch.tensor([[0, 0, 1, 1]], dtype=torch.int32, device=dev),
                                    torch.tensor([False], device=dev), 1.0, 0.5)
    assert torch.equal(a.cpu(), torch.tensor([[2.0, 2.0, 2.0, 2.0]])) and torch.equal(rt, a)
    r = _t([[0.0, 3.0, 0.0, 0.0, 4.0]], dev)
    v = _t([[1.0, 5.0, 9.0, 2.0, 8.0]], dev)
    a, rt = _compute_turn_level_gae(r, v, _t([[1.0, 1.0, 0.0, 1.0, 1.0]], dev),
                                    torch.tensor([[0, 0, -1, 2, 2]], device=dev),
                                    torch.tensor([True], device=dev), 0.5, 0.25)
    assert torch.equal(a.cpu(), torch.tensor([[3.75, 3.75, 0.0, 6.0, 6.0]]))
    assert torch.equal(rt.cpu(), torch.tensor([[4.75, 4.75, 9.0, 8.0, 8.0]]))
    r = _t([[0.0, 1.0, 0.0, 2.0]] * 2, dev)
    a, _ = _compute_turn_level_gae(r, torch.zeros_like(r), torch.ones_like(r),
                                   torch.tensor([[0, 0, 1, 1]] * 2, dtype=torch.int32, device=dev),
                                   torch.tensor([False, False], device=dev), 1.0, _t([0.5, 0.0], dev))
    assert torch.equal(a.cpu(), torch.tensor([[2.0, 2.0, 2.0, 2.0], [1.0, 1.0, 2.0, 2.0]]))


@pytest.mark.parametrize("ids,message", [([-1, 0, 0, 1], "non-negative"), ([0, 0, 4, 4], "smaller than the sequence length"),
                                         ([0, 1, 0, 2], "temporally nondecreasing")])
def test_turn_level_gae_rejects_malformed_ids(dev, ids, message):
    from areal_amd.ppo.gae import _compute_turn_level_gae

    r = torch.zeros(1, 4, device=dev)
    with pytest.raises(RuntimeError, match=message):
        _compute_turn_level_gae(r, r, torch.ones_like(r), torch.tensor([ids], device=dev),
                                torch.tensor([False], device=dev), 1.0, 1.0)
    with pytest.raises(ValueError, match="integer dtype"):
        _compute_turn_level_gae(r, r, torch.ones_like(r), torch.zeros(1, 4, device=dev),
                                torch.tensor([False], device=dev), 1.0, 1.0)
    with pytest.raises(ValueError, match="must have shape"):
        _compute_turn_level_gae(r, r, torch.ones_like(r), torch.zeros(1, 3, dtype=torch.long, device=dev),
                                torch.tensor([False], device=dev), 1.0, 1.0)


@pytest.mark.parametrize("bs,L,max_turn_len", [(5, 37, 4), (16, 3000, 200), (3, 9000, 3000), (4, 1500, 1)])
def test_turn_level_gae_matches_oracle(dev, bs, L, max_turn_len):
    from areal_amd.ppo.gae import _compute_turn_level_gae

    g = torch.Generator().manual_seed(bs * 7 + L)
    ids = torch.full((bs, L), -1, dtype=torch.int64)
    mask = torch.zeros(bs, L)
    for b in range(bs):
        t, k = int(torch.randint(0, 5, (1,), generator=g)), 0
        while t < L:
            n = int(torch.randint(1, max_turn_len + 1, (1,), generator=g))
            ids[b, t:t + n] = k
            mask[b, t:t + n] = (torch.rand(min(n, L - t), generator=g) > 0.1).float()
            t += n + int(torch.randint(0, 6, (1,), generator=g))  # a gap (prompt / tool output)
            k += int(torch.randint(1, 3, (1,), generator=g))      # ids may skip
        ids[b][ids[b] >= L] = -1
        mask[b][ids[b] < 0] = 0
    r = torch.randn(bs, L, generator=g) * (torch.rand(bs, L, generator=g) > 0.7)
    v = torch.randn(bs, L, generator=g)
    ne = torch.rand(bs, generator=g) > 0.5
    lam = torch.rand(bs, generator=g) * 0.3 + 0.7
    for lam_arg in (0.9, lam):
        want_a, want_r = G.gae_turn_level(r, v, mask, ids, ne, 0.97, lam_arg)
        a, rt = _compute_turn_level_gae(r.to(dev), v.to(dev), mask.to(dev), ids.to(dev), ne.to(dev), 0.97,
                                        lam_arg.to(dev) if isinstance(lam_arg, torch.Tensor) else lam_arg)
        scale = max(want_a.abs().max().item(), 1.0)
        torch.testing.assert_close(a.cpu(), want_a, rtol=1e-4, atol=1e-5 * scale)
        torch.testing.assert_close(rt.cpu(), want_r, rtol=1e-4, atol=1e-5 * scale)


# ---------------------------------------------------------------- per-sample lambda, turn-mode advantages
def test_gae_lambda_context_reference_literals(dev):
    # reference tests/test_ppo_gae.py:279-341, :436-480
    from areal_amd.ppo.gae import _build_gae_lambda_context, compute_gae_lambda
    from areal_amd.ppo.lambda_fn import relative_position_gae_lambda, vapo_length_adaptive_gae

    mask = _t([[1, 1, 1, 1, 0], [1, 1, 0, 0, 0], [0, 0, 0, 0, 0]], dev)
    ids = torch.tensor([[0, 0, 1, 1, -1], [0, 1, -1, -1, -1], [-1, -1, -1, -1, -1]], dtype=torch.int32, device=dev)
    c = _build_gae_lambda_context(mask, ids, gae_timestep_unit="token")
    assert c["effective_token_lengths"].tolist() == [4, 2, 0] and c["turn_counts"].tolist() == [2, 2, 0]
    lam = compute_gae_lambda(vapo_length_adaptive_gae, {"alpha": 1.0}, mask, ids, "token")
    assert torch.equal(lam.cpu(), torch.tensor([0.75, 0.5, 0.0]))
    mask2 = _t([[1, 1, 0, 1, 1], [1, 1, 1, 1, 0], [0, 0, 0, 0, 0]], dev)
    ids2 = torch.tensor([[0, 0, -1, 2, 2], [0, 0, 0, 0, -1], [-1, -1, -1, -1, -1]], dtype=torch.int32, device=dev)
    lam = compute_gae_lambda(vapo_length_adaptive_gae, {"alpha": 1.0}, mask2, ids2, "turn")
    assert torch.equal(lam.cpu(), torch.tensor([0.5, 0.0, 0.0]))
    lam = compute_gae_lambda(relative_position_gae_lambda, {"q": 0.3}, torch.ones(2, 6, device=dev),
                             torch.tensor([[0, 0, 1, 1, 2, 2], [0] * 6], dtype=torch.int32, device=dev), "turn")
    torch.testing.assert_close(lam.cpu(), torch.tensor([0.3 ** 0.5, 1.0]), rtol=1e-6, atol=1e-7)
    lam = compute_gae_lambda(vapo_length_adaptive_gae, {"alpha": 1.0}, _t([[1, 1], [1, 0]], dev), None, "token")
    assert torch.equal(lam.cpu(), torch.tensor([0.5, 0.0]))
    with pytest.raises(ValueError, match="one value per local trajectory"):
        compute_gae_lambda(lambda context: torch.tensor(0.5, device=dev), {}, torch.ones(2, 2, device=dev),
                           torch.zeros(2, 2, dtype=torch.int32, device=dev), "token")
    with pytest.raises(ValueError, match="requires rollout data to include 'turn_ids'"):
        _build_gae_lambda_context(mask, None, gae_timestep_unit="turn")
    # long rows: counts over several chunks of the row
    g = torch.Generator().manual_seed(0)
    m = (torch.rand(7, 5000, generator=g) > 0.4).float()
    tid = (torch.arange(5000) // 37).expand(7, -1).to(torch.int32)
    c = _build_gae_lambda_context(m.to(dev), tid.to(dev), gae_timestep_unit="turn")
    assert torch.equal(c["effective_token_lengths"].cpu(), m.sum(1).long())
    want_turns = torch.tensor([len(set(tid[b][m[b] > 0].tolist())) for b in range(7)])
    assert torch.equal(c["timestep_lengths"].cpu(), want_turns)


def test_compute_advantages_relative_position_lambda_main_path(dev):
    # reference tests/test_ppo_gae.py:406-433: a terminal reward decays as q^((L-k)/(L-1))
    from areal_amd.ppo.actor import compute_advantages

    q, L = 0.3, 10
    batch = {
        "input_ids": torch.zeros(1, L + 1, dtype=torch.long, device=dev),
        "loss_mask": torch.tensor([[0] + [1] * L], dtype=torch.float32, device=dev),
        "logprobs": torch.zeros(1, L + 1, device=dev),
        "attention_mask": torch.ones(1, L + 1, dtype=torch.bool, device=dev),
        "rewards": torch.tensor([1.0], device=dev),
    }
    # the lambda function named by its dotted path, as the reference's configuration does
    out = compute_advantages(batch, gae_lambda="areal_amd.ppo.lambda_fn.relative_position_gae_lambda",
                             gae_lambda_kwargs={"q": q})
    want = torch.tensor([[q ** ((L - k) / (L - 1)) for k in range(1, L + 1)] + [0.0]])
    torch.testing.assert_close(out["advantages"].cpu(), want, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(out["returns"].cpu(), want, rtol=1e-6, atol=1e-7)


def test_compute_advantages_turn_mode_keeps_kl_token_local(dev):
    # reference tests/test_ppo_gae.py:551-583 in spirit: turn advantages broadcast, the token
    # KL penalty added per token, returns carry the task reward only
    from areal_amd.ppo.actor import compute_advantages
    from areal_amd.data import KLEstimator

    L = 6
    batch = {
        "input_ids": torch.zeros(1, L, dtype=torch.long, device=dev),
        "loss_mask": torch.tensor([[0, 1, 1, 1, 1, 0]], dtype=torch.float32, device=dev),
        "logprobs": torch.tensor([[0.0, -1.0, -2.0, -1.0, -3.0, 0.0]], device=dev),
        "ref_logp": torch.tensor([[-1.5, -1.0, -1.0, -2.5, 0.0, 0.0]], device=dev),
        "attention_mask": torch.tensor([[1, 1, 1, 1, 1, 0]], dtype=torch.bool, device=dev),
        "rewards": torch.tensor([2.0], device=dev),
        "turn_ids": torch.tensor([[-1, 0, 0, 1, 1, -1]], device=dev),
    }
    out = compute_advantages(dict(batch), kl_ctl=0.1, kl_estimator=KLEstimator("k1"), gae_timestep_unit="turn",
                             gae_lambda=0.5)
    # rolled mask [1,1,1,1,0,0], rolled ids [0,0,1,1,-1,-1]; reward 2 at position seqlen-2 = 3
    # turns: R = [0, 2], V = 0: A_1 = 2, A_0 = 0 + 0.5 * 2 = 1
    kl = out["kl_rewards"].cpu()
    want_adv = torch.tensor([[1.0, 1.0, 2.0, 2.0, 0.0, 0.0]]) + kl * torch.tensor([[1, 1, 1, 1, 0, 0.0]])
    want_adv[0, 4] = 0.0
    torch.testing.assert_close(out["advantages"].cpu(), want_adv, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(out["returns"].cpu(), torch.tensor([[1.0, 1.0, 2.0, 2.0, 0.0, 0.0]]), rtol=1e-6, atol=1e-7)
    with pytest.raises(ValueError, match="requires rollout data to"):
        b2 = dict(batch)
        del b2["turn_ids"]
        compute_advantages(b2, gae_timestep_unit="turn")


@pytest.mark.parametrize("mean_level,std_level", [("group", "group"), ("batch", "batch"), ("batch", "group"),
                                                  ("group", None), (None, "batch")])
def test_compute_advantages_fused_gae_and_normalisation_equal_the_two_stage_route(dev, monkeypatch, mean_level,
                                                                                   std_level):
    """Long padded rows: the GAE kernel leaves each row's masked sums and the advantage
    normalisation is its apply pass alone. Same advantages as GAE followed by the full
    normalisation (and as the oracle), tail rows outside any group included."""
    import areal_amd.ppo.actor as A
    from areal_amd.config import NormConfig
    from areal_amd.data import KLEstimator, Normalization
    from oracle import gae as G
    from oracle import norm as N

    bs, L = 68, 4096  # 8 groups of 8 rows + 4 tail rows
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(300, L, (bs,), generator=g)
    pos = torch.arange(L)[None]
    attn = pos < lens[:, None]
    data = dict(input_ids=torch.zeros(bs, L, dtype=torch.long), attention_mask=attn,
                loss_mask=(pos >= (lens // 4)[:, None]) & attn,
                logprobs=torch.randn(bs, L, generator=g) * 0.1 - 1,
                values=torch.randn(bs, L, generator=g), rewards=(torch.rand(bs, generator=g) > 0.5).float())
    data = {k: v.to(dev) for k, v in data.items()}
    norm = Normalization(NormConfig(mean_level=mean_level, std_level=std_level, group_size=8))
    kw = dict(kl_ctl=0.0, kl_estimator=KLEstimator("k1"), adv_norm=norm, discount=1.0, gae_lambda=0.95)

    calls = []
    real = A._token_level_gae_with_row_stats

    def spy(*a, **k):
        calls.append(1)
        return real(*a, **k)

    monkeypatch.setattr(A, "_token_level_gae_with_row_stats", spy)
    fused = A.compute_advantages(dict(data), **kw)
    assert calls, "the fused route was not taken"
    monkeypatch.setattr(A, "_token_level_gae_with_row_stats", lambda *a, **k: None)
    staged = A.compute_advantages(dict(data), **kw)
    assert torch.equal(fused["returns"], staged["returns"])
    scale = staged["advantages"].abs().max().item()
    torch.testing.assert_close(fused["advantages"], staged["advantages"], rtol=1e-5, atol=1e-6 * scale)
    # and against the oracle: GAE of the shaped rewards, then the normalisation
    want_a, _ = G.gae_padded(fused["tot_rewards"].cpu(), data["values"].cpu(), fused["loss_mask"].cpu().float(),
                             torch.zeros(bs, dtype=torch.bool), 1.0, 0.95)
    want = N.normalization(want_a, fused["loss_mask"].cpu().float(), mean_level=mean_level, std_level=std_level,
                           group_size=8)
    torch.testing.assert_close(fused["advantages"].cpu(), want, rtol=1e-4, atol=1e-5 * want.abs().max().item())


def _pad_packed(x, cu, fill=0.0):
    lens = (cu[1:] - cu[:-1]).long()
    L = max(int(lens.max()), 1)
    out = torch.full((lens.numel(), L), fill, dtype=x.dtype)
    pos = torch.arange(x.numel()) - cu[:-1].long().repeat_interleave(lens)
    rows = torch.arange(lens.numel()).repeat_interleave(lens)
    out[rows, pos] = x
    return out, (rows, pos)


_MANY = torch.Generator().manual_seed(99)
PACKED_NORM_LAYOUTS = {
    # more sequences than the kernel keeps of cu_seqlens in LDS, six or seven groups per 2048-token tile
    "many": dict(lens=torch.randint(1, 40, (5000,), generator=_MANY).tolist(), group_size=16),
    # sequences per tile of 2048 tokens: several groups inside one tile
    "short": dict(lens=[300, 17, 450, 1, 612, 95, 800, 333, 64, 2, 700, 410, 129, 256, 31, 999], group_size=2),
    # groups that cross tile boundaries, one sequence of several tiles, an empty sequence
    "long": dict(lens=[5000, 1200, 0, 2048, 4096, 37, 7000, 2047, 2049, 1], group_size=2),
    # explicit uneven groups
    "uneven": dict(lens=[1500, 700, 2600, 90, 3100, 512, 800, 1300, 1900], group_sizes=[1, 3, 2, 3]),
    # rows after the last whole group form the tail (mean 0, deviation 0 at group level)
    "tail": dict(lens=[900, 1100, 2100, 700, 1600, 450, 3000], group_size=3),
}


@pytest.mark.parametrize("cfg", [
    dict(mean_level="group", std_level="group"),
    dict(mean_level="group", std_level="group", std_unbiased=False, eps=0.0),
    dict(mean_level="batch", std_level="batch"),
    dict(mean_level="batch", std_level="group"),
    dict(mean_level="group", std_level=None),
    dict(mean_level="group", std_level="batch"),           # needs the second statistics pass
    dict(mean_level="group", std_level="group", mean_leave1out=True),  # so does leave-one-out
], ids=["gg", "gg_biased", "bb", "bg", "g_none", "gb", "gg_loo"])
@pytest.mark.parametrize("layout", list(PACKED_NORM_LAYOUTS))
@pytest.mark.parametrize("float_mask", [False, True], ids=["mask01", "maskf"])
def test_packed_gae_then_normalisation_matches_oracle(dev, cfg, layout, float_mask):
    """GAE over packed sequences whose kernel also leaves the normalisation's sums, then the one
    apply launch: against the oracle's GAE and its normalisation of the padded form."""
    from areal_amd.ppo.gae import compute_gae_packed_normalized

    spec = PACKED_NORM_LAYOUTS[layout]
    lens = torch.tensor(spec["lens"])
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32)
    T = int(cu[-1])
    g = torch.Generator().manual_seed(T)
    r = torch.randn(T, generator=g) * 0.3
    v = torch.randn(T, generator=g)
    m = (torch.rand(T, generator=g) > 0.3).float()
    if float_mask:
        m = m * (0.5 + torch.rand(T, generator=g))
    ne = torch.rand(lens.numel(), generator=g) > 0.5
    group_sizes = spec.get("group_sizes")
    full = dict(cfg, group_size=spec.get("group_size", 1))
    norm = Normalization(NormConfig(**full))
    # a lambda per sequence on the float-mask runs, one scalar otherwise
    lam = (0.5 + 0.5 * torch.rand(lens.numel(), generator=g)) if float_mask else 0.9
    got, ret, raw = compute_gae_packed_normalized(r.to(dev), v.to(dev), m.to(dev), cu.to(dev), ne.to(dev), 0.99,
                                                  lam.to(dev) if float_mask else lam, norm, group_sizes=group_sizes)
    want_a, want_r = G.gae_packed(r, v, m, cu, ne, 0.99, lam)
    scale = want_a.abs().max().item()
    torch.testing.assert_close(raw.cpu(), want_a, rtol=1e-4, atol=1e-5 * scale)
    torch.testing.assert_close(ret.cpu(), want_r, rtol=1e-4, atol=1e-5 * scale)
    # the oracle normalises the padded form of the advantages the kernel wrote
    pa, idx = _pad_packed(raw.cpu(), cu)
    pm, _ = _pad_packed(m, cu)
    want = N.normalization(pa, pm, group_sizes=group_sizes, **full)[idx]
    big = max(1.0, want[torch.isfinite(want)].abs().max().item())
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-5 * big, equal_nan=True)  # 0 / 0 in a tail group with eps 0
    # and the separate statistics pass gives the same
    two_stage = norm.packed(raw, m.to(dev), cu.to(dev), group_sizes)
    torch.testing.assert_close(got, two_stage, rtol=1e-5, atol=1e-6 * big, equal_nan=True)


def test_packed_gae_segment_sums_equal_fp64_group_sums(dev):
    """The (tile, group) segment sums the packed GAE kernel leaves (four entries per segment, one
    per wave of the tile's block) add up, per segment, per group and over the whole array, to the
    fp64 sums of the advantages it wrote; slots of no segment are zero."""
    from areal_amd import _lib

    lib = _lib.load()
    g = torch.Generator().manual_seed(11)
    lens = torch.clamp((torch.randn(96, generator=g) + 6.5).exp().long(), 1, 6000)
    lens[7] = 0
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32)
    T, S = int(cu[-1]), lens.numel()
    seq_off = torch.tensor([0, 8, 9, 9, 24, 40, 60, 96])  # uneven groups of whole sequences, one empty
    goff = cu.long()[seq_off]
    G_ = goff.numel() - 1
    r = torch.randn(T, generator=g)
    v = torch.randn(T, generator=g)
    m = (torch.rand(T, generator=g) > 0.4).float() * (0.25 + torch.rand(T, generator=g))
    nbytes = lib.areal_gae_segment_stats_bytes(T, G_)
    slots = nbytes // 160
    assert slots == (T + 2047) // 2048 + G_
    seg = torch.full((5, slots, 4), float("nan"), dtype=torch.float64, device=dev)
    adv, ret = torch.empty(T, device=dev), torch.empty(T, device=dev)
    rd, vd, md, cud, gd = r.to(dev), v.to(dev), m.to(dev), cu.to(dev), goff.to(dev)
    rc = lib.areal_gae_packed_group_stats(_lib.ptr(rd), _lib.ptr(vd), _lib.ptr(md), _lib.ptr(cud), None, None, T, S,
                                          1.0, 0.95, _lib.ptr(gd), G_, _lib.ptr(adv), _lib.ptr(ret), _lib.ptr(seg),
                                          nbytes, _lib.stream_ptr(dev))
    assert rc == 0
    seg = seg.cpu()
    assert torch.isfinite(seg).all()
    seg = seg.sum(2)
    x, md64 = adv.cpu().double(), m.double()
    terms = torch.stack([md64, x * md64, md64 * md64, md64 * md64 * x, (md64 * x) ** 2])
    used = torch.zeros(slots, dtype=torch.bool)
    for j in range(G_):
        a, b = int(goff[j]), int(goff[j + 1])
        if b == a:
            continue
        k0, k1 = a // 2048, (b - 1) // 2048
        used[k0 + j:k1 + j + 1] = True
        torch.testing.assert_close(seg[:, k0 + j:k1 + j + 1].sum(1), terms[:, a:b].sum(1), rtol=1e-12, atol=1e-12)
        for k in range(k0, k1 + 1):  # every segment on its own
            lo, hi = max(a, k * 2048), min(b, (k + 1) * 2048)
            torch.testing.assert_close(seg[:, k + j], terms[:, lo:hi].sum(1), rtol=1e-12, atol=1e-12)
    assert (seg[:, ~used] == 0).all()
    torch.testing.assert_close(seg.sum(1), terms.sum(1), rtol=1e-12, atol=1e-12)
