"""HIP packing / padding / statistics kernels through the C ABI against the CPU oracle
(byte-exact for the data movement, 1e-6 relative for the fp64 sums)."""

import types

import pytest
import torch

from areal_amd.packing import pack_tensor_dict, pad_packed_tensor_dict, reorder_and_pad_outputs, unpack_reorder_pad
from areal_amd.stats import masked_stats
from oracle import packing as P

pytestmark = pytest.mark.gpu


def _to(d, dev):
    return {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in d.items()}


def _same(a, b):
    assert a.keys() == b.keys()
    for k in a:
        if torch.is_tensor(b[k]):
            assert a[k].dtype == b[k].dtype and a[k].shape == b[k].shape, k
            assert torch.equal(a[k].cpu(), b[k]), k
        else:
            assert a[k] == b[k], k


def _batch(bs, S, seed):
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(1, S + 1, (bs,), generator=g)
    lens[0] = S
    mask = torch.arange(S)[None] < lens[:, None]
    return dict(
        attention_mask=mask,
        input_ids=torch.randint(0, 150000, (bs, S), generator=g),
        loss_mask=(torch.rand(bs, S, generator=g) > 0.5) & mask,
        logprobs=torch.randn(bs, S, generator=g),
        values=torch.randn(bs, S, generator=g).bfloat16(),
        feats=torch.randn(bs, S, 3, generator=g),
        odd=torch.randint(0, 255, (bs, S, 5), generator=g).to(torch.uint8),
        rewards=torch.randn(bs, generator=g),
        name="batch",
    )


@pytest.mark.parametrize("bs,S", [(1, 1), (3, 4), (37, 700), (600, 33)])
def test_pack_tensor_dict_matches_oracle(dev, bs, S):
    data = _batch(bs, S, bs + S)
    want = P.pack_tensor_dict(data)
    got = pack_tensor_dict(_to(data, dev))
    assert isinstance(got["max_seqlen"], int)
    _same(got, want)
    with pytest.raises(AssertionError):
        pack_tensor_dict(dict(x=data["input_ids"].to(dev)))


def test_pack_more_tensors_than_one_launch_takes_and_a_wide_one(dev):
    """Ten packed tensors (two launches of at most eight) and one with 8 KiB per token, whose
    chunks are two tokens long."""
    g = torch.Generator().manual_seed(7)
    bs, S = 9, 300
    lens = torch.randint(1, S + 1, (bs,), generator=g)
    mask = torch.arange(S)[None] < lens[:, None]
    data = dict(attention_mask=mask, wide=torch.randn(bs, S, 2048, generator=g))
    for i in range(9):
        data[f"t{i}"] = torch.randint(-1000, 1000, (bs, S), generator=g).to(
            [torch.int64, torch.int32, torch.int16, torch.int8][i % 4])
    _same(pack_tensor_dict(_to(data, dev)), P.pack_tensor_dict(data))


@pytest.mark.parametrize("align", [None, 8, 256])
@pytest.mark.parametrize("three", [False, True])
def test_pad_packed_tensor_dict_matches_oracle(dev, align, three):
    g = torch.Generator().manual_seed(17)
    lens = torch.randint(1, 300, (23,), generator=g)
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32)
    total = int(cu[-1])
    pos = torch.cat([torch.arange(n) for n in lens.tolist()])
    if three:
        pos = torch.stack([pos, pos + 1, pos * 2], dim=1)
    data = dict(cu_seqlens=cu, max_seqlen=int(lens.max()), input_ids=torch.randint(0, 1000, (total,), generator=g),
                loss_mask=torch.rand(total, generator=g) > 0.5, logprobs=torch.randn(total, generator=g),
                old=torch.randn(total, generator=g).bfloat16(), position_ids=pos, scalar=torch.ones(3), tag="x")
    for pad_to, pad_value in ((total + 100, 0.0), (total, 0.0), (4096, -1.0)):
        want = P.pad_packed_tensor_dict(dict(data), pad_to, pad_value, align)
        got = pad_packed_tensor_dict(_to(data, dev), pad_to, pad_value, align)
        _same(got[0], want[0])
        assert got[1] == want[1] and got[3] == want[3]
        assert torch.equal(got[2].cpu(), want[2])
    with pytest.raises(ValueError, match="smaller than total length"):
        pad_packed_tensor_dict(_to(data, dev), total - 1)


def test_unpack_reorder_pad_and_round_trip(dev):
    g = torch.Generator().manual_seed(3)
    lens = torch.randint(1, 500, (41,), generator=g).tolist()
    perm = torch.randperm(41, generator=g).tolist()
    for x in (torch.randn(sum(lens), generator=g), torch.randn(sum(lens), 7, generator=g).bfloat16(),
              torch.randint(0, 100, (sum(lens), 2, 3), generator=g)):
        want = P.unpack_reorder_pad(x, lens, perm)
        got = unpack_reorder_pad(x.to(dev), lens, perm)
        assert got.dtype == want.dtype and torch.equal(got.cpu(), want)
    mb = types.SimpleNamespace(forward_indices=perm, backward_indices=torch.argsort(torch.tensor(perm)).tolist())
    seqlens = torch.randint(1, 50, (41,), generator=g).tolist()
    outs = [torch.randn(seqlens[i], generator=g) for i in perm]          # micro-batch order
    got = reorder_and_pad_outputs([o.to(dev) for o in outs[:20]] + [torch.cat(outs[20:]).to(dev)], seqlens, mb)
    for i in range(41):                                                   # back in the original order
        assert torch.equal(got[i, : seqlens[i]].cpu(), outs[perm.index(i)])
        assert (got[i, seqlens[i]:] == 0).all()
    # pack then unpack restores the padded batch
    data = _batch(19, 130, 5)
    packed = pack_tensor_dict(_to(data, dev))
    lens2 = data["attention_mask"].sum(1).tolist()
    back = unpack_reorder_pad(packed["feats"], lens2)
    assert torch.equal(back.cpu(), (data["feats"] * data["attention_mask"][..., None])[:, : max(lens2)])
    with pytest.raises(ValueError):
        unpack_reorder_pad(packed["feats"], [1, 2])


def test_masked_stats_matches_oracle(dev):
    g = torch.Generator().manual_seed(9)
    n = 200_003
    vals = {f"s{i}": torch.randn(n, generator=g) * (i + 1) for i in range(35)}   # more than one launch
    dens = {k: (torch.rand(n, generator=g) > 0.3) for k in vals}
    dens["s3"] = None
    dens["s4"] = torch.zeros(n, dtype=torch.bool)
    vals["s5"] = (torch.rand(n, generator=g) > 0.5).float().view(n // 1, 1).view(n)
    want = P.masked_stats(vals, dens)
    got = masked_stats({k: v.to(dev) for k, v in vals.items()},
                       {k: (v.to(dev) if v is not None else None) for k, v in dens.items()})
    for k in vals:
        assert got[k]["count"] == want[k]["count"], k
        if want[k]["avg"] is None:
            assert got[k]["avg"] is None and got[k]["min"] is None and got[k]["max"] is None
            continue
        assert abs(got[k]["sum"] - want[k]["sum"]) <= 1e-6 * max(1.0, abs(want[k]["sum"])) + 1e-3, k
        assert got[k]["min"] == want[k]["min"] and got[k]["max"] == want[k]["max"], k
