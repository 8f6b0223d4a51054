"""Pins of the CPU oracle for packing / padding and the masked statistics: hand-written cases for
every branch (the reference's tests hold no literals for these functions)."""

import pytest
import torch

from oracle import packing as P


def test_pack_takes_the_left_part_of_every_row():
    mask = torch.tensor([[1, 1, 1, 0], [1, 0, 0, 0], [1, 1, 1, 1]])
    x = torch.arange(12).view(3, 4)
    y = torch.arange(24.0).view(3, 4, 2)
    out = P.pack_tensor_dict(dict(attention_mask=mask, input_ids=x, feats=y, other="keep", vec=torch.ones(3)))
    assert out["cu_seqlens"].tolist() == [0, 3, 4, 8] and out["cu_seqlens"].dtype == torch.int32
    assert out["max_seqlen"] == 4
    assert out["input_ids"].tolist() == [0, 1, 2, 4, 8, 9, 10, 11]
    assert out["feats"][3].tolist() == [8.0, 9.0]
    assert out["other"] == "keep" and out["vec"].shape == (3,) and "attention_mask" not in out


def test_pad_appends_one_pad_sequence():
    data = dict(cu_seqlens=torch.tensor([0, 3, 5], dtype=torch.int32), max_seqlen=3,
                input_ids=torch.tensor([7, 8, 9, 1, 2]), loss_mask=torch.ones(5),
                position_ids=torch.tensor([0, 1, 2, 0, 1]), meta=3)
    out, pad, old_cu, align = P.pad_packed_tensor_dict(data, 9, pad_value=0.0)
    assert pad == 4 and align is None and old_cu.tolist() == [0, 3, 5]
    assert out["cu_seqlens"].tolist() == [0, 3, 5, 9] and out["max_seqlen"] == 4
    assert out["input_ids"].tolist() == [7, 8, 9, 1, 2, 0, 0, 0, 0]
    assert out["position_ids"].tolist() == [0, 1, 2, 0, 1, 0, 1, 2, 3]
    assert out["meta"] == 3
    same, pad0, _, _ = P.pad_packed_tensor_dict(data, 5)
    assert pad0 == 0 and same is data
    with pytest.raises(ValueError, match="smaller than total length"):
        P.pad_packed_tensor_dict(data, 4)


def test_sequence_alignment_and_page_rounding():
    data = dict(cu_seqlens=torch.tensor([0, 3, 5], dtype=torch.int32), max_seqlen=3,
                input_ids=torch.tensor([7, 8, 9, 1, 2]), position_ids=torch.tensor([5, 6, 7, 5, 6]),
                pos3=None)
    out, pad, old_cu, align = P.pad_packed_tensor_dict(data, 10, pad_value=-1, seq_align_to=4)
    # sequences 3 -> 4 and 2 -> 4 tokens; pad_to_length rounded up to lcm(4, 256) = 256
    assert align == 8 and pad == 248 and old_cu.tolist() == [0, 3, 5]
    assert out["cu_seqlens"].tolist() == [0, 4, 8, 256] and out["max_seqlen"] == 248
    assert out["input_ids"][:8].tolist() == [7, 8, 9, -1, 1, 2, -1, -1]
    assert (out["input_ids"][8:] == -1).all()
    # 1-D position ids are rewritten as 0..len-1 of the aligned sequence, then the pad counts on
    assert out["position_ids"][:10].tolist() == [0, 1, 2, 3, 0, 1, 2, 3, 0, 1]


def test_sequence_alignment_three_channel_position_ids_and_total_bump():
    pos = torch.tensor([[0, 0, 0], [1, 1, 1], [2, 5, 5], [0, 0, 0], [1, 2, 3]])
    data = dict(cu_seqlens=torch.tensor([0, 3, 5], dtype=torch.int32), max_seqlen=3, position_ids=pos)
    out, pad, _, align = P.pad_packed_tensor_dict(data, 0, seq_align_to=256)
    # total after alignment (512) exceeds pad_to_length (0 -> 0): bumped to 512, no batch pad
    assert align == 512 and pad == 0
    p = out["position_ids"]
    assert p.shape == (512, 3) and p[2].tolist() == [2, 5, 5]
    assert p[3].tolist() == [0, 0, 0] and p[4].tolist() == [1, 1, 1] and p[255].tolist() == [252] * 3
    assert p[256 + 1].tolist() == [1, 2, 3] and p[256 + 2].tolist() == [0, 0, 0]


def test_unpack_reorder_pad_and_round_trip():
    packed = torch.arange(12.0).view(6, 2)
    out = P.unpack_reorder_pad(packed, [1, 3, 2], [2, 0, 1])
    assert out.shape == (3, 3, 2)
    assert out[0, :2].tolist() == [[8.0, 9.0], [10.0, 11.0]] and out[0, 2].tolist() == [0.0, 0.0]
    assert out[1, 0].tolist() == [0.0, 1.0] and (out[1, 1:] == 0).all()
    g = torch.Generator().manual_seed(0)
    lens = torch.randint(1, 9, (5,), generator=g)
    mask = (torch.arange(8)[None] < lens[:, None]).long()
    x = torch.randn(5, 8, generator=g) * mask
    d = P.pack_tensor_dict(dict(attention_mask=mask, x=x))
    back = P.unpack_reorder_pad(d["x"], lens.tolist())
    assert torch.equal(back, x[:, : int(lens.max())])


def test_masked_stats_brute_force():
    g = torch.Generator().manual_seed(1)
    v = torch.randn(50, generator=g)
    m = torch.rand(50, generator=g) > 0.5
    out = P.masked_stats(dict(a=v, b=v, c=v), dict(a=m, b=None, c=torch.zeros(50, dtype=torch.bool)))
    sel = [float(v[i]) for i in range(50) if m[i]]
    assert abs(out["a"]["sum"] - sum(sel)) < 1e-5 and out["a"]["count"] == len(sel)
    assert abs(out["a"]["min"] - min(sel)) < 1e-7 and abs(out["a"]["max"] - max(sel)) < 1e-7
    assert abs(out["b"]["avg"] - float(v.double().mean())) < 1e-7 and out["b"]["count"] == 50
    assert out["c"]["avg"] is None and out["c"]["min"] is None and out["c"]["max"] is None
