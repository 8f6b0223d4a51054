"""Oracle: packing / padding of token batches and masked logging statistics (CPU, test-only).

Restates with the reference's own per-sequence loops:
  * ``areal/utils/data.py:496-545`` pack_tensor_dict;
  * ``data.py:822-982`` pad_packed_tensor_dict (``N_TOKENS_PER_PAGE = 256``, :819);
  * ``data.py:436-449`` unpack_sequence, ``:50-52`` reorder_list, ``:548-559``
    pad_and_stack_tensors_along_first_dim, composed as ``reorder_and_pad_outputs`` does
    (``areal/engine/core/train_engine.py:110-144``);
  * ``areal/utils/stats_tracker.py:455-560`` the masked sum / average / min / max of a logged
    tensor under its denominator.

The reference's tests hold no literal for these functions (tests/test_utils.py:41-53 only packs
inside a micro-batch split): "parity unpinned" against golden vectors.  Pinned by
(tests/test_oracle_packing.py): hand-written small cases for every branch (right-padded rows,
sequence alignment with both position-id layouts, the trailing pad sequence, the lcm rounding
and the "total exceeds pad_to_length" bump), the pack -> unpack round trip, and brute-force
Python loops for the statistics.
"""

from __future__ import annotations

import math
from typing import Any

import torch
import torch.nn.functional as F

N_TOKENS_PER_PAGE = 256


def pack_tensor_dict(data: dict[str, Any]) -> dict[str, Any]:
    mask = data["attention_mask"]
    bs, seq_len = mask.shape
    lens = mask.sum(dim=1, dtype=torch.int32)
    max_seqlen = int(lens.max())
    cu = F.pad(torch.cumsum(lens, dim=0, dtype=torch.int32), (1, 0), value=0)
    total = int(cu[-1])
    out: dict[str, Any] = {}
    for key, value in data.items():
        if key == "attention_mask":
            out["cu_seqlens"] = cu
            out["max_seqlen"] = max_seqlen
        elif torch.is_tensor(value) and value.ndim >= 2 and value.shape[0] == bs and value.shape[1] == seq_len:
            packed = torch.empty((total, *value.shape[2:]), dtype=value.dtype)
            for i in range(bs):
                s, e = int(cu[i]), int(cu[i + 1])
                packed[s:e] = value[i][: e - s]
            out[key] = packed
        else:
            out[key] = value
    return out


def pad_packed_tensor_dict(data, pad_to_length, pad_value=0.0, seq_align_to=None):
    cu = data["cu_seqlens"]
    max_seqlen = data["max_seqlen"]
    old_cu = cu.clone()
    total = int(cu[-1])
    align_to_length = None
    if seq_align_to is not None:
        lens = cu[1:] - cu[:-1]
        bs = lens.shape[0]
        lens_p = lens + (-lens) % seq_align_to
        cu_p = torch.zeros(bs + 1, dtype=torch.int32)
        cu_p[1:] = torch.cumsum(lens_p, dim=0)
        new: dict[str, Any] = {}
        for key, value in data.items():
            if key == "cu_seqlens":
                new[key] = cu_p
            elif key == "max_seqlen":
                new[key] = int(lens_p.max())
            elif key == "position_ids":
                if value.ndim == 2 and value.shape[1] == 3:
                    v = torch.zeros((int(lens_p.sum()), 3), dtype=value.dtype)
                    for i in range(bs):
                        ns, ne, os_, oe = int(cu_p[i]), int(cu_p[i + 1]), int(cu[i]), int(cu[i + 1])
                        n = oe - os_
                        v[ns : ns + n] = value[os_:oe]
                        v[ns + n : ne] = torch.arange(ne - ns - n).unsqueeze(1).expand(-1, 3)
                else:
                    v = torch.zeros((int(lens_p.sum()),), dtype=value.dtype)
                    for i in range(bs):
                        ns, ne = int(cu_p[i]), int(cu_p[i + 1])
                        v[ns:ne] = torch.arange(ne - ns, dtype=value.dtype)
                new[key] = v
            elif torch.is_tensor(value) and value.numel() == total:
                v = torch.full((int(lens_p.sum()),), fill_value=pad_value, dtype=value.dtype)
                for i in range(bs):
                    ns, s, e = int(cu_p[i]), int(cu[i]), int(cu[i + 1])
                    v[ns : ns + e - s] = value[s:e]
                new[key] = v
            else:
                new[key] = value
        data = new
        align_to_length = int(cu_p[-1])
        lcm = math.lcm(seq_align_to, N_TOKENS_PER_PAGE)
        pad_to_length = (pad_to_length + lcm - 1) // lcm * lcm
        cu, max_seqlen, total = data["cu_seqlens"], data["max_seqlen"], int(data["cu_seqlens"][-1])
        if pad_to_length < total:
            pad_to_length = (total + lcm - 1) // lcm * lcm
    pad_length = pad_to_length - total
    if pad_length < 0:
        raise ValueError(f"pad_to_length {pad_to_length} is smaller than total length {total}.")
    if pad_length == 0:
        return data, pad_length, old_cu, align_to_length
    out: dict[str, Any] = {}
    for key, value in data.items():
        if key == "cu_seqlens":
            out[key] = F.pad(cu, (0, 1), value=pad_to_length)
        elif key == "max_seqlen":
            out[key] = max(max_seqlen, pad_length)
        elif key == "position_ids":
            pad = torch.arange(pad_length, dtype=torch.long)
            if value.ndim == 2 and value.shape[1] == 3:
                pad = pad.unsqueeze(1).expand(-1, 3)
            out[key] = torch.cat([value, pad])
        elif torch.is_tensor(value) and value.numel() == total:
            out[key] = F.pad(value, (0, pad_length), value=pad_value)
        else:
            out[key] = value
    return out, pad_length, old_cu, align_to_length


def unpack_reorder_pad(packed, seqlens, backward_indices=None):
    parts = list(torch.split(packed, seqlens, dim=0))
    if backward_indices is not None:
        assert len(set(backward_indices)) == len(parts)
        parts = [parts[i] for i in backward_indices]
    max_len = max(p.shape[0] for p in parts)
    n_dim = parts[0].ndim
    rows = [F.pad(p, (0,) * (2 * (n_dim - 1)) + (0, max_len - p.shape[0]), value=0.0) for p in parts]
    return torch.stack(rows, dim=0)


def masked_stats(values, denominators):
    out = {}
    for k, v in values.items():
        d = denominators.get(k)
        d = torch.ones_like(v, dtype=torch.bool) if d is None else d.bool()
        cnt = float(d.sum())
        s = float(torch.where(d, v.double(), 0.0).sum())
        mn = float(torch.where(d, v, float("inf")).min()) if v.numel() else float("inf")
        mx = float(torch.where(d, v, -float("inf")).max()) if v.numel() else -float("inf")
        out[k] = dict(sum=s, count=cnt, avg=None if cnt == 0 else s / cnt,
                      min=None if math.isinf(mn) else mn, max=None if math.isinf(mx) else mx)
    return out
