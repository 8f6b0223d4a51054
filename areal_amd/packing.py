"""Packing and padding of token batches on MI355X.

Same signatures and return structures as the reference's ``areal/utils/data.py``
``pack_tensor_dict`` (:496-545) and ``pad_packed_tensor_dict`` (:822-982), and the unpack ->
reorder -> pad-and-stack composition of ``reorder_and_pad_outputs``
(``areal/engine/core/train_engine.py:110-144``).  Every per-sequence Python loop of the
reference (one ``.item()`` or slice assignment per sequence and tensor) is one gather kernel by
``cu_seqlens`` here; a call performs one device-to-host copy (the total length and the
longest sequence, which the reference returns as Python ints as well).
"""

from __future__ import annotations

import ctypes
import math
from typing import Any

import torch

from areal_amd import _lib

N_TOKENS_PER_PAGE = 256  # data.py:819
_PACK_MAX_TENSORS = 8  # tensors per areal_pack_padded_multi launch


def _elem_bytes(t: torch.Tensor, lead_dims: int) -> int:
    return int(math.prod(t.shape[lead_dims:])) * t.element_size()


def _fill_bytes(dtype: torch.dtype, value: float):
    """Bit pattern of ``value`` in ``dtype`` as a ctypes buffer (<= 16 bytes)."""
    raw = torch.tensor([value], dtype=dtype).view(torch.uint8).numpy().tobytes()
    return ctypes.create_string_buffer(raw, len(raw)), len(raw)


def pack_tensor_dict(data: dict[str, Any]) -> dict[str, Any]:
    """Pack a dict of ``[B, S, ...]`` tensors into ``[total_length, ...]``; ``attention_mask`` is
    replaced by ``cu_seqlens`` (int32 ``[B+1]``) and ``max_seqlen`` (int)."""
    assert "attention_mask" in data, "Input data must contain 'attention_mask' key."
    attention_mask = data["attention_mask"]
    assert attention_mask.ndim == 2, "Attention mask must be a 2D tensor."
    lib = _lib.load()
    dev = _lib.require_gpu(attention_mask)
    bs, seq_len = attention_mask.shape
    mask_u8 = (attention_mask != 0).contiguous().view(torch.uint8)
    lens = torch.empty(bs, dtype=torch.int32, device=dev)
    cu_seqlens = torch.empty(bs + 1, dtype=torch.int32, device=dev)
    max_len = torch.empty(1, dtype=torch.int32, device=dev)
    rc = lib.areal_seqlens_from_mask(
        _lib.ptr(mask_u8), bs, seq_len, _lib.ptr(lens), _lib.ptr(cu_seqlens), _lib.ptr(max_len),
        _lib.stream_ptr(dev),
    )
    _lib.check(rc, "areal_seqlens_from_mask")
    total_length, max_seqlen = torch.stack([cu_seqlens[-1], max_len[0]]).tolist()  # the one host copy
    packed_data: dict[str, Any] = {}
    moved = []  # (contiguous source, packed destination) of the tensors that are packed
    for key, value in data.items():
        if key == "attention_mask":
            packed_data["cu_seqlens"] = cu_seqlens
            packed_data["max_seqlen"] = max_seqlen
            continue
        if torch.is_tensor(value) and value.ndim >= 2 and value.shape[0] == bs and value.shape[1] == seq_len:
            _lib.require_gpu(value)
            src = value.contiguous()
            packed = torch.empty((total_length, *value.shape[2:]), dtype=value.dtype, device=value.device)
            moved.append((src, packed))
            packed_data[key] = packed
        else:
            packed_data[key] = value
    # eight tensors per launch
    for i in range(0, len(moved), _PACK_MAX_TENSORS):
        part = moved[i : i + _PACK_MAX_TENSORS]
        n = len(part)
        srcs = (ctypes.c_void_p * n)(*[s.data_ptr() for s, _ in part])
        dsts = (ctypes.c_void_p * n)(*[d.data_ptr() for _, d in part])
        sizes = (ctypes.c_int64 * n)(*[_elem_bytes(s, 2) for s, _ in part])
        rc = lib.areal_pack_padded_multi(
            srcs, dsts, sizes, n, _lib.ptr(cu_seqlens), bs, seq_len, total_length, _lib.stream_ptr(dev),
        )
        _lib.check(rc, "areal_pack_padded_multi")
    return packed_data


def _realign(lib, dev, value, cu_old, n_old, cu_new, n_new, total_new, pad_value, position_ids, whole_arange):
    out_shape = (total_new, *value.shape[1:])
    out = torch.empty(out_shape, dtype=value.dtype, device=value.device)
    src = value.contiguous()
    if position_ids:
        if value.dtype != torch.int64:
            src = src.to(torch.int64)
            out = torch.empty(out_shape, dtype=torch.int64, device=value.device)
        fill, nfill = None, 0
    else:
        fill, nfill = _fill_bytes(value.dtype, pad_value)
    rc = lib.areal_realign_packed(
        _lib.ptr(None if whole_arange else src), _lib.ptr(out), _lib.ptr(cu_old), n_old,
        _lib.ptr(cu_new), n_new, _elem_bytes(src, 1), fill, nfill, int(position_ids), total_new,
        _lib.stream_ptr(dev),
    )
    _lib.check(rc, "areal_realign_packed")
    return out.to(value.dtype) if out.dtype != value.dtype else out


def pad_packed_tensor_dict(
    data: dict[str, Any],
    pad_to_length: int,
    pad_value: float = 0.0,
    seq_align_to: int | None = None,
) -> tuple[dict[str, Any], int, torch.Tensor, int | None]:
    """Pad a packed dict of tensors to ``pad_to_length`` by appending one pad sequence, after
    optionally aligning every sequence to a multiple of ``seq_align_to``.  Returns
    ``(padded_data, pad_length, old_cu_seqlens, align_to_length)``."""
    assert "cu_seqlens" in data, "Input data must contain 'cu_seqlens' key."
    assert "max_seqlen" in data, "Input data must contain 'max_seqlen' key."
    lib = _lib.load()
    cu_seqlens = data["cu_seqlens"]
    dev = _lib.require_gpu(cu_seqlens)
    cu_seqlens = cu_seqlens.to(torch.int32).contiguous()
    max_seqlen = data["max_seqlen"]
    old_cu_seqlens = cu_seqlens.clone()
    n_seqs = cu_seqlens.numel() - 1
    align_to_length = None
    if seq_align_to is not None:
        input_lens = cu_seqlens[1:] - cu_seqlens[:-1]
        lens_padded = input_lens + (-input_lens) % seq_align_to
        cu_padded = torch.zeros(n_seqs + 1, dtype=torch.int32, device=dev)
        cu_padded[1:] = torch.cumsum(lens_padded, dim=0)
        total_length, total_padded, max_padded = torch.stack(
            [cu_seqlens[-1], cu_padded[-1], lens_padded.max()]
        ).tolist()
    else:
        total_length = int(cu_seqlens[-1].item())

    def is_token_tensor(key, value, total):
        if key == "position_ids":
            return torch.is_tensor(value)
        return torch.is_tensor(value) and value.numel() == total

    if seq_align_to is not None:
        aligned: dict[str, Any] = {}
        for key, value in data.items():
            if key == "cu_seqlens":
                aligned[key] = cu_padded
            elif key == "max_seqlen":
                aligned[key] = max_padded
            elif key == "position_ids":
                three = value.ndim == 2 and value.shape[1] == 3
                aligned[key] = _realign(lib, dev, value, cu_seqlens, n_seqs, cu_padded, n_seqs, total_padded,
                                        0.0, True, whole_arange=not three)
            elif is_token_tensor(key, value, total_length):
                aligned[key] = _realign(lib, dev, value.reshape(total_length), cu_seqlens, n_seqs, cu_padded,
                                        n_seqs, total_padded, pad_value, False, False)
            else:
                aligned[key] = value
        data = aligned
        align_to_length = total_padded
        lcm = math.lcm(seq_align_to, N_TOKENS_PER_PAGE)
        pad_to_length = (pad_to_length + lcm - 1) // lcm * lcm
        cu_seqlens, max_seqlen, total_length = cu_padded, max_padded, total_padded
        if pad_to_length < total_length:
            pad_to_length = (total_length + lcm - 1) // lcm * lcm

    pad_length = pad_to_length - total_length
    if pad_length < 0:
        raise ValueError(f"pad_to_length {pad_to_length} is smaller than total length {total_length}.")
    if pad_length == 0:
        return data, pad_length, old_cu_seqlens, align_to_length
    new_cu = torch.nn.functional.pad(cu_seqlens, (0, 1), value=pad_to_length)
    padded: dict[str, Any] = {}
    for key, value in data.items():
        if key == "cu_seqlens":
            padded[key] = new_cu
        elif key == "max_seqlen":
            padded[key] = max(max_seqlen, pad_length)
        elif key == "position_ids":
            padded[key] = _realign(lib, dev, value, cu_seqlens, n_seqs, new_cu, n_seqs + 1, pad_to_length,
                                   0.0, True, False)
        elif is_token_tensor(key, value, total_length):
            padded[key] = _realign(lib, dev, value.reshape(total_length), cu_seqlens, n_seqs, new_cu,
                                   n_seqs + 1, pad_to_length, pad_value, False, False)
        else:
            padded[key] = value
    return padded, pad_length, old_cu_seqlens, align_to_length


def unpack_reorder_pad(
    packed: torch.Tensor,
    seqlens: list[int],
    backward_indices: list[int] | None = None,
) -> torch.Tensor:
    """``pad_and_stack_tensors_along_first_dim(reorder_list(unpack_sequence(packed, lens=seqlens),
    backward_indices))`` in one gather: row ``r`` of the ``[n, max(seqlens), ...]`` result holds
    packed sequence ``backward_indices[r]``, zero padded."""
    lib = _lib.load()
    dev = _lib.require_gpu(packed)
    n = len(seqlens)
    if backward_indices is not None:
        assert len(set(backward_indices)) == n
    if sum(seqlens) != packed.shape[0]:
        raise ValueError(f"seqlens sum to {sum(seqlens)}, the packed tensor has {packed.shape[0]} rows")
    cu = torch.tensor([0] + list(torch.tensor(seqlens, dtype=torch.int64).cumsum(0)), dtype=torch.int32).to(dev)
    row_seq = torch.tensor(backward_indices, dtype=torch.int32).to(dev) if backward_indices is not None else None
    max_len = max(seqlens) if n > 0 else 0
    src = packed.contiguous()
    out = torch.empty((n, max_len, *packed.shape[1:]), dtype=packed.dtype, device=dev)
    rc = lib.areal_unpack_to_padded(
        _lib.ptr(src), _lib.ptr(out), _lib.ptr(cu), _lib.ptr(row_seq), n, max_len,
        _elem_bytes(src, 1), None, 0, _lib.stream_ptr(dev),
    )
    _lib.check(rc, "areal_unpack_to_padded")
    return out


def reorder_and_pad_outputs(outputs, output_seqlens, mb_list, aggregate_fn=torch.cat) -> torch.Tensor:
    """Aggregate micro-batch outputs, then unpack / reorder / pad in one kernel
    (``train_engine.py:110-144``).  ``mb_list`` needs ``forward_indices`` and ``backward_indices``."""
    res = aggregate_fn(outputs)
    seqlens = [output_seqlens[i] for i in mb_list.forward_indices]
    return unpack_reorder_pad(res, seqlens, list(mb_list.backward_indices))
