"""Packing, padding and un-padding of sequence batches on the GPU.

Host-side mirror of ``pack_tensor_dict``, ``pad_packed_tensor_dict`` and ``unpad_logits``
(areal/utils/data.py:492-541, 818-978, 1046-1074).  The reference moves one sequence at a time from a Python loop;
here every tensor moves in one launch of the segmented row copy.  As in the reference, sizing the outputs reads the
total length back from the device once per call.
"""
from __future__ import annotations

import math
from typing import Any

import torch

from . import _native as N
from .functional import _ptr, _require_gpu, _stream

N_TOKENS_PER_PAGE = 256  # areal/utils/data.py:815


def segment_copy(src: torch.Tensor, dst: torch.Tensor, src_starts: torch.Tensor, dst_starts: torch.Tensor,
                 seg_cu: torch.Tensor, total_rows: int) -> torch.Tensor:
    """``dst[dst_starts[i] + o] = src[src_starts[i] + o]`` for every row ``o`` of every segment ``i``.

    ``src`` and ``dst`` are contiguous with the same trailing shape and dtype; a row is one index of dim 0.
    ``seg_cu`` is the int32 ``[B + 1]`` cumulative row count of the segments, ``total_rows = seg_cu[-1]``.
    """
    _require_gpu(src, "src")
    _require_gpu(dst, "dst")
    if src.dtype != dst.dtype or src.shape[1:] != dst.shape[1:]:
        raise ValueError("src and dst must agree in dtype and trailing shape")
    if not (src.is_contiguous() and dst.is_contiguous()):
        raise ValueError("src and dst must be contiguous")
    B = seg_cu.numel() - 1
    if B <= 0 or total_rows <= 0:
        return dst
    dev = src.device
    row_bytes = src.element_size() * int(math.prod(src.shape[1:]))
    ss = src_starts.to(device=dev, dtype=torch.int64).contiguous()
    ds = dst_starts.to(device=dev, dtype=torch.int64).contiguous()
    cu = seg_cu.to(device=dev, dtype=torch.int32).contiguous()
    with torch.cuda.device(dev):
        N.check(N.load().aa_segment_copy(_ptr(src), _ptr(dst), row_bytes, _ptr(ss), _ptr(ds), _ptr(cu), B,
                                         int(total_rows), _stream(dev)), "aa_segment_copy")
    return dst


def pack_tensor_dict(data: dict[str, Any]) -> dict[str, Any]:
    """``[B, S, ...]`` tensors to ``[total_length, ...]``; data.py:492-541 (same keys: ``cu_seqlens``, ``max_seqlen``)."""
    assert "attention_mask" in data, "Input data must contain 'attention_mask' key."
    attention_mask = data["attention_mask"]
    assert attention_mask.ndim == 2, "Attention mask must be a 2D tensor."
    _require_gpu(attention_mask, "attention_mask")
    bs, seq_len = attention_mask.shape
    lens = attention_mask.sum(dim=1, dtype=torch.int32)
    cu_seqlens = torch.nn.functional.pad(torch.cumsum(lens, dim=0, dtype=torch.int32), (1, 0), value=0)
    max_seqlen, total_length = (int(v) for v in torch.stack([lens.max(), cu_seqlens[-1]]).tolist())
    src_starts = torch.arange(bs, device=attention_mask.device, dtype=torch.int64) * seq_len
    dst_starts = cu_seqlens[:-1].to(torch.int64)
    packed = {}
    for key, value in data.items():
        if key == "attention_mask":
            packed["cu_seqlens"] = cu_seqlens
            packed["max_seqlen"] = max_seqlen
            continue
        if torch.is_tensor(value) and value.ndim >= 2 and value.shape[0] == bs and value.shape[1] == seq_len:
            v = value.contiguous()
            out = torch.empty((total_length, *v.shape[2:]), dtype=v.dtype, device=v.device)
            segment_copy(v.reshape(bs * seq_len, *v.shape[2:]), out, src_starts, dst_starts, cu_seqlens, total_length)
            packed[key] = out
        else:
            packed[key] = value
    return packed


def _segment_ids(cu: torch.Tensor, total: int) -> torch.Tensor:
    lens = (cu[1:] - cu[:-1]).to(torch.int64)
    return torch.repeat_interleave(torch.arange(lens.numel(), device=cu.device), lens, output_size=total)


def pad_packed_tensor_dict(data: dict[str, Any], pad_to_length: int, pad_value: float = 0.0,
                           seq_align_to: int | None = None) -> tuple[dict[str, Any], int, torch.Tensor, int | None]:
    """Pad a packed dict to ``pad_to_length`` with one trailing pad sequence, optionally aligning every sequence to a
    multiple of ``seq_align_to`` first; data.py:818-978 (same return tuple)."""
    assert "cu_seqlens" in data, "Input data must contain 'cu_seqlens' key."
    assert "max_seqlen" in data, "Input data must contain 'max_seqlen' key."
    cu_seqlens = data["cu_seqlens"]
    _require_gpu(cu_seqlens, "cu_seqlens")
    dev = cu_seqlens.device
    max_seqlen = data["max_seqlen"]
    old_cu_seqlens = cu_seqlens.clone()
    total_length = int(cu_seqlens[-1].item())
    align_to_length = None
    if seq_align_to is not None:
        input_lens = cu_seqlens[1:] - cu_seqlens[:-1]
        batch_size = input_lens.shape[0]
        input_lens_padded = input_lens + (-input_lens) % seq_align_to
        cu_padded = torch.zeros(batch_size + 1, dtype=torch.int32, device=dev)
        cu_padded[1:] = torch.cumsum(input_lens_padded, dim=0)
        max_padded, total_padded = (int(v) for v in torch.stack([input_lens_padded.max(), cu_padded[-1]]).tolist())
        src_starts, dst_starts = cu_seqlens[:-1].to(torch.int64), cu_padded[:-1].to(torch.int64)
        seg = _segment_ids(cu_padded, total_padded)
        pos_in_seg = torch.arange(total_padded, device=dev) - cu_padded[:-1].to(torch.int64)[seg]
        aligned = {}
        for key, value in data.items():
            if key == "cu_seqlens":
                aligned[key] = cu_padded
            elif key == "max_seqlen":
                aligned[key] = max_padded
            elif key == "position_ids":
                if value.ndim == 2 and value.shape[1] == 3:
                    new_value = torch.zeros((total_padded, 3), dtype=value.dtype, device=value.device)
                    segment_copy(value.contiguous(), new_value, src_starts, dst_starts, cu_seqlens, total_length)
                    pad_pos = pos_in_seg - input_lens.to(torch.int64)[seg]
                    new_value = torch.where((pad_pos >= 0).unsqueeze(1), pad_pos.unsqueeze(1).to(value.dtype), new_value)
                else:
                    new_value = pos_in_seg.to(value.dtype)
                aligned[key] = new_value
            elif torch.is_tensor(value) and value.numel() == total_length:
                new_value = torch.full((total_padded,), fill_value=pad_value, dtype=value.dtype, device=value.device)
                segment_copy(value.contiguous().reshape(-1), new_value, src_starts, dst_starts, cu_seqlens, total_length)
                aligned[key] = new_value
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
    padded = {}
    for key, value in data.items():
        if key == "cu_seqlens":
            padded[key] = torch.nn.functional.pad(cu_seqlens, (0, 1), value=pad_to_length)
        elif key == "max_seqlen":
            padded[key] = max(max_seqlen, pad_length)
        elif key == "position_ids":
            pad = torch.arange(pad_length, dtype=torch.long, device=value.device)
            if value.ndim == 2 and value.shape[1] == 3:
                pad = pad.unsqueeze(1).expand(-1, 3)
            padded[key] = torch.cat([value, pad])
        elif torch.is_tensor(value) and value.numel() == total_length:
            padded[key] = torch.nn.functional.pad(value, (0, pad_length), value=pad_value)
        else:
            padded[key] = value
    return padded, pad_length, old_cu_seqlens, align_to_length


def unpad_logits(logits: torch.Tensor, padding_length: int, cu_seqlens: torch.Tensor | None = None,
                 old_cu_seqlens: torch.Tensor | None = None) -> torch.Tensor:
    """Drop the trailing pad sequence, then the per-sequence alignment padding; data.py:1046-1074."""
    if padding_length > 0:
        logits = logits[:-padding_length]
    if old_cu_seqlens is None:
        return logits
    _require_gpu(logits, "logits")
    total = int(old_cu_seqlens[-1].item())
    out = torch.empty((total, *logits.shape[1:]), dtype=logits.dtype, device=logits.device)
    B = old_cu_seqlens.shape[0] - 1
    segment_copy(logits.contiguous(), out, cu_seqlens[:B].to(torch.int64), old_cu_seqlens[:B].to(torch.int64),
                 old_cu_seqlens, total)
    return out
