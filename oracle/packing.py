"""CPU oracle of the packing helpers.  TEST INFRASTRUCTURE ONLY.

Restates the per-sequence loops of ``pack_tensor_dict``, ``pad_packed_tensor_dict`` and ``unpad_logits``
(areal/utils/data.py:492-541, 818-978, 1046-1074).  How each is pinned is listed in ``oracle/PINNING.md``.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F

N_TOKENS_PER_PAGE = 256  # data.py:815


def pack_tensor_dict(data):
    """data.py:492-541."""
    attention_mask = data["attention_mask"]
    bs, seq_len = attention_mask.shape
    lens = attention_mask.sum(dim=1, dtype=torch.int32)
    max_seqlen = lens.max().item()
    cu_seqlens = F.pad(torch.cumsum(lens, dim=0, dtype=torch.int32), (1, 0), value=0)
    total_length = int(cu_seqlens[-1].item())
    packed = {}
    for key, value in data.items():
        if key == "attention_mask":
            packed["cu_seqlens"] = cu_seqlens
            packed["max_seqlen"] = max_seqlen
            continue
        if torch.is_tensor(value) and value.ndim >= 2 and value.shape[0] == bs and value.shape[1] == seq_len:
            out = torch.empty((total_length, *value.shape[2:]), dtype=value.dtype)
            for i in range(bs):                                        # :533-536
                start, end = cu_seqlens[i].item(), cu_seqlens[i + 1].item()
                out[start:end] = value[i][: end - start]
            packed[key] = out
        else:
            packed[key] = value
    return packed


def pad_packed_tensor_dict(data, pad_to_length, pad_value=0.0, seq_align_to=None):
    """data.py:818-978."""
    cu_seqlens = data["cu_seqlens"]
    max_seqlen = data["max_seqlen"]
    old_cu_seqlens = cu_seqlens.clone()
    total_length = data["cu_seqlens"][-1].item()
    align_to_length = None
    if seq_align_to is not None:
        input_lens = cu_seqlens[1:] - cu_seqlens[:-1]
        batch_size = input_lens.shape[0]
        pad_size = (-input_lens) % seq_align_to                        # :852
        input_lens_padded = input_lens + pad_size
        cu_padded = torch.zeros(batch_size + 1, dtype=torch.int32)
        cu_padded[1:] = torch.cumsum(input_lens_padded, dim=0)
        max_padded = input_lens_padded.max().item()
        padded_shape = (input_lens_padded.sum().item(),)
        out = {}
        for key, value in data.items():
            if key == "cu_seqlens":
                out[key] = cu_padded
            elif key == "max_seqlen":
                out[key] = max_padded
            elif key == "position_ids":
                if len(value.shape) == 2 and value.shape[1] == 3:      # :866-887
                    nv = torch.zeros((padded_shape[0], 3), dtype=value.dtype)
                    for i in range(batch_size):
                        ns, ne = cu_padded[i], cu_padded[i + 1]
                        os_, oe = cu_seqlens[i], cu_seqlens[i + 1]
                        length = oe - os_
                        pad_length = ne - ns - length
                        nv[ns : ns + length] = value[os_:oe]
                        nv[ns + length : ne] = torch.arange(pad_length, dtype=torch.long).unsqueeze(1).expand(-1, 3)
                else:                                                  # :888-897
                    nv = torch.zeros(padded_shape, dtype=value.dtype)
                    for i in range(batch_size):
                        ns, ne = cu_padded[i], cu_padded[i + 1]
                        nv[ns:ne] = torch.arange(ne - ns, dtype=value.dtype)
                out[key] = nv
            elif torch.is_tensor(value) and value.numel() == total_length:   # :899-912
                nv = torch.full(padded_shape, fill_value=pad_value, dtype=value.dtype)
                for i in range(batch_size):
                    ns = cu_padded[i]
                    start, end = cu_seqlens[i], cu_seqlens[i + 1]
                    nv[ns : ns + (end - start)] = value[start:end]
                out[key] = nv
            else:
                out[key] = value
        data = out
        align_to_length = cu_padded[-1].item()
        lcm = np.lcm(seq_align_to, N_TOKENS_PER_PAGE).item()           # :919-920
        pad_to_length = (pad_to_length + lcm - 1) // lcm * lcm
        cu_seqlens = data["cu_seqlens"]
        max_seqlen = data["max_seqlen"]
        total_length = data["cu_seqlens"][-1].item()
        if pad_to_length < total_length:                               # :925-929
            pad_to_length = (total_length + lcm - 1) // lcm * lcm
    pad_length = pad_to_length - total_length                          # :932
    if pad_length < 0:
        raise ValueError(f"pad_to_length {pad_to_length} is smaller than total length {total_length}.")
    elif pad_length == 0:
        return data, pad_length, old_cu_seqlens, align_to_length
    new_cu = F.pad(cu_seqlens, (0, 1), value=pad_to_length)            # :944
    new_max = max(max_seqlen, pad_length)
    padded = {}
    for key, value in data.items():
        if key == "cu_seqlens":
            padded[key] = new_cu
        elif key == "max_seqlen":
            padded[key] = new_max
        elif key == "position_ids":
            pad = torch.arange(pad_length, dtype=torch.long)
            if len(value.shape) == 2 and value.shape[1] == 3:
                pad = pad.unsqueeze(1).expand(-1, 3)
            padded[key] = torch.cat([value, pad])
        elif torch.is_tensor(value) and value.numel() == total_length:
            padded[key] = F.pad(value, (0, pad_length), value=pad_value)
        else:
            padded[key] = value
    return padded, pad_length, old_cu_seqlens, align_to_length


def unpad_logits(logits, padding_length, cu_seqlens=None, old_cu_seqlens=None):
    """data.py:1046-1074."""
    if padding_length > 0:
        logits = logits[:-padding_length]
    if old_cu_seqlens is not None:
        new_logits = torch.empty((old_cu_seqlens[-1].item(), *logits.shape[1:]), dtype=logits.dtype)
        for i in range(old_cu_seqlens.shape[0] - 1):
            old_start, old_end = old_cu_seqlens[i].item(), old_cu_seqlens[i + 1].item()
            start = cu_seqlens[i].item()
            new_logits[old_start:old_end] = logits[start : start + old_end - old_start]
        return new_logits
    return logits
