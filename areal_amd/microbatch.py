"""From a padded batch to the packed, padded micro-batches the engine runs: balanced allocation of sequences to
micro-batches, the split, packing and page padding.

Host-side mirror of ``areal/utils/seqpack.py`` (``ffd_allocate`` :196-267, ``kk_allocate`` :272-381, 446-537),
``MicroBatchSpec`` (areal/api/cli_args.py:99-159) and of ``areal/utils/data.py``: ``allocate_balanced_mbs`` :448-472,
``MicroBatchList`` :586-690, ``split_padded_tensor_dict_into_mb_list`` :696-812, ``pad_mb_list`` :981-1043,
``amend_position_ids`` :1111-1123.  The allocation is integer work on a few hundred lengths and stays on the host;
the rows move on the GPU (one gather per tensor instead of one slice per sequence).
"""
from __future__ import annotations

import heapq
import math
from dataclasses import dataclass
from typing import Any, Iterator, NamedTuple

import numpy as np
import torch

from .packing import pack_tensor_dict, pad_packed_tensor_dict

PACKING_ALGORITHM_FFD = "ffd"
PACKING_ALGORITHM_KK = "kk"
PACKING_ALGORITHMS = {PACKING_ALGORITHM_FFD, PACKING_ALGORITHM_KK}
DEFAULT_MAX_TOKENS_PER_MB = int(1e12)
N_TOKENS_PER_PAGE = 256


@dataclass
class MicroBatchSpec:
    """How a batch is cut into micro-batches; cli_args.py:99-159."""

    n_mbs: int | None = 1
    granularity: int = 1
    max_tokens_per_mb: int | None = None
    n_mbs_divisor: int = 1
    packing_algorithm: str = PACKING_ALGORITHM_FFD

    def __post_init__(self):
        if self.packing_algorithm not in PACKING_ALGORITHMS:
            raise ValueError(
                f"packing_algorithm must be one of {sorted(PACKING_ALGORITHMS)}, got '{self.packing_algorithm}'"
            )

    @classmethod
    def new(cls, mb_spec: "MicroBatchSpec", **kwargs):
        fields = dict(n_mbs=mb_spec.n_mbs, granularity=mb_spec.granularity, max_tokens_per_mb=mb_spec.max_tokens_per_mb,
                      n_mbs_divisor=mb_spec.n_mbs_divisor,
                      packing_algorithm=getattr(mb_spec, "packing_algorithm", PACKING_ALGORITHM_FFD))
        fields.update(kwargs)
        return cls(**fields)


# ----------------------------------------------------------------------------------------------------------------
# first fit decreasing
# ----------------------------------------------------------------------------------------------------------------
def _ffd_once(values: np.ndarray, capacity: int, min_groups: int) -> list[list[int]]:
    """One greedy pass (seqpack.py:196-231).  Values are taken in decreasing order; a value opens a new group while
    fewer than ``min_groups`` exist or when it does not fit into the lightest group; otherwise, among the groups it
    fits into, it joins the one with the fewest members (the lightest of those, then the oldest, on ties)."""
    order = np.argsort(-values)
    sums: list[float] = []
    members: list[list[int]] = []
    for idx in order:
        v = float(values[idx])
        if len(sums) < min_groups or min(sums) + v > capacity:
            sums.append(v)
            members.append([idx])
            continue
        room = capacity - values[idx]
        fits = [g for g in range(len(sums)) if sums[g] <= room]
        g = min(fits, key=lambda q: (len(members[q]), sums[q], q))
        sums[g] += v
        members[g].append(idx)
    return members


def ffd_allocate(values: list[int], capacity: int, min_groups: int, n_groups_divisor: int = 1) -> list[list[int]]:
    """Groups of indices into ``values`` whose sums stay within ``capacity``, at least ``min_groups`` of them and a
    multiple of ``n_groups_divisor``; seqpack.py:234-267."""
    if min_groups is None or min_groups < n_groups_divisor:
        min_groups = n_groups_divisor
    if any(v > capacity for v in values):
        raise RuntimeError(f"Values {values} is larger than capacity {capacity}")
    if len(values) < min_groups:
        raise RuntimeError(f"Number of values {len(values)} is smaller than min_groups {min_groups}")
    arr = np.array(values)
    while True:
        groups = _ffd_once(arr, capacity, min_groups)
        min_groups += n_groups_divisor - min_groups % n_groups_divisor   # the next multiple above, for a retry
        if len(groups) % n_groups_divisor == 0:
            return groups
        if len(values) < min_groups:
            raise RuntimeError(
                f"Cannot allocate values {values} that satisfies capacity {capacity}, "
                f"min_groups {min_groups} and n_groups_divisor {n_groups_divisor}."
            )


# ----------------------------------------------------------------------------------------------------------------
# Karmarkar-Karp largest differencing
# ----------------------------------------------------------------------------------------------------------------
# A bin is the tuple (sum, number of items, [(index, value), ...]); Python's tuple order on it is the order the
# reference gives its sets (sum, then size, then the item lists; seqpack.py:290-295).
def _bin_merge(a, b):
    return (a[0] + b[0], a[1] + b[1], a[2] + b[2])


class _Partial:
    """k bins, heaviest first.  In the heap the partial solution with the largest spread comes out first; on equal
    spread the one whose heaviest bin is larger (seqpack.py:330-334)."""

    __slots__ = ("bins",)

    def __init__(self, bins):
        self.bins = sorted(bins, reverse=True)

    @property
    def spread(self) -> int:
        return self.bins[0][0] - self.bins[-1][0]

    def __lt__(self, other: "_Partial") -> bool:
        if self.spread != other.spread:
            return self.spread > other.spread
        return other.bins[0] < self.bins[0]

    def absorb(self, other: "_Partial") -> None:
        """Heaviest bin with the other's lightest and so on (seqpack.py:319-324)."""
        k = len(self.bins)
        self.bins = sorted((_bin_merge(self.bins[i], other.bins[k - 1 - i]) for i in range(k)), reverse=True)


def _kk_partition(values: list[int], k: int, equal_size: bool = False) -> list[list[int]]:
    """k groups of indices by repeatedly merging the two partial solutions of largest spread; seqpack.py:337-381."""
    ranked = sorted((val, idx) for idx, val in enumerate(values))
    empty = (0, 0, [])
    heap: list[_Partial] = []
    if equal_size:
        assert len(values) % k == 0, f"{len(values)} % {k} != 0"
        for off in range(0, len(ranked), k):
            heapq.heappush(heap, _Partial([(val, 1, [(idx, val)]) for val, idx in ranked[off:off + k]]))
    else:
        for val, idx in ranked:
            heapq.heappush(heap, _Partial([(val, 1, [(idx, val)])] + [empty] * (k - 1)))
    while len(heap) > 1:
        first = heapq.heappop(heap)
        second = heapq.heappop(heap)
        first.absorb(second)
        heapq.heappush(heap, first)
    return [[idx for idx, _ in b[2]] for b in heap[0].bins]


def kk_allocate(values: list[int], capacity: int, min_groups: int, n_groups_divisor: int = 1,
                equal_size: bool = False) -> list[list[int]]:
    """Same contract as ``ffd_allocate``; the number of groups is ``max(min_groups, ceil(total / capacity))`` rounded
    up to the divisor and capped by the number of values, and a result that breaks the capacity falls back to
    ``ffd_allocate``; seqpack.py:446-537."""
    if min_groups is None or min_groups < n_groups_divisor:
        min_groups = n_groups_divisor
    if any(v > capacity for v in values):
        raise RuntimeError(
            f"Some values exceed capacity {capacity}. Cannot pack a single item that is larger than the bin."
        )
    if len(values) < min_groups:
        raise RuntimeError(f"Number of values {len(values)} is smaller than min_groups {min_groups}")
    k = max(min_groups, math.ceil(sum(values) / capacity))
    if n_groups_divisor > 1:
        k = math.ceil(k / n_groups_divisor) * n_groups_divisor
    k = min(k, len(values))
    if equal_size and len(values) % k != 0:
        raise RuntimeError(f"equal_size=True requires len(values) ({len(values)}) to be divisible by k ({k})")
    groups = _kk_partition(values, k, equal_size=equal_size)
    if any(sum(values[i] for i in g) > capacity for g in groups):
        return ffd_allocate(values, capacity, min_groups, n_groups_divisor)
    return groups


def get_allocate_fn(algorithm: str = PACKING_ALGORITHM_FFD):
    """seqpack.py:167-187."""
    if algorithm == PACKING_ALGORITHM_FFD:
        return ffd_allocate
    if algorithm == PACKING_ALGORITHM_KK:
        return kk_allocate
    raise ValueError(f"Unknown packing algorithm '{algorithm}'. Supported algorithms: {sorted(PACKING_ALGORITHMS)}")


def allocate_balanced_mbs(mb_spec: MicroBatchSpec, lens: list[int]) -> list[list[int]]:
    """Sorted groups of sorted indices, one group per micro-batch; data.py:448-472."""
    assert mb_spec.max_tokens_per_mb is not None
    allocate = get_allocate_fn(getattr(mb_spec, "packing_algorithm", PACKING_ALGORITHM_FFD))
    groups = allocate(lens, mb_spec.max_tokens_per_mb, min_groups=mb_spec.n_mbs, n_groups_divisor=mb_spec.n_mbs_divisor)
    return sorted(sorted(g) for g in groups)


# ----------------------------------------------------------------------------------------------------------------
# the list of micro-batches
# ----------------------------------------------------------------------------------------------------------------
class MicroBatchItem(NamedTuple):
    """What iterating a ``MicroBatchList`` yields; data.py:586-602."""

    orig_mb: dict[str, Any]
    padded_mb: dict[str, Any]
    padding_length: int
    old_cu_seqlens: torch.Tensor | None
    padded_to_length: int | None = None


@dataclass
class MicroBatchList:
    """data.py:605-690."""

    data: dict[str, Any]
    mb_spec: MicroBatchSpec
    mbs: list[dict[str, Any]]
    group_lens: list[int]
    forward_indices: list[int] | None = None
    backward_indices: list[int] | None = None
    padded_mbs: list[dict[str, Any]] | None = None
    _max_seqlen: int | None = None
    padding_lengths: list[int] | None = None
    padded_to_lengths: list[int] | None = None
    align_to_lengths: list[int] | None = None
    old_cu_seqlens_list: list[torch.Tensor] | None = None

    @property
    def max_seqlen(self) -> int:
        if self.padded_mbs is None:
            raise ValueError("padded_mbs is None. Call pad_mb_list first.")
        if self._max_seqlen is None:
            assert all("cu_seqlens" in m for m in self.padded_mbs), "cu_seqlens not found in some padded micro-batches."
            self._max_seqlen = max(m["cu_seqlens"][-1].item() for m in self.padded_mbs)
        return self._max_seqlen

    def __len__(self) -> int:
        return len(self.mbs)

    def __iter__(self) -> Iterator[MicroBatchItem]:
        if self.padded_mbs is None:
            raise ValueError("padded_mbs is None. Call pad_mb_list first.")
        for i in range(len(self.mbs)):
            yield MicroBatchItem(
                orig_mb=self.mbs[i],
                padded_mb=self.padded_mbs[i],
                padding_length=self.padding_lengths[i],
                old_cu_seqlens=self.old_cu_seqlens_list[i] if self.old_cu_seqlens_list else None,
                padded_to_length=self.padded_to_lengths[i] if self.padded_to_lengths else None,
            )

    def to(self, *args, **kwargs) -> "MicroBatchList":
        """A copy with every tensor moved / cast; data.py:661-690."""
        return MicroBatchList(
            data=tensor_container_to(self.data, *args, **kwargs),
            mb_spec=self.mb_spec,
            mbs=[tensor_container_to(mb, *args, **kwargs) for mb in self.mbs],
            forward_indices=self.forward_indices,
            backward_indices=self.backward_indices,
            group_lens=self.group_lens,
            padded_mbs=None if self.padded_mbs is None else [tensor_container_to(mb, *args, **kwargs)
                                                             for mb in self.padded_mbs],
            _max_seqlen=self._max_seqlen,
            padding_lengths=self.padding_lengths,
            padded_to_lengths=self.padded_to_lengths,
            old_cu_seqlens_list=None if self.old_cu_seqlens_list is None else [t.to(*args, **kwargs)
                                                                             for t in self.old_cu_seqlens_list],
            align_to_lengths=self.align_to_lengths,
        )


def tensor_container_to(d: Any, *args, **kwargs) -> Any:
    """``.to(...)`` applied to every tensor of a nested dict / list / tuple; data.py:558-583."""
    if torch.is_tensor(d):
        return d.to(*args, **kwargs)
    if isinstance(d, list):
        return [tensor_container_to(v, *args, **kwargs) for v in d]
    if isinstance(d, tuple):
        return tuple(tensor_container_to(v, *args, **kwargs) for v in d)
    if isinstance(d, dict):
        return {k: tensor_container_to(v, *args, **kwargs) for k, v in d.items()}
    return d


def is_multi_modal_key(key: str) -> bool:
    return key.startswith("multi_modal_input")


def amend_position_ids(data: dict) -> dict:
    """``position_ids = arange(seqlen)`` for every row; data.py:1111-1123 (whose ``masked_fill`` is not in place, so
    padding positions keep their index there too)."""
    attn_mask = data["attention_mask"]
    bs, seqlen = attn_mask.shape[:2]
    data["position_ids"] = torch.arange(0, seqlen, dtype=torch.long, device=attn_mask.device).unsqueeze(0).expand(bs, -1)
    return data


def split_padded_tensor_dict_into_mb_list(data: dict[str, Any], mb_spec: MicroBatchSpec, group=None) -> MicroBatchList:
    """Rows of a padded batch distributed over balanced micro-batches; data.py:696-812.

    Tensors with ``bs * max_seqlen`` elements (and ``position_ids``) are split by rows, everything else is shared by
    all micro-batches.  The lengths come to the host once (they size the allocation); each tensor is then reordered
    with one gather and handed out as views, where the reference slices and stacks row by row.  ``group`` must be
    None: agreeing on the number of micro-batches across ranks is not part of this build."""
    if group is not None:
        raise NotImplementedError("synchronising the number of micro-batches across ranks is not built")
    if "attention_mask" not in data:
        raise ValueError("Input data must be padded and contain 'attention_mask' key.")
    if mb_spec.max_tokens_per_mb is None:
        mb_spec = MicroBatchSpec.new(mb_spec, max_tokens_per_mb=DEFAULT_MAX_TOKENS_PER_MB)
    granularity = mb_spec.granularity
    attn = data["attention_mask"]
    bs, max_seqlen = attn.shape[0], attn.shape[1]
    if bs % granularity != 0:
        raise RuntimeError(f"Batch size {bs} cannot divide granularity {granularity}.")
    seq_lens = attn.sum(1).long().cpu().numpy().tolist()
    input_lens = np.asarray(seq_lens, dtype=np.int64).reshape(bs // granularity, granularity).sum(1)

    multimodal_keys = {key for key in data if is_multi_modal_key(key)}
    to_split, not_to_split = {}, {}
    for key, value in data.items():
        if key in multimodal_keys:
            continue
        if key == "position_ids" or (torch.is_tensor(value) and value.numel() == bs * max_seqlen):
            to_split[key] = value
        else:
            not_to_split[key] = value

    groups = allocate_balanced_mbs(mb_spec, input_lens)
    groups = [[i * granularity + j for i in g for j in range(granularity)] for g in groups]
    group_n_seqs = [len(g) for g in groups]
    group_lens = [sum(seq_lens[i] for i in g) for g in groups]
    forward_indices = [i for g in groups for i in g]
    backward_indices = np.zeros(bs, dtype=np.int64)
    backward_indices[forward_indices] = np.arange(bs)

    order = torch.as_tensor(forward_indices, dtype=torch.long, device=attn.device)
    split: dict[str, list] = {}
    for key, value in to_split.items():
        rows = value.index_select(0, order.to(value.device))
        split[key] = list(torch.split(rows, group_n_seqs, dim=0))
    for key in multimodal_keys:
        split[key] = [[data[key][i] for i in g] for g in groups]
    mbs = [{**{key: parts[i] for key, parts in split.items()}, **not_to_split} for i in range(len(groups))]
    return MicroBatchList(data=data, mb_spec=mb_spec, mbs=mbs, forward_indices=forward_indices,
                          backward_indices=backward_indices.tolist(), group_lens=group_lens)


def _align(x: int, to: int) -> int:
    return (x + to - 1) // to * to


def pad_mb_list(mb_list: MicroBatchList, pad_value: float = 0.0, pad_to_maximum: bool = False,
                batch_align_to: int | None = None, seq_align_to: int | None = None) -> MicroBatchList:
    """Pads every (packed) micro-batch to a multiple of 256 tokens (and of ``batch_align_to``), or to
    ``max_tokens_per_mb``, optionally aligning each sequence to ``seq_align_to`` first; data.py:981-1043."""
    if pad_to_maximum and (mb_list.mb_spec.max_tokens_per_mb is None
                           or mb_list.mb_spec.max_tokens_per_mb == DEFAULT_MAX_TOKENS_PER_MB):
        pad_to_maximum = False   # no usable maximum to pad to
    padded, pad_lengths, pad_to_lengths, old_cus, align_tos = [], [], [], [], []
    for mb, length in zip(mb_list.mbs, mb_list.group_lens):
        if pad_to_maximum:
            pad_to_length = mb_list.mb_spec.max_tokens_per_mb
        else:
            pad_to_length = _align(length, N_TOKENS_PER_PAGE)
            if batch_align_to is not None:
                pad_to_length = _align(pad_to_length, batch_align_to)
        padded_mb, pad_len, old_cu, align_to = pad_packed_tensor_dict(mb, pad_to_length, pad_value=pad_value,
                                                                     seq_align_to=seq_align_to)
        padded.append(padded_mb)
        pad_lengths.append(pad_len)
        pad_to_lengths.append(pad_to_length)
        old_cus.append(old_cu)
        align_tos.append(align_to)
    mb_list.padded_mbs = padded
    mb_list.padding_lengths = pad_lengths
    mb_list.padded_to_lengths = pad_to_lengths
    if seq_align_to is not None:
        mb_list.old_cu_seqlens_list = old_cus
        mb_list.align_to_lengths = align_tos
    return mb_list


def unsqueeze_packed_tensor_dict(data: dict[str, Any], total_length: int | None = None) -> dict[str, Any]:
    """A leading batch dimension of 1 on every packed tensor (``position_ids`` and every tensor with as many elements
    as there are tokens), the form the model's forward takes; data.py:1077-1096.  ``total_length`` saves the read-back
    of ``cu_seqlens[-1]`` when the caller knows it."""
    assert "cu_seqlens" in data, "Input data must contain 'cu_seqlens' key."
    assert "max_seqlen" in data, "Input data must contain 'max_seqlen' key."
    if total_length is None:
        total_length = int(data["cu_seqlens"][-1].item())
    out = {}
    for key, value in data.items():
        packed = key == "position_ids" or (key not in ("cu_seqlens", "max_seqlen") and torch.is_tensor(value)
                                           and value.numel() == total_length)
        out[key] = value.unsqueeze(dim=0) if packed else value
    return out


def unsqueeze_mb_list(mb_list: MicroBatchList) -> MicroBatchList:
    """``unsqueeze_packed_tensor_dict`` on every padded micro-batch; data.py:1099-1108.  The padded lengths are
    known on the host, so nothing is read back."""
    if mb_list.padded_mbs is not None:
        lengths = mb_list.padded_to_lengths or [None] * len(mb_list.padded_mbs)
        mb_list.padded_mbs = [unsqueeze_packed_tensor_dict(mb, n) for mb, n in zip(mb_list.padded_mbs, lengths)]
    return mb_list


def packed_mb_list(data: dict[str, Any], mb_spec: MicroBatchSpec, pad_value: float = 0.0, pad_to_maximum: bool = False,
                   batch_align_to: int | None = None, seq_align_to: int | None = None) -> MicroBatchList:
    """The chain an engine runs before its forward passes (areal/engine/fsdp_engine.py:1778-1786): position ids,
    split into balanced micro-batches, pack each, pad each."""
    data = dict(data)
    if "position_ids" not in data:
        data = amend_position_ids(data)
    mb_list = split_padded_tensor_dict_into_mb_list(data, mb_spec)
    mb_list.mbs = [pack_tensor_dict(mb) for mb in mb_list.mbs]
    return pad_mb_list(mb_list, pad_value=pad_value, pad_to_maximum=pad_to_maximum, batch_align_to=batch_align_to,
                       seq_align_to=seq_align_to)
