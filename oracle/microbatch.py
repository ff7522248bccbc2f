"""CPU oracle of the micro-batch allocation and split.  TEST INFRASTRUCTURE ONLY.

Restates ``ffd_allocate`` / ``kk_allocate`` (areal/utils/seqpack.py:196-267, 272-381, 446-537) and
``split_padded_tensor_dict_into_mb_list`` (areal/utils/data.py:696-812) in the slowest obvious way: a sorted list
that is re-sorted after every change instead of bisection, a list of partial solutions that is re-sorted every round
instead of a heap, and one slice per row instead of a gather.  How it is pinned is listed in ``oracle/PINNING.md``.
"""
from __future__ import annotations

import functools
import math

import numpy as np
import torch


def ffd_once(values, capacity, min_groups):
    """seqpack.py:196-231."""
    values = np.asarray(values)
    groups = []          # [sum, creation number, members]
    for idx in np.argsort(-values):
        v = values[idx]
        by_weight = sorted(groups, key=lambda g: (g[0], g[1]))
        if len(groups) < min_groups or by_weight[0][0] + v > capacity:          # :214-220
            groups.append([float(v), len(groups), [idx]])
            continue
        candidates = [g for g in by_weight if (g[0], g[1]) <= (capacity - v, len(values))]   # :222-223
        fewest = min(len(g[2]) for g in candidates)
        chosen = next(g for g in candidates if len(g[2]) == fewest)             # first of the lightest-first list
        chosen[0] = float(v + chosen[0])
        chosen[2].append(idx)
    return [g[2] for g in sorted(groups, key=lambda g: g[1])]


def ffd_allocate(values, capacity, min_groups, n_groups_divisor=1):
    """seqpack.py:234-267."""
    if min_groups is None or min_groups < n_groups_divisor:
        min_groups = n_groups_divisor
    if any(v > capacity for v in values):
        raise RuntimeError("value larger than capacity")
    if len(values) < min_groups:
        raise RuntimeError("fewer values than groups")
    while True:
        res = ffd_once(values, capacity, min_groups)
        min_groups += n_groups_divisor - min_groups % n_groups_divisor
        if len(res) % n_groups_divisor == 0:
            return res
        if len(values) < min_groups:
            raise RuntimeError("cannot allocate")


def _set_less(a, b):
    """a, b = (sum, items); seqpack.py:290-295."""
    if a[0] != b[0]:
        return a[0] < b[0]
    if len(a[1]) != len(b[1]):
        return len(a[1]) < len(b[1])
    return a[1] < b[1]


def _sets_descending(sets):
    cmp = lambda a, b: -1 if _set_less(b, a) else (1 if _set_less(a, b) else 0)
    return sorted(sets, key=functools.cmp_to_key(cmp))


def _state_less(a, b):
    """States are lists of sets, heaviest first; seqpack.py:330-334."""
    sa, sb = a[0][0] - a[-1][0], b[0][0] - b[-1][0]
    if sa != sb:
        return sa > sb
    return _set_less(b[0], a[0])


def kk_partition(values, k, equal_size=False):
    """seqpack.py:337-381 with the priority queue replaced by a full sort per round (the order is total: the
    heaviest sets of two states hold different original indices)."""
    ranked = sorted((val, idx) for idx, val in enumerate(values))
    states = []
    if equal_size:
        assert len(values) % k == 0
        for off in range(0, len(ranked), k):
            states.append(_sets_descending([(val, [(idx, val)]) for val, idx in ranked[off:off + k]]))
    else:
        for val, idx in ranked:
            states.append(_sets_descending([(val, [(idx, val)])] + [(0, []) for _ in range(k - 1)]))
    cmp = lambda a, b: -1 if _state_less(a, b) else (1 if _state_less(b, a) else 0)
    while len(states) > 1:
        states = sorted(states, key=functools.cmp_to_key(cmp))
        s0, s1, rest = states[0], states[1], states[2:]
        merged = [(s0[i][0] + s1[k - 1 - i][0], s0[i][1] + s1[k - 1 - i][1]) for i in range(k)]     # :319-324
        states = rest + [_sets_descending(merged)]
    return [[idx for idx, _ in s[1]] for s in states[0]]


def kk_allocate(values, capacity, min_groups, n_groups_divisor=1, equal_size=False):
    """seqpack.py:446-537."""
    if min_groups is None or min_groups < n_groups_divisor:
        min_groups = n_groups_divisor
    if any(v > capacity for v in values):
        raise RuntimeError("value exceeds capacity")
    if len(values) < min_groups:
        raise RuntimeError("fewer values than groups")
    k = max(min_groups, math.ceil(sum(values) / capacity))
    if n_groups_divisor > 1:
        k = math.ceil(k / n_groups_divisor) * n_groups_divisor
    k = min(k, len(values))
    if equal_size and len(values) % k != 0:
        raise RuntimeError("not divisible")
    parts = kk_partition(values, k, equal_size)
    for g in parts:
        if sum(values[i] for i in g) > capacity:
            return ffd_allocate(values, capacity, min_groups, n_groups_divisor)
    return parts


def allocate_balanced_mbs(lens, max_tokens_per_mb, n_mbs=1, n_mbs_divisor=1, algorithm="ffd"):
    """data.py:448-472."""
    fn = dict(ffd=ffd_allocate, kk=kk_allocate)[algorithm]
    groups = fn(lens, max_tokens_per_mb, min_groups=n_mbs, n_groups_divisor=n_mbs_divisor)
    return sorted([sorted(g) for g in groups])


def split_padded_tensor_dict(data, max_tokens_per_mb=None, n_mbs=1, granularity=1, n_mbs_divisor=1, algorithm="ffd"):
    """(mbs, group_lens, forward_indices, backward_indices); data.py:711-812 for tensor-only inputs."""
    if max_tokens_per_mb is None:
        max_tokens_per_mb = int(1e12)
    attn = data["attention_mask"]
    bs, max_seqlen = attn.shape
    seq_lens = attn.sum(1).long().tolist()
    input_lens = attn.view(bs // granularity, granularity, -1).sum(dim=(1, 2)).long().numpy()
    groups = allocate_balanced_mbs(input_lens, max_tokens_per_mb, n_mbs, n_mbs_divisor, algorithm)
    groups = [[i * granularity + j for i in g for j in range(granularity)] for g in groups]
    forward = [i for g in groups for i in g]
    backward = np.zeros(bs, dtype=np.int64)
    backward[forward] = np.arange(bs)
    mbs = []
    for g in groups:
        mb = {}
        for key, value in data.items():
            if key == "position_ids" or (torch.is_tensor(value) and value.numel() == bs * max_seqlen):
                mb[key] = torch.stack([value[i] for i in g])
            else:
                mb[key] = value
        mbs.append(mb)
    return mbs, [sum(seq_lens[i] for i in g) for g in groups], forward, backward.tolist()
