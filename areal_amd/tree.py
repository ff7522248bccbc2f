"""Log-probs and entropy for sequences packed as a prefix tree.

Host-side mirror of ``gather_packed_tree_logprobs`` / ``gather_packed_tree_logprobs_entropy``
(areal/models/tree_attn/functional.py:206-467).  In a packed tree several sequences share the tokens of their
common prefixes, so the label of a row is not the next row: the last token of a node predicts the first token of
each child, which sits elsewhere in the packed tensor.  The reference walks the trie in Python, one small
``gather_logprobs`` call per node and per transition (with caches); here the trie is flattened once into
``(row, label position)`` pairs, every distinct pair is computed once by one pass over the logits, and the
per-sequence results are an index select.
"""
from __future__ import annotations

from typing import Any

import torch

from . import _native as N
from .functional import _DTYPES, _f32, _ptr, _require_gpu, _rows, _stream


class _PairLogprobs(torch.autograd.Function):
    """logp / entropy of distinct (row, label) pairs; differentiable in logits."""

    @staticmethod
    def forward(ctx, logits2d, stride, rows, labels, temperature, want_entropy):
        lib = N.load()
        T, V = logits2d.shape
        dev = logits2d.device
        K = rows.numel()
        f32 = dict(dtype=torch.float32, device=dev)
        none_label = torch.full((T,), -1, dtype=torch.int64, device=dev)
        row_lse, row_ez = torch.empty(T, **f32), torch.empty(T, **f32)
        row_ent = torch.empty(T, **f32)
        scratch = torch.empty(T, **f32)
        logp = torch.empty(K, **f32)
        entropy = torch.empty(K, **f32) if want_entropy else None
        inv_t = 1.0 / float(temperature)
        with torch.cuda.device(dev):
            st = _stream(dev)
            N.check(lib.aa_logits_fwd(_ptr(logits2d), _DTYPES[logits2d.dtype], T, V, stride, _ptr(none_label), inv_t,
                                      _ptr(scratch), _ptr(row_ent), _ptr(row_lse), _ptr(row_ez), None, None, st),
                    "aa_logits_fwd")
            N.check(lib.aa_logits_pairs_fwd(_ptr(logits2d), _DTYPES[logits2d.dtype], T, V, stride, _ptr(rows),
                                            _ptr(labels), K, inv_t, _ptr(row_lse), _ptr(row_ent), _ptr(logp),
                                            _ptr(entropy), st), "aa_logits_pairs_fwd")
        ctx.save_for_backward(logits2d, rows, labels, row_lse, row_ez, none_label)
        ctx.inv_t, ctx.stride = inv_t, stride
        return logp, entropy

    @staticmethod
    def backward(ctx, g_logp, g_entropy):
        lib = N.load()
        logits2d, rows, labels, row_lse, row_ez, none_label = ctx.saved_tensors
        T, V = logits2d.shape
        dev = logits2d.device
        K = rows.numel()
        gl = torch.zeros(K, dtype=torch.float32, device=dev) if g_logp is None else _f32(g_logp)
        # softmax part: per row, the sums of the pair gradients; one-hot part: scattered afterwards
        G = torch.zeros(T, dtype=torch.float32, device=dev).index_add_(0, rows, gl)
        H = None
        if g_entropy is not None:
            H = torch.zeros(T, dtype=torch.float32, device=dev).index_add_(0, rows, _f32(g_entropy))
        if ctx.stride == V:
            dlogits = torch.empty_like(logits2d, memory_format=torch.contiguous_format)
        else:
            dlogits = torch.empty_strided((T, V), (ctx.stride, 1), dtype=logits2d.dtype, device=dev)
        with torch.cuda.device(dev):
            st = _stream(dev)
            N.check(lib.aa_logits_bwd(_ptr(logits2d), _DTYPES[logits2d.dtype], T, V, ctx.stride, _ptr(none_label),
                                      ctx.inv_t, _ptr(row_lse), _ptr(row_ez), _ptr(G), _ptr(H), T, _ptr(dlogits), st),
                    "aa_logits_bwd")
            N.check(lib.aa_logits_pairs_scatter(_ptr(dlogits), _DTYPES[logits2d.dtype], T, V, ctx.stride, _ptr(rows),
                                                _ptr(labels), K, _ptr(gl), ctx.inv_t, st), "aa_logits_pairs_scatter")
        return dlogits, None, None, None, None, None


def gather_logprobs_entropy_pairs(logits: torch.Tensor, rows: torch.Tensor, labels: torch.Tensor,
                                  temperature: float = 1.0, with_entropy: bool = True):
    """``log_softmax(logits[rows] / temperature)[labels]`` (and the entropy of those rows) for ``K`` pairs.

    ``logits`` is ``[T, V]``; ``rows`` and ``labels`` are ``[K]`` integer tensors.  The pairs must be distinct
    (repeat results with an index select instead): the backward scatters into ``d(logits)`` without atomics.
    One streaming pass over all ``T`` rows however many pairs there are.
    """
    _require_gpu(logits, "logits")
    if logits.ndim != 2 or rows.ndim != 1 or rows.shape != labels.shape:
        raise ValueError(f"expected logits [T, V] and rows, labels [K]; got {tuple(logits.shape)}, "
                         f"{tuple(rows.shape)}, {tuple(labels.shape)}")
    assert logits.shape[0] > 0, "Input logits must have at least one element"
    x, _, _, stride = _rows(logits)
    r = rows.to(device=x.device, dtype=torch.int64).contiguous()
    y = labels.to(device=x.device, dtype=torch.int64).contiguous()
    return _PairLogprobs.apply(x, stride, r, y, float(temperature), with_entropy)


def tree_sequence_pairs(trie: Any) -> tuple[list[int], list[int], list[int]]:
    """Flatten a trie into prediction pairs, the way the reference walks it (functional.py:283-312).

    ``trie`` is any object with ``all_sequence_ids`` and ``get_sequence_tree_indices(seq_id)`` (a list of
    inclusive ``(start, end)`` ranges of packed positions, one per node on the sequence's path).  Returns
    ``(pred_pos, label_pos, select)``: the distinct (prediction row, label position) pairs in first-visit order,
    and for every token of every sequence (concatenated in ``all_sequence_ids`` order) the index of its pair.
    Inside a node position ``p`` predicts ``p + 1``; the last position of a node predicts the first position of
    the next node on the path, and the last node wraps to position 0, as the reference does.
    """
    index: dict[tuple[int, int], int] = {}
    pred_pos: list[int] = []
    label_pos: list[int] = []
    select: list[int] = []

    def pair(p: int, q: int) -> int:
        k = index.get((p, q))
        if k is None:
            k = index[(p, q)] = len(pred_pos)
            pred_pos.append(p)
            label_pos.append(q)
        return k

    for seq_id in trie.all_sequence_ids:
        indices = trie.get_sequence_tree_indices(seq_id)
        for i, (start, end) in enumerate(indices):
            for p in range(start, end):
                select.append(pair(p, p + 1))
            next_start = indices[i + 1][0] if i + 1 < len(indices) else 0
            select.append(pair(end, next_start))
    return pred_pos, label_pos, select


def gather_packed_tree_logprobs_entropy(logits: torch.Tensor, trie: Any, input_ids: torch.Tensor,
                                        temperature: float = 1.0, chunk_size: int = 1024, tp_group=None):
    """``(logprobs, entropy)`` of all sequences of a packed tree, concatenated in ``trie.all_sequence_ids`` order;
    functional.py:430-467.  ``chunk_size`` is accepted for signature compatibility (nothing is chunked here)."""
    from .functional import _check_tp

    _check_tp(tp_group)
    if not trie.all_sequence_ids:
        empty = torch.empty(0, device=logits.device, dtype=torch.float)
        return empty, empty
    pred_pos, label_pos, select = tree_sequence_pairs(trie)
    dev = logits.device
    ids = input_ids.reshape(-1).to(dev)
    if not select:
        empty = torch.empty(0, device=dev, dtype=torch.float)
        return empty, empty
    rows = torch.tensor(pred_pos, dtype=torch.int64, device=dev)
    labels = ids[torch.tensor(label_pos, dtype=torch.int64, device=dev)].to(torch.int64)
    x = logits.reshape(-1, logits.shape[-1])
    lp, ent = gather_logprobs_entropy_pairs(x, rows, labels, temperature, True)
    sel = torch.tensor(select, dtype=torch.int64, device=dev)
    return lp[sel], ent[sel]


def gather_packed_tree_logprobs(logits: torch.Tensor, trie: Any, input_ids: torch.Tensor, temperature: float = 1.0,
                                chunk_size: int = 1024, tp_group=None) -> torch.Tensor:
    """Log-probs only; functional.py:403-427."""
    return gather_packed_tree_logprobs_entropy(logits, trie, input_ids, temperature, chunk_size, tp_group)[0]


@torch.no_grad()
def gather_packed_tree_vocab_stats(logits: torch.Tensor, trie: Any) -> tuple[torch.Tensor, torch.Tensor]:
    """``(vocab_min_logits, vocab_max_logits)`` of all sequences of a packed tree, concatenated in
    ``trie.all_sequence_ids`` order; functional.py:471-564.  Every position of every node on a sequence's path
    contributes the minimum / maximum of its row of logits (inclusive ranges, no shift).  One streaming pass gives the
    extrema of all rows; the per-sequence results are one index select."""
    if not trie.all_sequence_ids:
        empty = torch.empty(0, device=logits.device, dtype=torch.float)
        return empty, empty
    _require_gpu(logits, "logits")
    x, T, V, stride = _rows(logits.reshape(-1, logits.shape[-1]))
    dev = x.device
    positions: list[int] = []
    for seq_id in trie.all_sequence_ids:
        for start, end in trie.get_sequence_tree_indices(seq_id):
            positions.extend(range(start, end + 1))
    f32 = dict(dtype=torch.float32, device=dev)
    vmax, vmin, scratch = torch.empty(T, **f32), torch.empty(T, **f32), torch.empty(T, **f32)
    none_label = torch.full((T,), -1, dtype=torch.int64, device=dev)
    with torch.cuda.device(dev):
        N.check(N.load().aa_logits_fwd(_ptr(x), _DTYPES[x.dtype], T, V, stride, _ptr(none_label), 1.0, _ptr(scratch),
                                       None, None, None, _ptr(vmax), _ptr(vmin), _stream(dev)), "aa_logits_fwd")
    sel = torch.tensor(positions, dtype=torch.int64, device=dev)
    return vmin[sel], vmax[sel]


def merge_packed_tree_results(results_list: list[dict[int, torch.Tensor]], batch_size: int,
                              max_seq_len: int | None = None, padding_value: float = 0.0) -> torch.Tensor:
    """Per-sequence results of several packed trees back into one ``[batch_size, max_seq_len]`` tensor, sequence
    ``seq_id`` in row ``seq_id``, cut or padded to ``max_seq_len`` (the longest result when None);
    functional.py:567-639.  The rows are placed by one segment copy instead of one slice assignment each."""
    from .packing import segment_copy

    combined: dict[int, torch.Tensor] = {}
    for results in results_list:
        for seq_id, tensor in results.items():
            if seq_id in combined:
                raise ValueError(f"Duplicate sequence_id {seq_id} found across microbatches")
            combined[seq_id] = tensor
    if not combined:
        return torch.full((batch_size, max_seq_len or 0), padding_value, device=torch.device("cpu"))
    first = next(iter(combined.values()))
    if max_seq_len is None:
        max_seq_len = max(t.shape[0] for t in combined.values())
    output = torch.full((batch_size, max_seq_len), padding_value, dtype=first.dtype, device=first.device)
    for seq_id in combined:
        if seq_id >= batch_size:
            raise ValueError(f"sequence_id {seq_id} exceeds batch_size {batch_size}")
    ids = list(combined)
    lens = [int(combined[i].shape[0]) for i in ids]
    take = [min(n, max_seq_len) for n in lens]
    total = sum(take)
    if total == 0:
        return output
    flat = torch.cat([combined[i].reshape(-1) for i in ids]).contiguous()
    src_starts, dst_starts, cu = [], [], [0]
    off = 0
    for i, n, k in zip(ids, lens, take):
        src_starts.append(off)
        dst_starts.append(i * max_seq_len)
        cu.append(cu[-1] + k)
        off += n
    segment_copy(flat, output.view(-1), torch.tensor(src_starts), torch.tensor(dst_starts),
                 torch.tensor(cu, dtype=torch.int32), total)
    return output
