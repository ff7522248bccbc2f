"""One GPU's share of the vocabulary-parallel log-prob op.

The reference's tensor-parallel path (areal/utils/functional/vocab_parallel.py:84-372, 375-398) keeps a ``[T, V / tp]``
slice of the logits on every rank and combines per-row statistics with all-reduces.  The collectives are outside this
build; what one GPU does is here: the streaming pass over a slice, the reduction of the per-slice statistics (three
``[T]`` vectors per slice: what a single exchange would carry), and the backward of a slice from the combined
statistics.  ``gather_logprobs_entropy_vocab_shards`` runs all slices on one GPU, which is how the pieces are tested
against the unsharded op.
"""
from __future__ import annotations

import torch

from . import _native as N
from .functional import _DTYPES, _f32, _ptr, _require_gpu, _rows, _stream


def shard_statistics(logits_shard: torch.Tensor, labels: torch.Tensor, vocab_start: int, temperature: float = 1.0):
    """``(lse, ez, logp_local, labels_local)`` of one ``[T, V_i]`` slice that starts at vocabulary index
    ``vocab_start``: the slice's own logsumexp and ``sum_j softmax_j z_j`` per row, the label's log-prob within the
    slice (NaN where the label lies elsewhere), and the labels shifted into the slice (-1 where elsewhere)."""
    _require_gpu(logits_shard, "logits_shard")
    x, T, V, stride = _rows(logits_shard)
    dev = x.device
    y = labels.to(device=dev, dtype=torch.int64).reshape(-1) - int(vocab_start)
    y = torch.where((y >= 0) & (y < V), y, torch.full_like(y, -1)).contiguous()
    f32 = dict(dtype=torch.float32, device=dev)
    logp, lse, ez = torch.empty(T, **f32), torch.empty(T, **f32), torch.empty(T, **f32)
    with torch.cuda.device(dev):
        N.check(N.load().aa_logits_fwd(_ptr(x), _DTYPES[x.dtype], T, V, stride, _ptr(y), 1.0 / float(temperature),
                                       _ptr(logp), None, _ptr(lse), _ptr(ez), None, None, _stream(dev)), "aa_logits_fwd")
    return lse, ez, logp, y


def combine_shard_statistics(lse: torch.Tensor, ez: torch.Tensor, logp_local: torch.Tensor):
    """``(logp, entropy, row_lse, row_ez)`` from the stacked ``[n_shards, T]`` statistics of all slices."""
    _require_gpu(lse, "lse")
    S, T = lse.shape
    dev = lse.device
    f32 = dict(dtype=torch.float32, device=dev)
    logp, entropy, row_lse, row_ez = (torch.empty(T, **f32) for _ in range(4))
    with torch.cuda.device(dev):
        N.check(N.load().aa_vocab_partials_combine(_ptr(_f32(lse)), _ptr(_f32(ez)), _ptr(_f32(logp_local)), S, T,
                                                   _ptr(logp), _ptr(entropy), _ptr(row_lse), _ptr(row_ez),
                                                   _stream(dev)), "aa_vocab_partials_combine")
    return logp, entropy, row_lse, row_ez


def shard_backward(logits_shard: torch.Tensor, labels_local: torch.Tensor, row_lse: torch.Tensor, row_ez: torch.Tensor,
                   g_logp: torch.Tensor | None, g_entropy: torch.Tensor | None, temperature: float = 1.0):
    """Gradient of one slice from the combined statistics: ``(g_logp (1[j = label] - p_j) + g_entropy p_j (row_ez -
    z_j)) / temperature`` with ``p_j = exp(z_j - row_lse)`` the probability under the full softmax
    (vocab_parallel.py:180-192, 339-370)."""
    x, T, V, stride = _rows(logits_shard)
    dev = x.device
    gl = torch.zeros(T, dtype=torch.float32, device=dev) if g_logp is None else _f32(g_logp)
    gh = None if g_entropy is None else _f32(g_entropy)
    if stride == V:
        out = torch.empty_like(x, memory_format=torch.contiguous_format)
    else:
        out = torch.empty_strided((T, V), (stride, 1), dtype=x.dtype, device=dev)
    with torch.cuda.device(dev):
        N.check(N.load().aa_logits_bwd(_ptr(x), _DTYPES[x.dtype], T, V, stride, _ptr(labels_local),
                                       1.0 / float(temperature), _ptr(row_lse), _ptr(row_ez), _ptr(gl), _ptr(gh), T,
                                       _ptr(out), _stream(dev)), "aa_logits_bwd")
    return out


class _ShardedLogprobsEntropy(torch.autograd.Function):
    @staticmethod
    def forward(ctx, labels, temperature, *shards):
        stats, locals_ = [], []
        start = 0
        for sh in shards:
            lse, ez, lp, y = shard_statistics(sh, labels, start, temperature)
            stats.append((lse, ez, lp))
            locals_.append(y)
            start += sh.shape[-1]
        logp, entropy, row_lse, row_ez = combine_shard_statistics(*(torch.stack(c) for c in zip(*stats)))
        ctx.save_for_backward(row_lse, row_ez, *locals_, *shards)
        ctx.n, ctx.temperature = len(shards), temperature
        return logp, entropy

    @staticmethod
    def backward(ctx, g_logp, g_entropy):
        row_lse, row_ez = ctx.saved_tensors[:2]
        locals_ = ctx.saved_tensors[2:2 + ctx.n]
        shards = ctx.saved_tensors[2 + ctx.n:]
        grads = tuple(
            shard_backward(sh, y, row_lse, row_ez, g_logp, g_entropy, ctx.temperature).view_as(sh)
            if sh.requires_grad else None
            for sh, y in zip(shards, locals_)
        )
        return (None, None) + grads


def gather_logprobs_entropy_vocab_shards(shards: list[torch.Tensor], labels: torch.Tensor, temperature: float = 1.0):
    """``gather_logprobs_entropy`` of the logits whose vocabulary axis is cut into ``shards`` (``[T, V_i]`` each, in
    vocabulary order): every slice is read once in the forward and once (plus the write of its gradient) in the
    backward, and only ``[T]`` vectors cross slices.  Differentiable in every shard."""
    if not shards:
        raise ValueError("at least one shard")
    T = shards[0].shape[0]
    if any(sh.ndim != 2 or sh.shape[0] != T for sh in shards) or labels.numel() != T:
        raise ValueError("shards must be [T, V_i] with one label per row")
    assert T > 0, "Input logits must have at least one element"
    logp, entropy = _ShardedLogprobsEntropy.apply(labels, float(temperature), *shards)
    return logp.view(labels.shape), entropy.view(labels.shape)
