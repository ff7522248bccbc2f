"""Supervised fine-tuning loss over a packed batch.

Host-side mirror of ``compute_packed_sft_loss`` (areal/trainer/sft/lm_engine.py:81-131), given log-probs, and fused
with the log-prob op (one pass over the logits that also writes their gradient) or with the lm_head as well.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _native as N
from .functional import (
    _DTYPES,
    _FusedLmHeadPpo,
    _FusedLogitsPpo,
    _count_nonzero,
    _f32,
    _mask_u8,
    _ptr,
    _require_gpu,
    _rows,
    _stream,
    gather_logprobs_entropy_stats,
    lm_head_logprobs_entropy,
)


def _nll_params() -> N.PpoParams:
    return N.PpoParams(clip_lo=0.0, clip_hi=0.0, c_clip=0.0, has_c_clip=0, has_behave_weight=0, loss_kind=1)


def _cu_i32(cu_seqlens, dev):
    if cu_seqlens is None:
        return None, 0
    cu = cu_seqlens.to(device=dev, dtype=torch.int32).contiguous()
    return cu, cu.numel() - 1


def _launch(logp, m8, cu, n_seqs, n_valid, scale, want_grad, want_stat):
    """``aa_sft_loss``: returns (loss, g_logp, stat_loss, seq_logp, seq_count, seq_ppl)."""
    lib = N.load()
    dev = logp.device
    T = logp.numel()
    f32 = dict(dtype=torch.float32, device=dev)
    loss = torch.empty((), **f32)
    g = torch.empty(T, **f32) if want_grad else None
    stat_loss = torch.empty(T, **f32) if want_stat else None
    seq_logp = torch.empty(n_seqs + 1, dtype=torch.float64, device=dev)
    seq_count = torch.empty(n_seqs + 1, dtype=torch.int32, device=dev)
    seq_ppl = torch.empty(n_seqs, **f32)
    with torch.cuda.device(dev):
        N.check(lib.aa_sft_loss(_ptr(logp), _ptr(m8), T, _ptr(cu), n_seqs, _ptr(n_valid), _ptr(scale), _ptr(loss),
                                _ptr(g), _ptr(stat_loss), _ptr(seq_logp), _ptr(seq_count), _ptr(seq_ppl),
                                _stream(dev)), "aa_sft_loss")
    return loss, g, stat_loss, seq_logp, seq_count, seq_ppl


class _SftLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logp, m8, cu, n_seqs, n_valid, scale):
        loss, g, stat_loss, seq_logp, seq_count, seq_ppl = _launch(logp, m8, cu, n_seqs, n_valid, scale, True, True)
        ctx.save_for_backward(g)
        ctx.mark_non_differentiable(stat_loss, seq_logp, seq_count, seq_ppl)
        return loss, stat_loss, seq_logp, seq_count, seq_ppl

    @staticmethod
    def backward(ctx, g_loss, *_unused):
        (g,) = ctx.saved_tensors
        # [T] floats: a copy is cheap and keeps the saved gradient intact for a second backward (retain_graph)
        out = g.clone()
        dev = g.device
        up = _f32(g_loss).reshape(1)
        if out.numel():
            with torch.cuda.device(dev):
                N.check(N.load().aa_scale_inplace(_ptr(out), _DTYPES[out.dtype], out.numel(), _ptr(up), _stream(dev)),
                        "aa_scale_inplace")
        return out, None, None, None, None, None


def _stat(stat_loss, seq_logp, seq_count, seq_ppl, n_seqs, extra=None):
    stat = dict(loss=stat_loss, seqlogp=seq_logp[:n_seqs], n_seqs=seq_count[:n_seqs] > 0, ppl=seq_ppl,
                valid_tokens_per_seq=seq_count[:n_seqs])
    if extra:
        stat.update(extra)
    return stat


def _scale_tensor(loss_scale, dev):
    if loss_scale is None:
        return None
    return torch.as_tensor(loss_scale, dtype=torch.float32, device=dev).reshape(1)


def sft_loss_fn(logprobs: torch.Tensor, loss_mask: torch.Tensor, cu_seqlens: torch.Tensor | None = None,
                loss_scale: torch.Tensor | float | None = None) -> tuple[torch.Tensor, dict]:
    """``-sum(where(loss_mask, logprobs, 0)) / (1e-5 + count_nonzero(loss_mask))`` over a packed ``[T]`` batch;
    lm_engine.py:93-96.  Returns ``(loss, stat)``: ``stat["loss"]`` is ``-where(mask, logprobs, 0)`` (what the
    reference logs per token), and per sequence of ``cu_seqlens`` ``seqlogp`` (fp64 mean log-prob of the selected
    tokens, 0 for a sequence without one), ``n_seqs`` (bool: has a selected token), ``ppl = exp(-seqlogp)`` and
    ``valid_tokens_per_seq``: lm_engine.py:97-121 without its loop of per-sequence read-backs."""
    _require_gpu(logprobs, "logprobs")
    if logprobs.dim() != 1 or loss_mask.shape != logprobs.shape:
        raise ValueError("logprobs and loss_mask must be 1-D and of the same length")
    dev = logprobs.device
    lp = logprobs if logprobs.dtype == torch.float32 and logprobs.is_contiguous() else logprobs.float().contiguous()
    m8 = _mask_u8(loss_mask.to(dev))
    cu, n_seqs = _cu_i32(cu_seqlens, dev)
    loss, stat_loss, seq_logp, seq_count, seq_ppl = _SftLoss.apply(lp, m8, cu, n_seqs, _count_nonzero(m8),
                                                                   _scale_tensor(loss_scale, dev))
    return loss, _stat(stat_loss, seq_logp, seq_count, seq_ppl, n_seqs)


def _check_fused_inputs(rows: torch.Tensor, labels: torch.Tensor, loss_mask: torch.Tensor, what: str) -> int:
    if rows.ndim != 2 or labels.ndim != 1 or labels.shape[0] != rows.shape[0]:
        raise ValueError(f"expected {what} [T, .] and labels [T], got {tuple(rows.shape)} and {tuple(labels.shape)}")
    assert rows.shape[0] > 0, "Input must have at least one token"
    T_active = loss_mask.shape[0]
    if loss_mask.ndim != 1 or T_active > rows.shape[0]:
        raise ValueError(f"loss_mask shape {tuple(loss_mask.shape)} does not fit {what} {tuple(rows.shape)}")
    return T_active


def fused_logprobs_sft_loss(logits: torch.Tensor, labels: torch.Tensor, loss_mask: torch.Tensor,
                            cu_seqlens: torch.Tensor | None = None, temperature: float = 1.0,
                            loss_scale: torch.Tensor | float | None = None,
                            inplace_backward: bool = False) -> tuple[torch.Tensor, dict]:
    """``gather_logprobs`` + ``compute_packed_sft_loss`` (+ backward) in one pass over the logits.

    ``logits`` is ``[T_pad, V]``, ``labels`` ``[T_pad]``, ``loss_mask`` the un-padded ``[T]`` mask with ``T <= T_pad``
    (rows past ``T`` get a zero gradient).  ``loss.backward()`` hands back the gradient written during the forward
    pass.  ``stat`` is that of ``sft_loss_fn`` plus ``logprobs``, ``entropy``, ``vocab_min_logits`` and
    ``vocab_max_logits`` (``[T]``).  Without a gradient to produce the call is the forward kernel and the loss.
    ``inplace_backward=True`` writes the gradient over the logits, as in ``fused_logprobs_ppo_loss``."""
    _require_gpu(logits, "logits")
    T_active = _check_fused_inputs(logits, labels, loss_mask, "logits")
    dev = logits.device
    scale_t = _scale_tensor(loss_scale, dev)
    cu, n_seqs = _cu_i32(cu_seqlens, dev)
    if not (torch.is_grad_enabled() and logits.requires_grad):
        logp, entropy, vmin, vmax = (t[:T_active] for t in gather_logprobs_entropy_stats(logits, labels, temperature))
        loss, stat = sft_loss_fn(logp, loss_mask, cu_seqlens, loss_scale)
        stat.update(logprobs=logp.detach(), entropy=entropy.detach(), vocab_min_logits=vmin, vocab_max_logits=vmax)
        return loss, stat
    x, T, V, stride = _rows(logits)
    y = labels.to(device=dev, dtype=torch.int64).contiguous()
    m8 = _mask_u8(loss_mask.to(dev))
    n_valid = _count_nonzero(m8)
    loss, logp, entropy, vmax, vmin, stat_loss, _ratio, _flags = _FusedLogitsPpo.apply(
        x, y, stride, float(temperature), T_active, None, None, m8, None, _nll_params(), n_valid, scale_t, True,
        bool(inplace_backward),
    )
    logp_a = logp[:T_active]
    _, _, _, seq_logp, seq_count, seq_ppl = _launch(logp_a, m8, cu, n_seqs, n_valid, None, False, False)
    return loss, _stat(stat_loss, seq_logp, seq_count, seq_ppl, n_seqs,
                       dict(logprobs=logp_a, entropy=entropy[:T_active], vocab_min_logits=vmin[:T_active],
                            vocab_max_logits=vmax[:T_active]))


def fused_lm_head_sft_loss(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor, loss_mask: torch.Tensor,
                           cu_seqlens: torch.Tensor | None = None, temperature: float = 1.0,
                           loss_scale: torch.Tensor | float | None = None, skip_masked_tokens: bool = True,
                           kept_per_chunk: list[int] | None = None) -> tuple[torch.Tensor, dict]:
    """lm_head + ``gather_logprobs`` + ``compute_packed_sft_loss`` (+ backward) for one micro-batch, in token chunks
    whose logits never leave the workspace (see ``fused_lm_head_ppo_loss``, of which this is the supervised
    counterpart: ``hidden`` ``[T_pad, H]`` and ``weight`` ``[V, H]`` in bf16, ``skip_masked_tokens`` /
    ``kept_per_chunk`` as there: prompt tokens have no gradient, so the gradient GEMMs leave them out)."""
    _require_gpu(hidden, "hidden")
    if weight.ndim != 2 or hidden.ndim != 2 or hidden.shape[1] != weight.shape[1]:
        raise ValueError(f"expected hidden [T, H] and weight [V, H], got {tuple(hidden.shape)} and {tuple(weight.shape)}")
    T_active = _check_fused_inputs(hidden, labels, loss_mask, "hidden")
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("fused lm_head expects bf16 hidden states and weights")
    dev = hidden.device
    scale_t = _scale_tensor(loss_scale, dev)
    cu, n_seqs = _cu_i32(cu_seqlens, dev)
    y = labels.to(device=dev, dtype=torch.int64).contiguous()
    if not (torch.is_grad_enabled() and (hidden.requires_grad or weight.requires_grad)):
        logp, entropy = lm_head_logprobs_entropy(hidden, weight, y, temperature)
        logp, entropy = logp[:T_active], entropy[:T_active]
        loss, stat = sft_loss_fn(logp, loss_mask, cu_seqlens, loss_scale)
        stat.update(logprobs=logp.detach(), entropy=entropy.detach())
        return loss, stat
    m8 = _mask_u8(loss_mask.to(dev))
    n_valid = _count_nonzero(m8)
    kept = None
    if skip_masked_tokens:
        chunk = int(N.load().aa_lmhead_chunk_tokens())
        n_chunks = (hidden.shape[0] + chunk - 1) // chunk
        if kept_per_chunk is not None:
            kept = [int(v) for v in kept_per_chunk]
            if len(kept) != n_chunks:
                raise ValueError(f"kept_per_chunk needs one count per chunk of {chunk} tokens")
        else:  # the device counts the tokens with a mask itself: nothing is read back
            kept = [N.AA_LMHEAD_COUNT_ON_DEVICE] * n_chunks
    loss, logp, entropy, stat_loss, _ratio, _flags, _vmax, _vmin = _FusedLmHeadPpo.apply(
        hidden.contiguous(), weight.contiguous(), y, float(temperature), T_active, None, None, m8, None, _nll_params(),
        n_valid, scale_t, kept, 1,  # aa_lmhead_backward_mode: carry
    )
    logp_a = logp[:T_active]
    _, _, _, seq_logp, seq_count, seq_ppl = _launch(logp_a, m8, cu, n_seqs, n_valid, None, False, False)
    return loss, _stat(stat_loss, seq_logp, seq_count, seq_ppl, n_seqs,
                       dict(logprobs=logp_a, entropy=entropy[:T_active]))
