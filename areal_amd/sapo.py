"""SAPO loss (soft sigmoid gates instead of the PPO clip) fused with the log-prob op or with the lm_head.

``sapo_loss_fn`` (areal/utils/functional/functional.py:562-638) on given log-probs is ``areal_amd.sapo_loss_fn``; the
two functions here put its token-level form into the single pass over the logits (one read, one write per logit instead
of the log-prob op's forward and backward passes) and into the chunked lm_head step (no logits in memory).
"""
from __future__ import annotations

import torch

from . import _native as N
from .functional import (
    _FusedLmHeadPpo,
    _FusedLogitsPpo,
    _count_nonzero,
    _f32,
    _mask_u8,
    _require_gpu,
    _rows,
    gather_logprobs_entropy_stats,
    lm_head_logprobs_entropy_stats,
    sapo_loss_fn,
)
from .sft import _check_fused_inputs, _scale_tensor


def _sapo_params(tau_pos: float, tau_neg: float) -> N.PpoParams:
    if tau_pos <= 0 or tau_neg <= 0:
        raise ValueError("SAPO temperatures (tau_pos, tau_neg) must be positive.")
    return N.PpoParams(clip_lo=0.0, clip_hi=0.0, c_clip=0.0, has_c_clip=0, has_behave_weight=0, loss_kind=2,
                       sapo_tau_pos=float(tau_pos), sapo_tau_neg=float(tau_neg))


def _sapo_stat(stat_loss, ratio, logp, old, adv, tau_pos, tau_neg, extra):
    """The stat dict of ``sapo_loss_fn`` (functional.py:624-636); the gates are functions of the ratio."""
    gate_pos = torch.sigmoid(tau_pos * (ratio - 1.0)) * (4.0 / tau_pos)
    gate_neg = torch.sigmoid(tau_neg * (ratio - 1.0)) * (4.0 / tau_neg)
    zeros = torch.zeros(ratio.shape, dtype=torch.bool, device=ratio.device)
    stat = dict(
        loss=stat_loss, importance_weight=ratio, approx_kl=logp - old, clip_mask=zeros, dual_clip_mask=zeros.clone(),
        sapo_soft_gate=torch.where(adv > 0, gate_pos, gate_neg), sapo_scaled_gate_pos=gate_pos,
        sapo_scaled_gate_neg=gate_neg,
    )
    stat.update(extra)
    return stat


def _check_per_token(loss_mask, **tensors):
    for name, t in tensors.items():
        if t.shape != loss_mask.shape:
            raise ValueError(f"{name} shape {tuple(t.shape)} != loss_mask shape {tuple(loss_mask.shape)}")


def fused_logprobs_sapo_loss(logits: torch.Tensor, labels: torch.Tensor, old_logprobs: torch.Tensor,
                             advantages: torch.Tensor, tau_pos: float, tau_neg: float, loss_mask: torch.Tensor,
                             temperature: float = 1.0, loss_scale: torch.Tensor | float | None = None,
                             inplace_backward: bool = False) -> tuple[torch.Tensor, dict]:
    """``gather_logprobs_entropy`` + token-level ``sapo_loss_fn`` (+ backward) in one pass over the logits.

    ``logits`` is ``[T_pad, V]``, ``labels`` ``[T_pad]``; ``old_logprobs``, ``advantages`` and ``loss_mask`` are the
    un-padded ``[T]`` tensors (rows past ``T`` get a zero gradient).  ``loss.backward()`` hands back the gradient
    written during the forward pass.  ``stat`` is that of ``sapo_loss_fn`` plus ``logprobs``, ``entropy``,
    ``vocab_min_logits`` and ``vocab_max_logits``.  Sequence-level SAPO needs every log-prob of a sequence first: use
    ``gather_logprobs`` and ``sapo_loss_fn``.  ``inplace_backward``: as in ``fused_logprobs_ppo_loss``."""
    _require_gpu(logits, "logits")
    params = _sapo_params(tau_pos, tau_neg)
    T_active = _check_fused_inputs(logits, labels, loss_mask, "logits")
    _check_per_token(loss_mask, old_logprobs=old_logprobs, advantages=advantages)
    dev = logits.device
    scale_t = _scale_tensor(loss_scale, dev)
    if not (torch.is_grad_enabled() and logits.requires_grad):
        logp, entropy, vmin, vmax = (t[:T_active] for t in gather_logprobs_entropy_stats(logits, labels, temperature))
        loss, stat = sapo_loss_fn(logp, old_logprobs, advantages, tau_pos, tau_neg, loss_mask)
        if scale_t is not None:
            loss = loss * scale_t.squeeze(0)
        stat.update(logprobs=logp.detach(), entropy=entropy.detach(), vocab_min_logits=vmin, vocab_max_logits=vmax)
        return loss, stat
    x, T, V, stride = _rows(logits)
    y = labels.to(device=dev, dtype=torch.int64).contiguous()
    old, adv = _f32(old_logprobs.detach()), _f32(advantages.detach())
    m8 = _mask_u8(loss_mask.to(dev))
    loss, logp, entropy, vmax, vmin, stat_loss, ratio, _flags = _FusedLogitsPpo.apply(
        x, y, stride, float(temperature), T_active, old, adv, m8, None, params, _count_nonzero(m8), scale_t, True,
        bool(inplace_backward),
    )
    logp_a = logp[:T_active]
    return loss, _sapo_stat(stat_loss, ratio, logp_a, old, adv, tau_pos, tau_neg,
                            dict(logprobs=logp_a, entropy=entropy[:T_active], vocab_min_logits=vmin[:T_active],
                                 vocab_max_logits=vmax[:T_active]))


def fused_lm_head_sapo_loss(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor,
                            old_logprobs: torch.Tensor, advantages: torch.Tensor, tau_pos: float, tau_neg: float,
                            loss_mask: torch.Tensor, temperature: float = 1.0,
                            loss_scale: torch.Tensor | float | None = None, skip_masked_tokens: bool = True,
                            kept_per_chunk: list[int] | None = None, backward: str = "carry") -> tuple[torch.Tensor, dict]:
    """lm_head + ``gather_logprobs_entropy`` + token-level ``sapo_loss_fn`` (+ backward) for one micro-batch, in token
    chunks whose logits are never written (``fused_lm_head_ppo_loss`` with the SAPO gate in place of the clip; the
    arguments they share mean the same)."""
    _require_gpu(hidden, "hidden")
    params = _sapo_params(tau_pos, tau_neg)
    if backward not in ("carry", "recompute"):
        raise ValueError(f"backward must be one of ['carry', 'recompute'], got {backward!r}")
    T_active = _check_fused_inputs(hidden, labels, loss_mask, "hidden")
    _check_per_token(loss_mask, old_logprobs=old_logprobs, advantages=advantages)
    if weight.ndim != 2 or hidden.shape[1] != weight.shape[1]:
        raise ValueError(f"expected hidden [T, H] and weight [V, H], got {tuple(hidden.shape)} and {tuple(weight.shape)}")
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("fused lm_head expects bf16 hidden states and weights")
    dev = hidden.device
    scale_t = _scale_tensor(loss_scale, dev)
    y = labels.to(device=dev, dtype=torch.int64).contiguous()
    if not (torch.is_grad_enabled() and (hidden.requires_grad or weight.requires_grad)):
        logp, entropy, vmin, vmax = (t[:T_active] for t in lm_head_logprobs_entropy_stats(hidden, weight, y, temperature))
        loss, stat = sapo_loss_fn(logp, old_logprobs, advantages, tau_pos, tau_neg, loss_mask)
        if scale_t is not None:
            loss = loss * scale_t.squeeze(0)
        stat.update(logprobs=logp.detach(), entropy=entropy.detach(), vocab_min_logits=vmin, vocab_max_logits=vmax)
        return loss, stat
    old, adv = _f32(old_logprobs.detach()), _f32(advantages.detach())
    m8 = _mask_u8(loss_mask.to(dev))
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
    loss, logp, entropy, stat_loss, ratio, _flags, vmax, vmin = _FusedLmHeadPpo.apply(
        hidden.contiguous(), weight.contiguous(), y, float(temperature), T_active, old, adv, m8, None, params,
        _count_nonzero(m8), scale_t, kept, 1 if backward == "carry" else 0,
    )
    logp_a = logp[:T_active]
    return loss, _sapo_stat(stat_loss, ratio, logp_a, old, adv, tau_pos, tau_neg,
                            dict(logprobs=logp_a, entropy=entropy[:T_active], vocab_min_logits=vmin[:T_active],
                                 vocab_max_logits=vmax[:T_active]))
