"""Oracle of the PPO actor loss and of rejection sampling (test infrastructure, CPU only).

Follows areal/utils/functional/functional.py:
  :56-149   sequence-level (GSPO) ratio and advantages
  :167-182  bound check
  :185-426  apply_rejection_sampling
  :429-559  ppo_actor_loss_fn
and areal/utils/data.py:1620-1656 (KL estimators k1/k2/k3, no clamping).

Sequences are walked with explicit Python loops over ``cu_seqlens`` (or over the
rows of a 2-D tensor) rather than scatter ops: slower, but each segment's sum,
mean and max is then the textbook definition.  The loss itself is written with
the same PyTorch ops as the reference (clamp, max, min, sign, where) so that
autograd of this oracle carries the reference's tie conventions.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch


@dataclass
class RejectionSamplingOutput:
    loss_mask: torch.Tensor
    behave_imp_weight: torch.Tensor
    filtered_fraction: float


def _segments(shape, cu_seqlens) -> list[tuple[int, int]]:
    """Flat [begin, end) index ranges of the sequences of a packed 1-D or padded 2-D tensor."""
    if len(shape) == 1:
        bounds = [int(v) for v in cu_seqlens.tolist()]
        return list(zip(bounds[:-1], bounds[1:]))
    rows, width = shape
    return [(r * width, (r + 1) * width) for r in range(rows)]


def kl_estimate(log_probs: torch.Tensor, log_probs_base: torch.Tensor, estimator: str) -> torch.Tensor:
    """k1 / k2 / k3 estimators of KL(new || base) per token; data.py:1620-1656, apply_clamp=False."""
    d = log_probs.float() - log_probs_base.float()
    if estimator == "k1":
        return d
    if estimator == "k2":
        return d**2 / 2.0
    if estimator == "k3":
        nd = -d
        return nd.exp() - 1 - nd
    raise ValueError(f"Invalid KL estimator: {estimator}")


def _within(metric: torch.Tensor, cfg: Any) -> torch.Tensor:
    """functional.py:167-182"""
    ok = metric <= cfg.upper
    if cfg.lower is not None:
        ok = ok & (metric >= cfg.lower)
    return ok


def rejection_sampling(
    proximal_logprobs: torch.Tensor,
    old_logprobs: torch.Tensor,
    loss_mask: torch.Tensor,
    cu_seqlens: torch.Tensor | None,
    cfg: Any,
) -> RejectionSamplingOutput:
    """functional.py:185-426"""
    if proximal_logprobs.shape != old_logprobs.shape:
        raise ValueError(f"proximal_logprobs shape {proximal_logprobs.shape} != old_logprobs shape {old_logprobs.shape}")
    if proximal_logprobs.shape != loss_mask.shape:
        raise ValueError(f"proximal_logprobs shape {proximal_logprobs.shape} != loss_mask shape {loss_mask.shape}")
    if proximal_logprobs.ndim not in (1, 2):
        raise ValueError(f"Expected 1D (packed) or 2D (padded) tensors, got ndim={proximal_logprobs.ndim}")
    shape = proximal_logprobs.shape
    prox = proximal_logprobs.detach().float().reshape(-1)
    old = old_logprobs.detach().float().reshape(-1)
    valid = loss_mask.reshape(-1) != 0

    log_ratio = prox - old                                    # :231
    log_ratio = torch.where(torch.isfinite(log_ratio), log_ratio, torch.zeros_like(log_ratio))  # :233
    if cfg.metric == "ratio":                                 # :236-249
        metric = log_ratio.exp()
    elif cfg.metric in ("kl_k1", "kl_k2", "kl_k3"):
        metric = kl_estimate(prox, old, cfg.metric[3:])
    else:
        raise ValueError(f"Unknown metric: {cfg.metric}")
    weight = log_ratio.exp()                                  # :252
    unclamped = weight.clone()
    lo = cfg.lower if cfg.lower is not None else 0.0
    in_bounds = torch.ones_like(valid)

    if cfg.level == "sequence":
        if len(shape) == 1 and cu_seqlens is None:
            raise ValueError("cu_seqlens is required for 1D packed tensors in sequence-level filtering.")
        geometric = cfg.metric == "ratio"                     # :262 aggregate the ratio in log space
        source = log_ratio if geometric else metric
        for a, b in _segments(shape, cu_seqlens):
            v = valid[a:b]
            n_valid = int(v.sum())
            picked = source[a:b][v]
            total = picked.sum() if n_valid else torch.zeros((), dtype=source.dtype)
            if geometric:                                     # :290-297 uniform weight = geometric mean
                weight[a:b] = (total / max(n_valid, 1)).exp()
                unclamped[a:b] = weight[a:b]
            if cfg.agg == "sum":
                agg = total
            elif cfg.agg == "mean":
                agg = total / max(n_valid, 1)
            elif cfg.agg == "max":                            # :308-323 an all-masked sequence counts as 0
                agg = picked.max() if n_valid else torch.zeros((), dtype=source.dtype)
            else:
                raise ValueError(f"Unknown agg method: {cfg.agg}")
            seq_metric = agg.exp() if geometric else agg      # :328
            ok = bool(_within(seq_metric, cfg))
            if cfg.action == "mask":
                in_bounds[a:b] = ok
            elif not ok:                                      # :336-346 clamp only out-of-bounds sequences
                weight[a:b] = weight[a:b].clamp(min=lo, max=cfg.upper)
    else:
        if cfg.action == "mask":                              # :393-394
            in_bounds = _within(metric, cfg)
        else:                                                 # :397-400
            weight = weight.clamp(min=lo, max=cfg.upper)

    if cfg.action == "mask":                                  # :403-408
        kept = valid & in_bounds
        new_mask = kept.to(loss_mask.dtype).reshape(shape)
        hit = int((valid & ~in_bounds).sum())
    else:                                                     # :409-417
        kept = valid
        new_mask = loss_mask
        hit = int((valid & (unclamped != weight)).sum())
    fraction = hit / max(int(valid.sum()), 1)
    weight = torch.where(kept, weight, torch.zeros_like(weight))  # :420
    return RejectionSamplingOutput(new_mask, weight.reshape(shape), fraction)


def sequence_level_ratio_and_advantages(log_ratio, advantages, loss_mask, cu_seqlens):
    """GSPO: per-sequence exp(mean masked log-ratio) and mean masked advantage, broadcast to the
    sequence's valid tokens, zero elsewhere; functional.py:56-149.  Differentiable in log_ratio."""
    shape = log_ratio.shape
    if len(shape) == 1 and cu_seqlens is None:
        raise ValueError("cu_seqlens is required for 1D tensors (packed format).")
    flat_lr = log_ratio.reshape(-1)
    flat_adv = advantages.reshape(-1)
    valid = loss_mask.reshape(-1)
    ratio_parts, adv_parts = [], []
    for a, b in _segments(shape, cu_seqlens):
        v = valid[a:b]
        count = max(int(v.sum()), 1)
        mean_lr = torch.where(v, flat_lr[a:b], torch.zeros_like(flat_lr[a:b])).sum() / count
        mean_adv = torch.where(v, flat_adv[a:b], torch.zeros_like(flat_adv[a:b])).sum() / count
        ratio_parts.append(torch.where(v, mean_lr.exp().expand(b - a), torch.zeros(b - a, dtype=flat_lr.dtype)))
        adv_parts.append(torch.where(v, mean_adv.expand(b - a), torch.zeros(b - a, dtype=flat_adv.dtype)))
    covered = sum(b - a for a, b in _segments(shape, cu_seqlens))
    assert covered == flat_lr.numel(), "cu_seqlens must cover every token"
    return torch.cat(ratio_parts).reshape(shape), torch.cat(adv_parts).reshape(shape)


def ppo_actor_loss(
    logprobs: torch.Tensor,
    proximal_logprobs: torch.Tensor,
    old_logprobs: torch.Tensor,
    advantages: torch.Tensor,
    eps_clip: float,
    loss_mask: torch.Tensor,
    eps_clip_higher: float | None = None,
    c_clip: float | None = None,
    rejection_sampling_cfg: Any | None = None,
    importance_sampling_level: str = "token",
    cu_seqlens: torch.Tensor | None = None,
):
    """(loss, stat) of the decoupled clipped PPO objective; functional.py:429-559."""
    denom = int(loss_mask.count_nonzero()) or 1               # :483 counted before the mask is edited
    stat_extra = {}
    behave_w = None
    if rejection_sampling_cfg is not None:                    # :486-497
        rs = rejection_sampling(proximal_logprobs, old_logprobs, loss_mask, cu_seqlens, rejection_sampling_cfg)
        loss_mask, behave_w = rs.loss_mask, rs.behave_imp_weight
        stat_extra["filtered_fraction"] = rs.filtered_fraction

    if importance_sampling_level == "sequence":               # :501-506
        ratio, advantages = sequence_level_ratio_and_advantages(
            logprobs - proximal_logprobs, advantages, loss_mask, cu_seqlens
        )
    elif importance_sampling_level == "token":                # :509
        ratio = torch.where(loss_mask, torch.exp(logprobs - proximal_logprobs), 0)
    else:
        raise ValueError(
            f"Invalid importance_sampling_level: {importance_sampling_level}. Must be 'token' or 'sequence'."
        )

    upper = 1.0 + (eps_clip if eps_clip_higher is None else eps_clip_higher)
    clipped = torch.clamp(ratio, 1.0 - eps_clip, upper)       # :516-520
    unclipped_term = -advantages * ratio                      # :522
    clipped_term = -advantages * clipped                      # :523
    clip_mask = unclipped_term.detach() < clipped_term.detach()
    per_token = torch.max(unclipped_term, clipped_term)       # :525
    if c_clip is not None:                                    # :526-530
        assert c_clip > 1.0, c_clip
        cap = torch.sign(advantages) * c_clip * advantages
        dual_mask = cap.detach() < per_token.detach()
        per_token = torch.min(per_token, cap)
    else:
        dual_mask = torch.zeros_like(clip_mask)
    if behave_w is not None:                                  # :535-539
        behave_mask = (behave_w > 0) & loss_mask.bool()
        stat_extra["behave_approx_kl"] = torch.where(
            behave_mask, (proximal_logprobs - old_logprobs).detach(), 0.0
        )
        stat_extra["behave_imp_weight"] = behave_w
        stat_extra["behave_mask"] = behave_mask
        per_token = per_token * behave_w
    loss = torch.where(loss_mask, per_token, 0).sum() / denom  # :542
    stat = dict(
        loss=per_token.detach(),
        importance_weight=ratio.detach(),
        approx_kl=(logprobs - proximal_logprobs).detach(),
        clip_mask=clip_mask & loss_mask,
        dual_clip_mask=dual_mask & loss_mask,
    )
    stat.update(stat_extra)
    return loss, stat
