"""The engine-side call contract of the path, as a small harness.

Mirrors what FSDPEngine does around the functional ops for one packed
micro-batch (areal/engine/fsdp_engine.py:1908-1964, 1977-2046) and the part of
``grpo_loss_fn`` that feeds ``ppo_actor_loss_fn`` (areal/trainer/ppo/actor.py:408-480):
labels are the packed ``input_ids`` rolled by one over the WHOLE packed tensor,
the batch padding is trimmed after the log-prob op, entropy is detached, and the
loss is scaled by ``local_weight / total_loss_weight * loss_multiplier``.
"""
from __future__ import annotations

from typing import Any

import torch

from .advantages import gae_advantages, kl_regularized_rewards
from .functional import (
    fused_lm_head_ppo_loss,
    fused_logprobs_ppo_loss,
    gather_logprobs,
    gather_logprobs_entropy_stats,
    lm_head_chunk_tokens,
    lm_head_logprobs_entropy,
    lm_head_logprobs_entropy_stats,
    ppo_actor_loss_fn,
)


def rolled_labels(model_inputs: dict[str, Any]) -> torch.Tensor:
    """``rolled_input_ids`` if present, else ``roll(input_ids, -1)``; a leading batch dim of 1 is dropped
    (fsdp_engine.py:1915-1921).  The roll is over the packed tensor, not per sequence: the last token of a
    sequence is labelled with the first token of the next one and is expected to be masked out."""
    labels = model_inputs.get("rolled_input_ids")
    if labels is None:
        labels = torch.roll(model_inputs["input_ids"], shifts=-1, dims=-1)
    if labels.ndim == 2 and labels.shape[0] == 1:
        labels = labels.squeeze(0)
    return labels


def compute_logprobs(logits: torch.Tensor, model_inputs: dict[str, Any], temperature: float = 1.0) -> torch.Tensor:
    """Forward-only log-probs of a micro-batch (fsdp_engine.py:1938-1964)."""
    return gather_logprobs(logits, rolled_labels(model_inputs), temperature=temperature)


def compute_logprobs_and_loss(
    logits: torch.Tensor,
    model_inputs: dict[str, Any],
    mb_input: dict[str, Any],
    pad_length: int,
    total_loss_weight: torch.Tensor | float,
    eps_clip: float,
    eps_clip_higher: float | None = None,
    c_clip: float | None = None,
    rejection_sampling: Any | None = None,
    importance_sampling_level: str = "token",
    temperature: float = 1.0,
    loss_multiplier: float = 1.0,
    fused: bool = True,
    inplace_backward: bool = False,
    use_sapo_loss: bool = False,
    sapo_tau_pos: float = 1.0,
    sapo_tau_neg: float = 1.05,
) -> tuple[torch.Tensor, dict]:
    """Scaled PPO loss of one micro-batch and its stat dict (fsdp_engine.py:1977-2046 with
    ``loss_fn = grpo_loss_fn`` and ``loss_weight_fn = loss_mask.count_nonzero``, actor.py:345-364).

    ``logits`` is ``[T_pad, V]``; ``mb_input`` holds the un-padded ``[T]`` tensors ``loss_mask``, ``logprobs``
    (behaviour policy), ``prox_logp``, ``advantages`` and ``cu_seqlens``.  An all-masked micro-batch returns
    ``logits.mean() * 0`` like the reference (fsdp_engine.py:1988-1989).  ``inplace_backward``: the gradient is
    written over the logits, see ``fused_logprobs_ppo_loss``.  ``use_sapo_loss`` (token level, fused): the SAPO gate in
    place of the clip, on the behaviour log-probs (actor.py:448-462: SAPO takes ``old_logp``, no proximal policy).
    """
    loss_mask = mb_input["loss_mask"].bool()
    local_weight = loss_mask.count_nonzero()
    if local_weight == 0:
        return logits.mean() * 0.0, {}
    labels = rolled_labels(model_inputs)
    old_logp = mb_input["logprobs"]
    prox_logp = mb_input.get("prox_logp")
    if prox_logp is None and not use_sapo_loss:
        raise ValueError("prox_logp is None: only the recomputed proximal log-probs are supported here")
    scale = local_weight / total_loss_weight * loss_multiplier
    if use_sapo_loss and fused and importance_sampling_level == "token":
        from .sapo import fused_logprobs_sapo_loss

        return fused_logprobs_sapo_loss(logits, labels, old_logp, mb_input["advantages"], sapo_tau_pos, sapo_tau_neg,
                                        loss_mask, temperature=temperature, loss_scale=scale,
                                        inplace_backward=inplace_backward)
    if use_sapo_loss:
        raise ValueError("use_sapo_loss is built for the fused token-level call; use compute_loss_with(grpo_loss_fn) otherwise")
    kw = dict(
        eps_clip=eps_clip, eps_clip_higher=eps_clip_higher, c_clip=c_clip, rejection_sampling=rejection_sampling,
        importance_sampling_level=importance_sampling_level, cu_seqlens=mb_input.get("cu_seqlens"),
    )
    if fused:
        return fused_logprobs_ppo_loss(
            logits, labels, prox_logp, old_logp, mb_input["advantages"], loss_mask=loss_mask,
            temperature=temperature, loss_scale=scale, inplace_backward=inplace_backward, **kw,
        )
    logp, entropy, vmin, vmax = gather_logprobs_entropy_stats(logits, labels, temperature, inplace_backward)
    if pad_length > 0:
        logp, entropy, vmin, vmax = (t[:-pad_length] for t in (logp, entropy, vmin, vmax))
    loss, stat = ppo_actor_loss_fn(logp, prox_logp, old_logp, mb_input["advantages"], loss_mask=loss_mask, **kw)
    stat.update(logprobs=logp.detach(), entropy=entropy.detach(), vocab_min_logits=vmin, vocab_max_logits=vmax)
    return loss * scale, stat


def compute_lm_head_logprobs(hidden: torch.Tensor, weight: torch.Tensor, model_inputs: dict[str, Any],
                             temperature: float = 1.0, token_mask: torch.Tensor | None = None) -> torch.Tensor:
    """Forward-only log-probs of a micro-batch (fsdp_engine.py:1938-1964) from the final hidden states and the
    lm_head weight, without the ``[T_pad, V]`` logits.  ``token_mask`` (optional, beyond the reference's semantics):
    only these tokens go through the lm_head, the others get 0."""
    if hidden.ndim == 3 and hidden.shape[0] == 1:
        hidden = hidden.squeeze(0)
    return lm_head_logprobs_entropy(hidden, weight, rolled_labels(model_inputs), temperature, token_mask)[0]


def compute_lm_head_and_loss(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    model_inputs: dict[str, Any],
    mb_input: dict[str, Any],
    pad_length: int,
    total_loss_weight: torch.Tensor | float,
    eps_clip: float,
    eps_clip_higher: float | None = None,
    c_clip: float | None = None,
    rejection_sampling: Any | None = None,
    importance_sampling_level: str = "token",
    temperature: float = 1.0,
    loss_multiplier: float = 1.0,
    host_loss_mask: torch.Tensor | None = None,
    backward: str = "carry",
) -> tuple[torch.Tensor, dict]:
    """``compute_logprobs_and_loss`` (fsdp_engine.py:1977-2046) one step earlier in the model: from the final hidden
    states ``[T_pad, H]`` (a leading batch dimension of 1 is dropped, as ``outputs.logits.squeeze(0)``,
    fsdp_engine.py:747) and the lm_head weight ``[V, H]``, so that the ``[T_pad, V]`` logits are never written.

    Same contract otherwise: labels are the packed ``input_ids`` rolled by one over the whole tensor
    (``rolled_labels``), the last ``pad_length`` rows are batch padding (they get no gradient and no outputs), the loss
    is scaled by ``local_weight / total_loss_weight * loss_multiplier`` with ``local_weight =
    loss_mask.count_nonzero()`` (actor.py:363), and a micro-batch without any unmasked token returns a zero that keeps
    the graph to ``hidden`` and ``weight`` alive (fsdp_engine.py:1987-1989).  The stat dict is that of
    ``fused_logprobs_ppo_loss`` (``logprobs``, ``entropy``, ``vocab_min_logits``, ``vocab_max_logits`` and the entries
    of ``ppo_actor_loss_fn``), i.e. what ``grpo_loss_fn`` is given and returns.

    ``host_loss_mask``: the host (CPU) copy of ``mb_input["loss_mask"]`` that the data loader still holds.  With it
    nothing is read back from the device: the weight of the micro-batch and the number of tokens with a gradient per
    chunk of ``lm_head_chunk_tokens()`` tokens, which size the gradient GEMMs, are counted on the host.  Rejection
    sampling can only shrink the mask on the device; the counts are then upper bounds, and the rows beyond the true
    count are cleared on the device.  Without it the call reads them from the device, as the reference's
    ``local_weight == 0`` does.
    """
    if hidden.ndim == 3 and hidden.shape[0] == 1:
        hidden = hidden.squeeze(0)
    if hidden.ndim != 2 or hidden.shape[0] - pad_length != mb_input["loss_mask"].shape[0]:
        raise ValueError(
            f"hidden {tuple(hidden.shape)} with pad_length {pad_length} does not fit loss_mask "
            f"{tuple(mb_input['loss_mask'].shape)}"
        )
    loss_mask = mb_input["loss_mask"].bool()
    kept = None
    if host_loss_mask is not None:
        host = host_loss_mask.reshape(-1).ne(0)
        if host.is_cuda or host.shape[0] != loss_mask.shape[0]:
            raise ValueError("host_loss_mask must be the CPU copy of mb_input['loss_mask']")
        local_weight: Any = int(host.sum())
        chunk = lm_head_chunk_tokens()
        kept = [int(host[i:i + chunk].sum()) for i in range(0, hidden.shape[0], chunk)]
    else:
        local_weight = loss_mask.count_nonzero()
    if local_weight == 0:
        return hidden.mean() * 0.0 + weight.mean() * 0.0, {}
    old_logp = mb_input["logprobs"]
    prox_logp = mb_input.get("prox_logp")
    if prox_logp is None:
        raise ValueError("prox_logp is None: only the recomputed proximal log-probs are supported here")
    scale = local_weight / total_loss_weight * loss_multiplier
    return fused_lm_head_ppo_loss(
        hidden, weight, rolled_labels(model_inputs), prox_logp, old_logp, mb_input["advantages"], eps_clip=eps_clip,
        loss_mask=loss_mask, eps_clip_higher=eps_clip_higher, c_clip=c_clip, rejection_sampling=rejection_sampling,
        importance_sampling_level=importance_sampling_level, cu_seqlens=mb_input.get("cu_seqlens"),
        temperature=temperature, loss_scale=scale, kept_per_chunk=kept, backward=backward,
    )


def compute_advantages(
    data: dict[str, Any],
    *,
    kl_ctl: float = 0.0,
    kl_estimator: str = "k1",
    discount: float = 1.0,
    gae_lambda: float = 1.0,
    reward_bias: float = 0.0,
    reward_scaling: float = 1.0,
    reward_clip: float = 20.0,
    reward_norm: Any | None = None,
    adv_norm: Any | None = None,
    mask_no_eos_with_zero: bool = False,
    use_decoupled_loss: bool = False,
    recompute_logprob: bool = False,
    overlong_tokens: int | None = None,
    overlong_penalty_factor: float | None = None,
    max_new_tokens: int | None = None,
) -> dict[str, Any]:
    """``PPOActor._compute_advantages`` (areal/trainer/ppo/actor.py:145-250) on the GPU for one padded batch.

    ``data`` holds ``input_ids``, ``attention_mask``, ``loss_mask``, ``logprobs``, ``rewards`` as ``[bs, max_seqlen]``
    (``rewards`` is ``[bs]``) and optionally ``ref_logp``, ``values``, ``prox_logp``.  ``reward_norm`` / ``adv_norm``
    are ``Normalization`` objects or None.  Writes ``advantages``, ``returns``, ``kl_rewards``, ``tot_rewards``,
    the rolled ``loss_mask`` and ``logprobs`` back into ``data`` and returns it, as the reference does.  With
    ``overlong_tokens`` set (the reference's ``overlong_reward_penalty``), the length penalty of
    ``reward_overlong_penalty`` is applied to ``data["rewards"]`` first, in place (actor.py:152-164).
    """
    if overlong_tokens is not None:                                          # actor.py:152-164
        from .advantages import reward_overlong_penalty

        assert overlong_penalty_factor is not None and max_new_tokens is not None
        data = reward_overlong_penalty(data, overlong_tokens, overlong_penalty_factor, max_new_tokens)
    reward_score = (data["rewards"] + reward_bias) * reward_scaling          # actor.py:166-170
    reward_score = torch.clip(reward_score, max=reward_clip, min=-reward_clip)
    if reward_norm is not None:
        reward_score = reward_norm(reward_score)
    loss_mask = torch.roll(data["loss_mask"].float(), shifts=-1, dims=-1)    # :174-175
    if not use_decoupled_loss and recompute_logprob:                          # :177-186
        prox = data["prox_logp"]
        if prox is None:
            raise ValueError(
                "prox_logp is None but recompute_logprob=True. This indicates compute_logp() was skipped incorrectly."
            )
        old_logp = data["logprobs"] = prox
    else:
        old_logp = torch.roll(data["logprobs"], shifts=-1, dims=-1)          # :188
        if not use_decoupled_loss:
            data["prox_logp"] = old_logp
    # in place, as the reference does (:192-196): data["prox_logp"] (when it is this tensor) and data["ref_logp"]
    # come out masked as well
    old_logp.mul_(loss_mask)
    ref_logp = data.get("ref_logp")
    if ref_logp is not None:
        ref_logp.mul_(loss_mask)
    seqlens = data["attention_mask"].sum(-1).long()                           # :199-201
    rewards, kl_rewards = kl_regularized_rewards(old_logp, ref_logp, loss_mask, seqlens, reward_score, kl_ctl,
                                                 kl_estimator, mask_no_eos_with_zero)
    values = data.get("values")
    no_eos = seqlens == data["attention_mask"].shape[1]
    advantages, returns = gae_advantages(rewards, values, loss_mask, no_eos, discount, gae_lambda)   # :209-232
    data["returns"] = returns
    if adv_norm is not None:
        advantages = adv_norm(advantages, loss_mask)                          # :235-236
    data["advantages"] = advantages
    data["kl_rewards"] = kl_rewards
    data["tot_rewards"] = rewards
    data["loss_mask"] = loss_mask
    data["logprobs"] = old_logp
    return data


PROX_LOGP_METHOD_RECOMPUTE = "recompute"
PROX_LOGP_METHOD_LOGLINEAR = "loglinear"
PROX_LOGP_METHOD_METRICS = "metrics"


def infer_token_denominator(input_data: dict[str, Any], fallback: torch.Tensor) -> torch.Tensor:
    """All-true mask whose size is the number of logical tokens of the micro-batch, for the ``n_tokens``
    denominator of the logged statistics (areal/trainer/ppo/stats.py:10-40): the shape of ``attention_mask`` if
    that is a tensor, else ``cu_seqlens[-1]`` tokens, else the shape of ``input_ids`` when it matches ``fallback``,
    else the shape of ``fallback``."""
    common = dict(dtype=torch.bool, device=fallback.device)
    attention_mask = input_data.get("attention_mask")
    if isinstance(attention_mask, torch.Tensor):
        return torch.ones_like(attention_mask, **common)
    cu_seqlens = input_data.get("cu_seqlens")
    if isinstance(cu_seqlens, torch.Tensor) and cu_seqlens.numel() > 0:
        return torch.ones(int(cu_seqlens[-1].item()), **common)
    input_ids = input_data.get("input_ids")
    if isinstance(input_ids, torch.Tensor) and input_ids.shape == fallback.shape:
        return torch.ones_like(input_ids, **common)
    return torch.ones_like(fallback, **common)


def resolve_proximal_logp(prox_logp_gt, prox_logp_method: str, old_logp, logprobs, versions, current_version):
    """``_resolve_proximal_logp`` (areal/trainer/ppo/actor.py:687-765): the recomputed proximal log-probs when
    they are there, the log-linear approximation from per-token versions when the forward pass was skipped."""
    from .actor_ops import compute_prox_logp_approximations

    if prox_logp_method not in (PROX_LOGP_METHOD_RECOMPUTE, PROX_LOGP_METHOD_LOGLINEAR, PROX_LOGP_METHOD_METRICS):
        raise ValueError(f"'{prox_logp_method}' is not a valid ProxLogpMethod")
    if prox_logp_gt is None:
        if prox_logp_method != PROX_LOGP_METHOD_LOGLINEAR:  # the only method that skips the forward pass
            raise ValueError(
                f"prox_logp is None but prox_logp_method='{prox_logp_method}'. "
                "This indicates compute_logp() was skipped incorrectly."
            )
        if versions is None:
            raise ValueError(
                f"prox_logp is None with prox_logp_method='{prox_logp_method}' but versions not available. "
                "Cannot proceed without either ground truth or approximation."
            )
    prox_logp = prox_logp_gt
    if prox_logp_method == PROX_LOGP_METHOD_LOGLINEAR:
        if prox_logp_gt is None and versions is not None and current_version is not None:
            prox_logp = compute_prox_logp_approximations(old_logp, logprobs, versions, current_version,
                                                         method="loglinear")["loglinear"]
    if prox_logp is None:
        raise RuntimeError(
            f"prox_logp is None after handling prox_logp_method='{prox_logp_method}'. "
            "This indicates configuration or computation error."
        )
    return prox_logp


def grpo_loss_fn(
    logprobs: torch.Tensor,
    entropy: torch.Tensor,
    input_data: dict,
    eps_clip: float,
    eps_clip_higher: float | None,
    c_clip: float | None,
    rejection_sampling: Any | None = None,
    m2_threshold: float | None = None,
    importance_sampling_level: str = "token",
    current_version: int | None = None,
    prox_logp_method: str = PROX_LOGP_METHOD_RECOMPUTE,
    use_sapo_loss: bool = False,
    sapo_tau_pos: float = 1.0,
    sapo_tau_neg: float = 1.05,
    use_decoupled_loss: bool = False,
    vocab_min_logits: torch.Tensor | None = None,
    vocab_max_logits: torch.Tensor | None = None,
) -> tuple[torch.Tensor, dict]:
    """The actor's loss function for one micro-batch (areal/trainer/ppo/actor.py:408-480) on the GPU ops: proximal
    log-probs resolved, optional M2PO masking, SAPO or clipped PPO loss, and the joint-distillation terms
    (``teacher_logp`` with ``rl_loss_weight`` / ``distill_loss_weight``, actor.py:482-511).

    Returns ``(loss, stat)``.  ``stat`` is the per-token dict of the loss function plus ``"reduced"``: what the
    reference hands to its statistics tracker tensor by tensor (actor.py:513-573) as sums / averages / extrema
    under the same denominators, computed in one launch per denominator, and under ``"compute_logp"`` and
    ``"version_stats"`` what it logs in those scopes (actor.py:573-594, 982-1110; ``proximal_logging_stats``).
    """
    from .actor_ops import apply_m2po_masking, distillation_terms, proximal_logging_stats
    from .advantages import masked_moments
    from .functional import sapo_loss_fn

    old_logp = input_data["logprobs"]
    advantages = input_data["advantages"]
    loss_mask = input_data["loss_mask"].bool()
    entropy = entropy.detach()
    prox_logp = resolve_proximal_logp(input_data.get("prox_logp"), prox_logp_method, old_logp, logprobs.detach(),
                                      input_data.get("versions"), current_version)
    if m2_threshold is not None:
        loss_mask = apply_m2po_masking(old_logp, prox_logp, loss_mask, m2_threshold)
    if use_sapo_loss:
        if use_decoupled_loss:
            raise ValueError(
                "SAPO is not compatible with `use_decoupled_loss=True`. "
                "Please set `actor.use_decoupled_loss=false` in your configuration."
            )
        loss, stat = sapo_loss_fn(logprobs, old_logp, advantages, sapo_tau_pos, sapo_tau_neg, loss_mask,
                                  importance_sampling_level, input_data.get("cu_seqlens"))
    else:
        loss, stat = ppo_actor_loss_fn(logprobs, prox_logp, old_logp, advantages, eps_clip, loss_mask, eps_clip_higher,
                                       c_clip, rejection_sampling, importance_sampling_level,
                                       input_data.get("cu_seqlens"))
    rkl_stat = None
    teacher_logp = input_data.get("teacher_logp")
    if teacher_logp is not None:
        rl_loss_weight = input_data.get("rl_loss_weight", 1.0)
        distill_loss_weight = input_data.get("distill_loss_weight", 0.005)
        if rl_loss_weight == 0:  # pure distillation with the reverse KL as an importance-weighted reward
            mean, term = distillation_terms(logprobs, old_logp, teacher_logp, loss_mask, pure=True)
            loss = -distill_loss_weight * mean
            rkl_stat = -term
        else:                    # the RL loss plus a reverse-KL penalty
            mean, term = distillation_terms(logprobs, None, teacher_logp, loss_mask, pure=False)
            loss = rl_loss_weight * loss + distill_loss_weight * mean
            rkl_stat = term
    per_valid = dict(
        importance_weight=stat["importance_weight"], approx_kl=stat["approx_kl"], new_logp=logprobs.detach(),
        old_logp=old_logp, entropy=entropy.float(), actor_loss=stat["loss"], clip_ratio=stat["clip_mask"].float(),
        dual_clip_ratio=stat["dual_clip_mask"].float(),
    )
    if use_sapo_loss:
        per_valid.update(sapo_soft_gate=stat["sapo_soft_gate"], sapo_scaled_gate_pos=stat["sapo_scaled_gate_pos"],
                         sapo_scaled_gate_neg=stat["sapo_scaled_gate_neg"])
    if rkl_stat is not None:
        per_valid.update(rkl_loss=rkl_stat)
    reduced = masked_moments(per_valid, loss_mask)
    if not use_sapo_loss:
        clip_mask = stat["clip_mask"]
        reduced.update(masked_moments(dict(clipped_new_logp=logprobs.detach(), clipped_old_logp=old_logp), clip_mask))
    if "behave_imp_weight" in stat:
        reduced.update(masked_moments(dict(behave_imp_weight=stat["behave_imp_weight"],
                                           behave_approx_kl=stat["behave_approx_kl"]), stat["behave_mask"]))
    if "filtered_fraction" in stat:
        reduced["rs_filtered_fraction"] = stat["filtered_fraction"]
    if vocab_min_logits is not None and vocab_max_logits is not None:
        everything = torch.ones_like(loss_mask)
        reduced.update(masked_moments(dict(vocab_min_logits=vocab_min_logits, vocab_max_logits=vocab_max_logits),
                                      everything))
    reduced["n_tokens"] = infer_token_denominator(input_data, loss_mask).numel()
    # the compute_logp and version_stats scopes (actor.py:573-594) under the mask the loss kept
    reduced.update(proximal_logging_stats(old_logp, logprobs.detach(), input_data.get("prox_logp"),
                                          input_data.get("versions"), current_version,
                                          stat.get("behave_mask", loss_mask), prox_logp_method))
    stat = dict(stat, loss_mask=loss_mask, reduced=reduced)
    return loss, stat


def critic_loss_fn(value: torch.Tensor, input_data: dict[str, Any], eps_clip: float) -> tuple[torch.Tensor, dict]:
    """The critic's loss function for one micro-batch (areal/trainer/ppo/critic.py:105-149) on the GPU ops.

    Returns ``(loss, stat)`` with ``stat["reduced"]`` holding what the reference logs tensor by tensor (sums,
    averages, extrema under ``n_valid_tokens`` and ``clipped_tokens``) and ``n_tokens``."""
    from .advantages import masked_moments
    from .functional import ppo_critic_loss_fn

    value = value.squeeze(-1).float()
    old_value = input_data["values"].float()
    target_value = input_data["returns"].float()
    loss_mask = input_data["loss_mask"].bool()
    loss, stat = ppo_critic_loss_fn(value, old_value, target_value, eps_clip, loss_mask)
    clip_mask = stat["clip_mask"]
    reduced = masked_moments(dict(new_value=value.detach(), old_value=old_value, target_value=target_value,
                                  critic_loss=stat["loss"], clip_ratio=clip_mask.float()), loss_mask)
    reduced.update(masked_moments(dict(clipped_new_value=value.detach(), clipped_old_value=old_value), clip_mask))
    reduced["n_tokens"] = infer_token_denominator(input_data, value).numel()
    return loss, dict(stat, loss_mask=loss_mask, reduced=reduced)


def dpo_valid_pairs(x: dict[str, Any]) -> torch.Tensor:
    """Pairs whose chosen and rejected sequences are both non-empty (areal/trainer/dpo/dpo_engine.py:22-24)."""
    seqlens = x["cu_seqlens"][1:] - x["cu_seqlens"][:-1]
    return seqlens.view(-1, 2).ne(0).all(dim=1)


def dpo_loss_weight(x: dict[str, Any]) -> torch.Tensor:
    """Number of valid pairs as a float, the weight of a micro-batch (dpo_engine.py:27-28)."""
    return dpo_valid_pairs(x).count_nonzero().float()


def compute_dpo_loss(logprobs: torch.Tensor, entropy: torch.Tensor | None, input_: dict[str, Any], *, beta: float,
                     loss_type: str = "sigmoid", vocab_min_logits: torch.Tensor | None = None,
                     vocab_max_logits: torch.Tensor | None = None) -> tuple[torch.Tensor, dict]:
    """The DPO loss function of one packed micro-batch (dpo_engine.py:147-213) on the GPU ops.

    ``input_`` holds ``cu_seqlens``, ``loss_mask`` and ``ref_logprobs`` (``KeyError`` if one is missing), sequences
    interleaved chosen / rejected.  Returns ``(loss, stat)``: the mean over the valid pairs (0 when there are none,
    found on the device, without a read-back) and what the reference records per pair under its ``n_pairs``
    denominator: ``loss``, ``chosen_reward``, ``rejected_reward``, ``reward_accuracy``, ``reward_margin``, with
    ``valid_pairs`` selecting the pairs that count and ``n_pairs`` their number."""
    from .dpo import dpo_loss

    loss, stat = dpo_loss(logprobs, input_["ref_logprobs"], input_["cu_seqlens"], input_["loss_mask"], beta=beta,
                          loss_type=loss_type)
    with torch.no_grad():
        stat["reward_accuracy"] = (stat["chosen_reward"] > stat["rejected_reward"]).float()
        stat["reward_margin"] = stat["chosen_reward"] - stat["rejected_reward"]
    return loss, stat


def compute_packed_sft_loss(logprobs: torch.Tensor, entropy: torch.Tensor | None, input_: dict[str, Any],
                            vocab_min_logits: torch.Tensor | None = None,
                            vocab_max_logits: torch.Tensor | None = None) -> tuple[torch.Tensor, dict]:
    """The SFT loss function of one packed micro-batch (areal/trainer/sft/lm_engine.py:81-131) on the GPU ops.

    Returns ``(loss, stat)``; ``stat`` holds what the reference records: per token ``loss`` under ``n_valid_tokens``
    (= ``loss_mask``), per sequence ``ppl`` under ``n_seqs`` (the sequences with a selected token), and in
    ``stat["reduced"]`` the moments of ``loss`` and of the vocabulary extrema (under all tokens) when given."""
    from .advantages import masked_moments
    from .sft import sft_loss_fn

    del entropy  # SFT does not use entropy
    loss_mask = input_["loss_mask"].bool()
    loss, stat = sft_loss_fn(logprobs, loss_mask, input_["cu_seqlens"])
    reduced = masked_moments(dict(loss=stat["loss"]), loss_mask)
    if vocab_min_logits is not None and vocab_max_logits is not None:
        reduced.update(masked_moments(dict(vocab_min_logits=vocab_min_logits, vocab_max_logits=vocab_max_logits),
                                      torch.ones_like(loss_mask)))
    reduced["n_tokens"] = logprobs.shape[0]
    return loss, dict(stat, loss_mask=loss_mask, reduced=reduced)


def rw_valid_pairs(x: dict[str, Any]) -> torch.Tensor:
    """Pairs whose chosen and rejected sequences are both non-empty (areal/trainer/rw/rw_engine.py:20-22)."""
    return dpo_valid_pairs(x)


def rw_loss_weight(x: dict[str, Any]) -> torch.Tensor:
    """Number of valid pairs as a float (rw_engine.py:25-26)."""
    return rw_valid_pairs(x).count_nonzero().float()


def compute_rw_loss(scores: torch.Tensor, input_: dict[str, Any]) -> tuple[torch.Tensor, dict]:
    """The reward-model loss function of one packed micro-batch (rw_engine.py:115-146) on the GPU ops.  Returns
    ``(loss, stat)`` with what the reference records per pair under ``n_pairs``: ``loss``, ``pos_score``,
    ``neg_score``, ``correct_ratio``, selected by ``valid_pairs``."""
    from .dpo import rw_pair_loss

    loss, stat = rw_pair_loss(scores, input_["cu_seqlens"])
    with torch.no_grad():
        stat["correct_ratio"] = (stat["pos_score"] > stat["neg_score"]).float()
    return loss, stat


def compute_loss_with(logits: torch.Tensor, model_inputs: dict[str, Any], mb_input: dict[str, Any], pad_length: int,
                      loss_fn, loss_weight_fn, total_loss_weight: torch.Tensor | float, temperature: float = 1.0,
                      loss_multiplier: float = 1.0, is_critic: bool = False, trie_node: Any = None):
    """``_compute_logprobs_and_loss`` for any loss function (areal/engine/fsdp_engine.py:1977-2046): log-probs,
    entropy and the vocabulary extrema of the micro-batch in one pass over the logits (packed trees: through the
    tree gather), the batch padding trimmed, ``loss_fn(logprobs, entropy, mb_input, vocab_min_logits=...,
    vocab_max_logits=...)`` (a critic: ``loss_fn(values, mb_input)``), scaled by ``local_weight / total_loss_weight *
    loss_multiplier``.  ``loss_fn`` may return the loss alone, like the reference's, or ``(loss, stat)`` like the
    loss functions of this module; the return value has the same form.  A micro-batch of weight 0 returns
    ``logits.mean() * 0``."""
    local_weight = loss_weight_fn(mb_input)
    if local_weight == 0:
        return logits.mean() * 0.0
    if is_critic:
        if trie_node is not None:
            raise NotImplementedError("Tree training with critic model is not supported yet.")
        values = logits.squeeze(-1)
        if pad_length > 0:
            values = values[:-pad_length]
        out = loss_fn(values, mb_input)
    else:
        if trie_node is not None:
            from .tree import gather_packed_tree_logprobs_entropy, gather_packed_tree_vocab_stats

            if not trie_node.all_sequence_ids:
                return logits.mean() * 0.0
            vmin, vmax = gather_packed_tree_vocab_stats(logits, trie_node)
            logp, entropy = gather_packed_tree_logprobs_entropy(logits, trie_node, mb_input["input_ids"],
                                                                temperature=temperature)
        else:
            logp, entropy, vmin, vmax = gather_logprobs_entropy_stats(logits, rolled_labels(model_inputs), temperature)
            if pad_length > 0:
                logp, entropy, vmin, vmax = (t[:-pad_length] for t in (logp, entropy, vmin, vmax))
        out = loss_fn(logp, entropy, mb_input, vocab_min_logits=vmin, vocab_max_logits=vmax)
    scale = local_weight / total_loss_weight * loss_multiplier
    if isinstance(out, tuple):
        return out[0] * scale, out[1]
    return out * scale


def compute_lm_head_loss_with(hidden: torch.Tensor, weight: torch.Tensor, model_inputs: dict[str, Any],
                              mb_input: dict[str, Any], pad_length: int, loss_fn, loss_weight_fn,
                              total_loss_weight: torch.Tensor | float, temperature: float = 1.0,
                              loss_multiplier: float = 1.0, backward: str = "carry",
                              grad_token_mask: torch.Tensor | None = None, kept_per_chunk: list[int] | None = None):
    """``compute_loss_with`` one step earlier in the model: any loss function of the reference's form
    (``grpo_loss_fn`` with sequence-level ratios, SAPO, M2PO or distillation terms, ``compute_packed_sft_loss``, a custom
    one) on the final hidden states ``[T_pad, H]`` and the lm_head weight ``[V, H]``, without the ``[T_pad, V]`` logits:
    log-probs, entropy and the vocabulary extrema come from ``lm_head_logprobs_entropy_stats``, the batch padding is
    trimmed, ``loss_fn(logprobs, entropy, mb_input, vocab_min_logits=..., vocab_max_logits=...)`` is called as the
    engine calls it (fsdp_engine.py:2032-2040) and its result scaled by ``local_weight / total_loss_weight *
    loss_multiplier``.  A micro-batch of weight 0 returns a zero that keeps the graph to ``hidden`` and ``weight``.

    ``backward="carry"`` (default): the op keeps the bf16 probability ratios of the tokens named by ``grad_token_mask``
    (default: ``mb_input["loss_mask"]``; tokens outside it get no gradient) from its forward to its backward, which is
    then two GEMMs instead of three; ``kept_per_chunk``: their number per chunk of ``lm_head_chunk_tokens()`` tokens,
    if the host knows it (else it is read back).  ``"recompute"`` keeps nothing and forms the logits again."""
    if hidden.ndim == 3 and hidden.shape[0] == 1:
        hidden = hidden.squeeze(0)
    local_weight = loss_weight_fn(mb_input)
    if local_weight == 0:
        return hidden.mean() * 0.0 + weight.mean() * 0.0
    if grad_token_mask is None and backward == "carry":
        grad_token_mask = mb_input.get("loss_mask")
    if grad_token_mask is not None:
        grad_token_mask = grad_token_mask.reshape(-1).ne(0)
        if pad_length > 0:
            grad_token_mask = torch.nn.functional.pad(grad_token_mask, (0, hidden.shape[0] - grad_token_mask.shape[0]))
    logp, entropy, vmin, vmax = lm_head_logprobs_entropy_stats(
        hidden, weight, rolled_labels(model_inputs), temperature, backward=backward,
        grad_token_mask=grad_token_mask if backward == "carry" else None,
        kept_per_chunk=kept_per_chunk if backward == "carry" else None)
    if pad_length > 0:
        logp, entropy, vmin, vmax = (t[:-pad_length] for t in (logp, entropy, vmin, vmax))
    out = loss_fn(logp, entropy, mb_input, vocab_min_logits=vmin, vocab_max_logits=vmax)
    scale = local_weight / total_loss_weight * loss_multiplier
    if isinstance(out, tuple):
        return out[0] * scale, out[1]
    return out * scale


def compute_logprobs_and_sft_loss(logits: torch.Tensor, model_inputs: dict[str, Any], mb_input: dict[str, Any],
                                  total_loss_weight: torch.Tensor | float, temperature: float = 1.0,
                                  loss_multiplier: float = 1.0) -> tuple[torch.Tensor, dict]:
    """The supervised step of one micro-batch in one pass over the logits: what ``compute_loss_with`` does with
    ``loss_fn = compute_packed_sft_loss`` and ``loss_weight_fn = loss_mask.count_nonzero``
    (areal/trainer/sft/lm_engine.py:28-35), fused with the log-prob op and its backward.  ``mb_input`` holds the
    un-padded ``loss_mask`` and ``cu_seqlens``; the rows of ``logits`` past them are the batch padding."""
    from .sft import fused_logprobs_sft_loss

    loss_mask = mb_input["loss_mask"].bool()
    local_weight = loss_mask.count_nonzero()
    if local_weight == 0:
        return logits.mean() * 0.0, {}
    scale = local_weight / total_loss_weight * loss_multiplier
    return fused_logprobs_sft_loss(logits, rolled_labels(model_inputs), loss_mask, mb_input["cu_seqlens"], temperature,
                                   loss_scale=scale)
