"""CPU oracle of the sibling losses and actor-side filters.  TEST INFRASTRUCTURE ONLY.

Restates in plain PyTorch on the CPU: ``sapo_loss_fn`` (areal/utils/functional/functional.py:562-638),
``ppo_critic_loss_fn`` (functional.py:694-778), ``compute_prox_logp_approximations``
(areal/trainer/ppo/actor.py:604-684) and ``_apply_m2po_masking`` / ``_get_m2po_loss_mask`` (actor.py:769-850).
How each function is pinned is listed in ``oracle/PINNING.md``.
"""
from __future__ import annotations

import torch

from .ppo import sequence_level_ratio_and_advantages


def sapo_loss(logprobs, old_logprobs, advantages, tau_pos, tau_neg, loss_mask, importance_sampling_level="token",
              cu_seqlens=None):
    """(loss, stat); functional.py:589-638."""
    if tau_pos <= 0 or tau_neg <= 0:
        raise ValueError("SAPO temperatures (tau_pos, tau_neg) must be positive.")
    count = int(loss_mask.count_nonzero()) or 1                                   # :591
    advantages = advantages.detach()
    log_ratio = logprobs - old_logprobs                                           # :593
    if importance_sampling_level == "sequence":                                   # :595-598
        ratio, advantages = sequence_level_ratio_and_advantages(log_ratio, advantages, loss_mask, cu_seqlens)
    elif importance_sampling_level == "token":
        ratio = torch.exp(log_ratio)                                              # :600
    else:
        raise ValueError(
            f"Invalid importance_sampling_level: {importance_sampling_level}. Must be 'token' or 'sequence'."
        )
    gate_pos = torch.sigmoid(tau_pos * (ratio - 1.0))                             # :608-609
    gate_neg = torch.sigmoid(tau_neg * (ratio - 1.0))
    scaled_gate_pos = gate_pos * (4.0 / tau_pos)                                  # :610-613
    scaled_gate_neg = gate_neg * (4.0 / tau_neg)
    soft_gate = torch.where(advantages > 0, scaled_gate_pos, scaled_gate_neg)     # :616-617
    pg_loss = -soft_gate * advantages                                             # :620
    logging_loss = pg_loss.detach()
    pg_loss = torch.where(loss_mask, pg_loss, 0).sum() / count                    # :622
    stat = dict(
        loss=logging_loss,
        importance_weight=ratio.detach(),
        approx_kl=log_ratio.detach(),
        clip_mask=torch.zeros_like(loss_mask, dtype=torch.bool),
        dual_clip_mask=torch.zeros_like(loss_mask, dtype=torch.bool),
        sapo_soft_gate=soft_gate.detach(),
        sapo_scaled_gate_pos=scaled_gate_pos.detach(),
        sapo_scaled_gate_neg=scaled_gate_neg.detach(),
    )
    return pg_loss, stat


def _huber(x, y, delta):
    diff = torch.abs(x - y)                                                       # :695-696
    return torch.where(diff < delta, 0.5 * diff**2, delta * (diff - 0.5 * delta))


def critic_loss(value, old_value, target_value, value_eps_clip, loss_mask=None, loss_fn_type="mse"):
    """(loss, stat); functional.py:733-778."""
    if loss_fn_type == "huber":
        fn = lambda x, y: _huber(x, y, 10.0)                                      # :739
    elif loss_fn_type == "mse":
        fn = lambda x, y: 0.5 * (x - y) ** 2                                      # :699-700
    else:
        raise NotImplementedError(f"Unknown loss fn type: {loss_fn_type}")
    original = fn(value, target_value)                                            # :749
    value_clipped = old_value + (value - old_value).clamp(-value_eps_clip, value_eps_clip)   # :751-753
    clipped = fn(value_clipped, target_value)                                     # :755
    value_loss = torch.max(original, clipped)                                     # :757
    clip_mask = clipped.detach() > original.detach()                              # :760
    if loss_mask is not None:
        clip_mask = clip_mask & loss_mask
    stat = dict(clip_mask=clip_mask, loss=value_loss.detach())
    if loss_mask is not None:
        value_loss = torch.where(loss_mask, value_loss, 0).sum() / loss_mask.count_nonzero()  # :768-770
    else:
        value_loss = value_loss.mean()
    return value_loss, stat


def prox_logp_approximations(old_logp, logprobs, versions, current_version, method=None):
    """{method: tensor}; actor.py:630-684."""
    v_proximal = current_version - 1
    v_behave = versions.float()
    v_theta = float(current_version)
    generated = versions >= 0
    version_diff = v_theta - v_behave
    version_gap = v_proximal - v_behave
    alpha = torch.where((version_diff > 0) & generated, version_gap / version_diff, torch.zeros_like(v_behave))
    alpha = torch.clamp(alpha, 0.0, 1.0)
    out = {}
    for m in ([method] if method else ["loglinear", "linear", "rollout"]):
        if m == "loglinear":
            out[m] = old_logp + alpha * (logprobs - old_logp)
        elif m == "linear":
            out[m] = torch.log((1 - alpha) * torch.exp(old_logp) + alpha * torch.exp(logprobs) + 1e-10)
        elif m == "rollout":
            out[m] = old_logp.clone()
    return out


def m2po_sorted_mask(sorted_m2, m2_threshold):
    """actor.py:813-850 on values sorted in descending order."""
    n = sorted_m2.numel()
    if n == 0:
        return torch.ones_like(sorted_m2, dtype=torch.bool)
    suffix_sums = sorted_m2.flip(0).cumsum(0).flip(0)
    counts = torch.arange(n, 0, -1, dtype=sorted_m2.dtype)
    avg = suffix_sums / counts
    below = torch.where(avg < m2_threshold)[0]
    num_to_mask = int(below[0]) if len(below) > 0 else n - 1
    mask = torch.ones_like(sorted_m2, dtype=torch.bool)
    if num_to_mask > 0:
        mask[:num_to_mask] = False
    return mask


def m2po_mask(old_logp, prox_logp, loss_mask, m2_threshold):
    """actor.py:769-810; equal values are dropped in index order (a stable sort)."""
    delta = old_logp - prox_logp
    m2 = delta * delta
    mask_flat = loss_mask.reshape(-1)
    selected = m2.reshape(-1)[mask_flat]
    if selected.numel() == 0:
        return loss_mask
    sorted_m2, indices = torch.sort(selected, descending=True, stable=True)
    restored = torch.argsort(indices)
    sel_mask = m2po_sorted_mask(sorted_m2, m2_threshold)[restored]
    full = torch.zeros_like(mask_flat, dtype=torch.bool)
    full[mask_flat] = sel_mask
    return full.view_as(loss_mask)


def distillation_loss(loss, logprobs, old_logp, teacher_logp, loss_mask, rl_loss_weight=1.0, distill_loss_weight=0.005):
    """``(loss, rkl_stat)`` after the joint-distillation branch of ``grpo_loss_fn``; actor.py:482-511."""
    teacher_logp = teacher_logp.detach()                                          # :489-491
    if rl_loss_weight == 0:                                                       # :493
        rkl_reward = teacher_logp - logprobs.detach()                             # :495
        importance_weight = torch.exp(logprobs - old_logp)                        # :496
        rkl_weighted_term = importance_weight * rkl_reward * loss_mask            # :498
        kd_coef = -1 * distill_loss_weight                                        # :500
        loss = kd_coef * rkl_weighted_term.sum() / loss_mask.sum().clamp(min=1)   # :501
        return loss, -1 * rkl_weighted_term                                       # :503
    rkl_penalty_per_token = (logprobs - teacher_logp) * loss_mask                 # :506
    rkl_penalty = rkl_penalty_per_token.sum() / loss_mask.sum().clamp(min=1)      # :507
    loss = rl_loss_weight * loss + distill_loss_weight * rkl_penalty              # :509
    return loss, rkl_penalty_per_token                                            # :511


_EPSILON = 1e-8   # actor.py:856


def approximation_errors(ground_truth, approximation):
    """abs / rel / squared error; actor.py:867-886."""
    diff = ground_truth - approximation
    return dict(abs_error=torch.abs(diff).float(),
                rel_error=torch.abs(diff / (torch.abs(ground_truth) + _EPSILON)).float(),
                squared_error=(diff * diff).float())


def proximal_logging_tensors(old_logp, logprobs, prox_logp_gt, versions, current_version, mask,
                             prox_logp_method="recompute"):
    """The per-token tensors the reference hands to its statistics tracker in the ``compute_logp`` and
    ``version_stats`` scopes, before any reduction; actor.py:908-979 (one method), :982-1064 (which methods, the KL
    estimators), :1067-1110 (staleness).  Returns ``(compute_logp, staleness)``: ``{name: tensor}`` to be reduced
    over ``mask``, and ``{name: 1-D tensor of the selected generated tokens}`` (empty dict when the reference logs
    nothing)."""
    out = {}
    if prox_logp_gt is not None:                                                   # :1002-1006
        out["prox_logp_gt"] = prox_logp_gt.float()
    staleness = {}
    if versions is None or current_version is None:                                # :1009-1010
        return out, staleness

    def one_method(name, approx, gt):
        behave = torch.exp(approx - old_logp).float()                              # :924
        imp = torch.exp(logprobs - approx).float()                                 # :925
        out.update({f"{name}/approx_logp": approx.float(), f"{name}/behave_imp_weight": behave,
                    f"{name}/importance_weight": imp})
        if gt is not None:                                                         # :934-968
            for k, v in approximation_errors(gt, approx).items():
                out[f"{name}/{k}"] = v
            b = approximation_errors(torch.exp(gt - old_logp).float(), behave)
            i = approximation_errors(torch.exp(logprobs - gt).float(), imp)
            out[f"{name}/behave_imp_weight_abs_error"] = b["abs_error"]
            out[f"{name}/behave_imp_weight_rel_error"] = b["rel_error"]
            out[f"{name}/importance_weight_abs_error"] = i["abs_error"]
            out[f"{name}/importance_weight_rel_error"] = i["rel_error"]

    if prox_logp_method == "loglinear":                                            # :1012-1028
        for name, approx in prox_logp_approximations(old_logp, logprobs, versions, current_version,
                                                     "loglinear").items():
            one_method(name, approx, None)
    elif prox_logp_method == "metrics" and prox_logp_gt is not None:               # :1030-1046
        for name, approx in prox_logp_approximations(old_logp, logprobs, versions, current_version, None).items():
            one_method(name, approx, prox_logp_gt)
    log_ratio = (logprobs.float() - old_logp.float()).detach()                     # :1049
    out["kl_div_direct"] = -log_ratio                                              # :1053-1055
    out["kl_div_taylor"] = log_ratio ** 2 / 2.0
    out["kl_div_dual"] = log_ratio.exp() - 1 - log_ratio
    valid_generated = mask.bool() & (versions >= 0)                                # :1088
    if valid_generated.any():
        v_behave = versions.float()
        staleness = dict(sample_staleness_proximal=((current_version - 1) - v_behave)[valid_generated],
                         sample_staleness_theta=(current_version - v_behave)[valid_generated])
    return out, staleness
