"""CPU oracle of the advantage pipeline: GAE, Normalization, masked moments.  TEST INFRASTRUCTURE ONLY.

Restates, in plain PyTorch on the CPU,
  * the GAE loop of ``PPOActor._compute_advantages`` (areal/trainer/ppo/actor.py:209-236),
  * ``Normalization`` (areal/utils/data.py:1378-1596) for one process (no all-reduce),
  * the masked reductions of the statistics tracker (areal/utils/stats_tracker.py:227-285).
How each function is pinned is listed in ``oracle/PINNING.md``.
"""
from __future__ import annotations

import torch


def gae(rewards, values, loss_mask, seq_no_eos_mask, discount: float, gae_lambda: float):
    """(advantages, returns) for padded ``[bs, L]`` float tensors; actor.py:209-236, statement by statement."""
    bs, max_seqlen = rewards.shape
    advantages_reversed = [torch.zeros(bs, dtype=torch.float32)]          # :216-218
    lastgaelam = 0                                                        # :219
    nextvalues = values[:, max_seqlen - 1] * seq_no_eos_mask              # :220
    for t in reversed(range(max_seqlen - 1)):                             # :221
        delta = rewards[:, t] + discount * nextvalues - values[:, t]      # :222
        newgaelam = delta + discount * gae_lambda * lastgaelam            # :223
        mask = loss_mask[:, t]                                            # :226
        nextvalues = nextvalues * (1 - mask) + values[:, t] * mask        # :227
        lastgaelam = lastgaelam * (1 - mask) + newgaelam * mask           # :228
        advantages_reversed.append(lastgaelam)                            # :229
    advantages = torch.stack(advantages_reversed[::-1], dim=1)            # :231
    return advantages, advantages + values                                # :232


def _compute_mean(x, mask, high_precision: bool, leave_one_out: bool):
    """data.py:1506-1557 without the all-reduce."""
    dtype = torch.float64 if high_precision else torch.float32
    x = x.to(dtype)
    dim = tuple(range(x.dim()))
    if mask is None:
        factor = torch.tensor(float(x.numel()), dtype=dtype)
        x_masked = x
        x_sum = x.sum(dim=dim, keepdim=True)
    else:
        mask = mask.to(dtype)
        x_masked = x * mask
        factor = mask.sum(dim, keepdim=True)
        x_sum = x_masked.sum(dim=dim, keepdim=True)
    if leave_one_out:
        if factor.item() <= 1:
            return torch.zeros_like(x_sum)
        if mask is None:
            return (x_sum.expand_as(x) - x) / (factor - 1)
        regular = x_sum / factor
        loo = (x_sum.expand_as(x) - x_masked) / torch.clamp(factor - mask, min=1.0)
        return torch.where(mask > 0, loo, regular.expand_as(x))
    if factor.item() == 0:
        return torch.zeros_like(x_sum)
    return x_sum / factor


def _compute_std(x, mask, mean, unbiased: bool, high_precision: bool):
    """data.py:1559-1596 without the all-reduce."""
    dtype = torch.float64 if high_precision else torch.float32
    x = x.to(dtype)
    mean = mean.to(dtype)
    dim = tuple(range(x.dim()))
    if mask is None:
        factor = torch.tensor(float(x.numel()), dtype=dtype)
        x_sum_sq = ((x - mean) ** 2).sum(dim=dim, keepdim=True)
    else:
        mask = mask.to(dtype)
        factor = mask.sum(dim, keepdim=True)
        x_sum_sq = ((x * mask - mean * mask) ** 2).sum(dim=dim, keepdim=True)
    if unbiased:
        if factor.item() <= 1:
            return torch.ones_like(x_sum_sq)
        return (x_sum_sq / (factor - 1)).sqrt()
    if factor.item() == 0:
        return torch.ones_like(x_sum_sq)
    return (x_sum_sq / factor).sqrt()


def normalization(x, loss_mask=None, mean_level="batch", mean_leave1out=False, std_level="batch", std_unbiased=True,
                  eps: float = 1e-5, group_size: int = 1, high_precision: bool = True):
    """``Normalization(NormConfig(...))(x, loss_mask)``; data.py:1395-1504."""
    bs = x.size(0)
    if loss_mask is not None and loss_mask.sum().item() == 0:             # :1407-1408
        return x.float()
    if mean_level == "batch":                                             # :1411-1420
        mean = _compute_mean(x, loss_mask, high_precision, mean_leave1out).expand_as(x)
    elif mean_level == "group":                                           # :1421-1444
        mean = torch.zeros_like(x)
        for i in range(0, bs // group_size):
            s = slice(i * group_size, (i + 1) * group_size)
            xx = x[s]
            m = loss_mask[s] if loss_mask is not None else None
            if group_size == 1 and mean_leave1out:
                group_mean = torch.zeros((1, *xx.shape[1:]), dtype=torch.float64 if high_precision else torch.float32)
            else:
                group_mean = _compute_mean(xx, m, high_precision, mean_leave1out)
            mean[s] = group_mean.expand_as(xx)
    else:
        mean = torch.zeros_like(x)                                        # :1446
    x_centered = x - mean                                                 # :1449
    if loss_mask is not None:
        x_centered = x_centered * loss_mask                               # :1452
    if std_level == "batch":                                              # :1455-1465
        std = _compute_std(x, loss_mask, mean, std_unbiased, high_precision).expand_as(x)
    elif std_level == "group":                                            # :1466-1492
        std = torch.zeros_like(x)
        for i in range(0, bs // group_size):
            s = slice(i * group_size, (i + 1) * group_size)
            xx = x[s]
            m = loss_mask[s] if loss_mask is not None else None
            if group_size == 1 and std_unbiased:
                group_std = torch.ones((1, *xx.shape[1:]), dtype=torch.float64 if high_precision else torch.float32)
            else:
                group_std = _compute_std(xx, m, mean[s], std_unbiased, high_precision)
            std[s] = group_std.expand_as(xx)
    else:
        std = torch.ones_like(x)                                          # :1494-1495
        eps = 0.0
    return (x_centered / (std + eps)).float()                             # :1498


def masked_moments(values, mask):
    """``[K, 4]`` (sum, min, max, count) of each tensor under ``mask``; stats_tracker.py:238, 252-253, 270, 285."""
    d = mask.bool()
    rows = []
    for v in values:
        v = v.float()
        rows.append(torch.stack([
            torch.where(d, v, 0.0).double().sum().float(),
            torch.where(d, v, float("inf")).min() if v.numel() else torch.tensor(float("inf")),
            torch.where(d, v, -float("inf")).max() if v.numel() else torch.tensor(-float("inf")),
            d.sum().float(),
        ]))
    return torch.stack(rows) if rows else torch.zeros(0, 4)


def kl_rewards(old_logp, ref_logp, loss_mask, seqlens, reward_score, kl_ctl, kl_estimator="k1",
               mask_no_eos_with_zero=False):
    """(rewards, kl_rewards); actor.py:198-207 with KLEstimator(apply_clamp=True) (data.py:1620-1656)."""
    from .ppo import kl_estimate

    bs, L = old_logp.shape
    batch_indices = torch.arange(bs)
    kl = kl_estimate(old_logp, ref_logp, kl_estimator).clamp(min=-10, max=10)
    rewards = -kl_ctl * kl
    kl_rew = rewards.clone()
    rewards[batch_indices, seqlens - 1] = 0                                # :203
    indices = torch.clip(seqlens - 2, min=0)                               # :204
    seq_no_eos_mask = seqlens == L
    if mask_no_eos_with_zero:
        rewards[batch_indices, indices] += torch.where(seq_no_eos_mask, 0, reward_score)
    else:
        rewards[batch_indices, indices] += reward_score
    return rewards, kl_rew


def compute_advantages(data, kl_ctl=0.0, kl_estimator="k1", discount=1.0, gae_lambda=1.0, reward_bias=0.0,
                       reward_scaling=1.0, reward_clip=20.0, reward_norm=None, adv_norm=None,
                       mask_no_eos_with_zero=False, use_decoupled_loss=False, recompute_logprob=False,
                       overlong_tokens=None, overlong_penalty_factor=None, max_new_tokens=None):
    """PPOActor._compute_advantages, actor.py:145-250; ``reward_norm`` / ``adv_norm`` are kwargs dicts of
    ``normalization`` or None."""
    data = dict(data)
    if overlong_tokens is not None:                                       # :152-164
        data["rewards"] = data["rewards"].clone()
        data = overlong_penalty(data, overlong_tokens, overlong_penalty_factor, max_new_tokens)
    reward_score = (data["rewards"] + reward_bias) * reward_scaling
    reward_score = torch.clip(reward_score, max=reward_clip, min=-reward_clip)
    if reward_norm is not None:
        reward_score = normalization(reward_score, **reward_norm)
    loss_mask = torch.roll(data["loss_mask"].float(), shifts=-1, dims=-1)
    if not use_decoupled_loss and recompute_logprob:
        old_logp = data["logprobs"] = data["prox_logp"]
    else:
        old_logp = torch.roll(data["logprobs"], shifts=-1, dims=-1)
        if not use_decoupled_loss:
            data["prox_logp"] = old_logp
    ref_logp = data.get("ref_logp")
    if ref_logp is None:
        ref_logp = torch.zeros_like(old_logp)
    ref_logp *= loss_mask  # in place (actor.py:194-195): data["ref_logp"] and, where it is this tensor,
    old_logp *= loss_mask  # data["prox_logp"] come out masked too
    attn_mask = data["attention_mask"]
    seqlens = attn_mask.sum(-1).long()
    seq_no_eos_mask = seqlens == attn_mask.shape[1]
    rewards, kl_rew = kl_rewards(old_logp, ref_logp, loss_mask, seqlens, reward_score, kl_ctl, kl_estimator,
                                 mask_no_eos_with_zero)
    values = data["values"] if "values" in data else torch.zeros_like(rewards)
    advantages, returns = gae(rewards, values, loss_mask, seq_no_eos_mask.float(), discount, gae_lambda)
    data["returns"] = returns
    if adv_norm is not None:
        advantages = normalization(advantages, loss_mask, **adv_norm)
    data.update(advantages=advantages, kl_rewards=kl_rew, tot_rewards=rewards, loss_mask=loss_mask, logprobs=old_logp)
    return data


def overlong_penalty(data, overlong_tokens: int, overlong_penalty_factor: float, max_response_length: int):
    """``reward_overlong_penalty``; areal/utils/functional/functional.py:782-803, statement by statement."""
    reward_score = data["rewards"]
    response_lengths = (data["loss_mask"].sum(dim=-1)).long()                       # :790
    batch_size = data["input_ids"].shape[0]                                        # :791
    for sample_idx in range(batch_size):                                           # :792
        reward_score_cur = reward_score[sample_idx]
        response_length_cur = response_lengths[sample_idx]
        expected_len = max_response_length - overlong_tokens                       # :795
        exceed_len = response_length_cur - expected_len                            # :796
        overlong_reward = min(-exceed_len / overlong_tokens * overlong_penalty_factor, 0)   # :797-799
        reward_score_cur += overlong_reward                                        # :800
        reward_score[sample_idx] = reward_score_cur                                # :801
    data["rewards"] = reward_score
    return data


def masked_normalization(x, mask=None, dim=None, unbiased=False, eps=1e-5, high_precision=True):
    """areal/utils/functional/functional.py:16-53 on one process (the all-reduce of the three sums left out)."""
    dtype = torch.float64 if high_precision else torch.float32
    x = x.to(dtype)
    if dim is None:
        dim = tuple(range(len(x.shape)))
    if mask is None:
        n = 1
        for d in (dim if isinstance(dim, (tuple, list)) else (dim,)):
            n *= x.shape[d]
        factor = torch.tensor(n, dtype=dtype)                                      # :31-33
    else:
        mask = mask.to(dtype)
        x = x * mask                                                               # :36
        factor = mask.sum(dim, keepdim=True)                                       # :37
    x_sum = x.sum(dim=dim, keepdim=True)
    x_sum_sq = x.square().sum(dim=dim, keepdim=True)
    mean = x_sum / factor                                                          # :48
    meansq = x_sum_sq / factor
    var = meansq - mean ** 2                                                       # :50
    if unbiased:
        var = var * (factor / (factor - 1))                                        # :51-52
    return ((x - mean) / (var.sqrt() + eps)).float()                               # :53
