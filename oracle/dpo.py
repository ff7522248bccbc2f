"""CPU oracle of the DPO loss over a packed batch of interleaved pairs.  TEST INFRASTRUCTURE ONLY.

Restates in plain PyTorch on the CPU: ``dpo_pair_logratios`` and ``dpo_preference_loss``
(areal/utils/functional/functional.py:641-703), ``_dpo_valid_pairs`` and ``compute_dpo_loss``
(areal/trainer/dpo/dpo_engine.py:22-24, 147-213).  How each function is pinned is listed in ``oracle/PINNING.md``.
"""
from __future__ import annotations

import torch


def shifted_mask(loss_mask, cu_seqlens):
    """Mask moved to next-token alignment; functional.py:663-667.  Written as an explicit loop over sequences."""
    out = torch.zeros_like(loss_mask, dtype=torch.bool)
    cu = [int(v) for v in cu_seqlens]
    for s in range(len(cu) - 1):
        b, e = cu[s], cu[s + 1]
        for t in range(b, e - 1):          # the last position of a sequence has no next token
            out[t] = bool(loss_mask[t + 1])
    return out


def valid_pairs(cu_seqlens):
    """dpo_engine.py:22-24: both sequences of a pair are non-empty."""
    seqlens = cu_seqlens[1:] - cu_seqlens[:-1]
    return seqlens.view(-1, 2).ne(0).all(dim=1)


def pair_logratios(logprobs, ref_logprobs, cu_seqlens, loss_mask, valid):
    """(policy_logps, ref_logps, completion_lens), each [K, 2] fp64; functional.py:641-687."""
    sm = shifted_mask(loss_mask.bool(), cu_seqlens)
    masked = sm.to(logprobs.dtype)
    cu = [int(v) for v in cu_seqlens]
    n = len(cu) - 1
    pol, ref, lens = [], [], []
    for s in range(n):
        sl = slice(cu[s], cu[s + 1])
        pol.append((logprobs[sl] * masked[sl]).double().sum())      # :671-672
        ref.append((ref_logprobs[sl] * masked[sl]).double().sum())  # :673
        lens.append(sm[sl].double().sum())                          # :675-676
    stack = lambda xs: torch.stack(xs) if xs else torch.zeros(0, dtype=torch.float64)
    return tuple(stack(x).view(-1, 2)[valid] for x in (pol, ref, lens))


def preference_loss(logits, beta, loss_type="sigmoid"):
    """functional.py:689-703."""
    if loss_type == "sigmoid":
        return -torch.nn.functional.logsigmoid(beta * logits.float())
    if loss_type == "ipo":
        return (logits.float() - 1.0 / (2.0 * beta)) ** 2
    raise ValueError(f"Unsupported DPO loss_type: {loss_type!r}")


def compute_dpo_loss(logprobs, ref_logprobs, cu_seqlens, loss_mask, beta, loss_type="sigmoid"):
    """(loss, stat); dpo_engine.py:147-213 with the logged tensors returned instead of recorded."""
    cu_seqlens = cu_seqlens.long()
    valid = valid_pairs(cu_seqlens)
    if not valid.any():                                                            # :160-162
        z = torch.zeros(0, dtype=torch.float32)
        return torch.zeros((), dtype=torch.float32), dict(loss=z, chosen_reward=z, rejected_reward=z, valid_pairs=valid)
    pol, ref, lens = pair_logratios(logprobs, ref_logprobs, cu_seqlens, loss_mask, valid)
    if loss_type == "ipo":                                                         # :168-180
        chosen_avg = (pol[:, 0] - ref[:, 0]) / lens[:, 0].clamp(min=1)
        rejected_avg = (pol[:, 1] - ref[:, 1]) / lens[:, 1].clamp(min=1)
        logits = chosen_avg - rejected_avg
    else:                                                                          # :181-184
        logits = (pol[:, 0] - pol[:, 1]) - (ref[:, 0] - ref[:, 1])
    per_pair = preference_loss(logits, beta, loss_type)
    stat = dict(
        loss=per_pair.detach().float(),
        chosen_reward=(beta * (pol[:, 0] - ref[:, 0]).detach()).float(),           # :189
        rejected_reward=(beta * (pol[:, 1] - ref[:, 1]).detach()).float(),
        valid_pairs=valid,
    )
    return per_pair.mean(), stat


def compute_rw_loss(scores, cu_seqlens):
    """(loss, stat); areal/trainer/rw/rw_engine.py:115-146 with the logged tensors returned."""
    seqlens = cu_seqlens[1:] - cu_seqlens[:-1]
    valid = valid_pairs(cu_seqlens)                                                 # :20-22, 119
    if not valid.any():                                                            # :120-122
        z = torch.zeros(0, dtype=torch.float32)
        return torch.zeros((), dtype=torch.float32), dict(loss=z, pos_score=z, neg_score=z, valid_pairs=valid)
    terminal = seqlens.cumsum(0) - 1                                               # :125
    assert scores.shape[0] == seqlens.sum()
    s = scores[terminal].view(-1, 2)[valid].float()                                # :128
    loss = -(torch.nn.functional.logsigmoid(s[:, 0] - s[:, 1]))                    # :130
    stat = dict(loss=loss.detach(), pos_score=s[:, 0].detach(), neg_score=s[:, 1].detach(), valid_pairs=valid,
                correct_ratio=(s[:, 0] > s[:, 1]).float())
    return loss.mean(), stat
