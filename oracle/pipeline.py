"""Oracle of the whole step as the engine runs it (test infrastructure, CPU only).

``logits_ppo_step`` chains what FSDPEngine._compute_logprobs_and_loss
(areal/engine/fsdp_engine.py:1977-2046) and grpo_loss_fn
(areal/trainer/ppo/actor.py:408-480) do for one micro-batch: log-probs and entropy
of the padded rows, trimming of the batch padding, the PPO loss with a detached
entropy, the loss scale, and autograd back to the logits.  It is also what the
``cpu_baseline`` leg of the benchmark times.
"""
from __future__ import annotations

import torch

from .logprobs import logprobs_entropy
from .ppo import ppo_actor_loss


def lmhead_logits(hidden: torch.Tensor, weight: torch.Tensor, round_to_bf16: bool = False) -> torch.Tensor:
    """``hidden @ weight.T`` in fp32: the logits of the fp32 reference that the lm_head path is held to.

    With ``round_to_bf16`` the product is rounded to bf16, as the reference's bf16 lm_head hands it to
    ``gather_logprobs_entropy`` (differentiable: the rounding passes gradients through, as autograd's
    ``.to(torch.bfloat16)`` does).  That rounding moves a logit by up to 2^-9 of its magnitude, and a token's
    log-prob with it, so the bf16 pipeline itself sits that far from the fp32 reference."""
    logits = hidden.float() @ weight.float().t()
    return logits.to(torch.bfloat16) if round_to_bf16 else logits


def logits_ppo_step(
    logits: torch.Tensor,
    labels: torch.Tensor,
    proximal_logprobs: torch.Tensor,
    old_logprobs: torch.Tensor,
    advantages: torch.Tensor,
    eps_clip: float,
    loss_mask: torch.Tensor,
    eps_clip_higher: float | None = None,
    c_clip: float | None = None,
    rejection_sampling_cfg=None,
    importance_sampling_level: str = "token",
    cu_seqlens: torch.Tensor | None = None,
    temperature: float = 1.0,
    loss_scale: float = 1.0,
    chunk_size: int = 1024,
    backward: bool = True,
):
    """Returns (loss, stat, d_logits or None); logits may be ``[T_pad, V]`` with T_pad >= len(loss_mask)."""
    x = logits.detach().clone().requires_grad_(backward)
    logp, entropy = logprobs_entropy(x, labels, temperature, chunk_size)       # fsdp_engine.py:1922
    n = loss_mask.shape[0]
    logp, entropy = logp[:n], entropy[:n]                                      # fsdp_engine.py:2027-2031
    loss, stat = ppo_actor_loss(                                               # actor.py:468-480
        logp, proximal_logprobs, old_logprobs, advantages, eps_clip, loss_mask.bool(), eps_clip_higher, c_clip,
        rejection_sampling_cfg, importance_sampling_level, cu_seqlens,
    )
    loss = loss * loss_scale                                                   # fsdp_engine.py:2045-2046
    grad = None
    if backward:
        loss.backward()
        grad = x.grad
    stat = dict(stat, logprobs=logp.detach(), entropy=entropy.detach())
    return loss.detach(), stat, grad
