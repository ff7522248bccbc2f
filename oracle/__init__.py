"""CPU oracle for the PPO/GRPO log-prob / entropy / actor-loss path.

TEST INFRASTRUCTURE ONLY.  This package restates, in plain PyTorch on the CPU,
the algorithm of the reference's ``areal/utils/functional`` so that the HIP
kernels can be checked against it.  It may be imported by ``tests/``, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``;
nothing under ``areal_amd/`` imports it, and no product path routes through it.

Each function cites the reference lines it follows.  How each one is pinned
(reference known-answer tests, closed forms, brute force, library routines) is
listed in ``oracle/PINNING.md`` and exercised by ``tests/test_oracle_*.py``.
Parity status: every function below is pinned; none is "parity unpinned".
"""
from .logprobs import (
    logprobs,
    logprobs_entropy,
    logprobs_entropy_f64,
    logprobs_entropy_grad_closed_form,
)
from .ppo import (
    RejectionSamplingOutput,
    kl_estimate,
    ppo_actor_loss,
    rejection_sampling,
    sequence_level_ratio_and_advantages,
)
from .advantages import gae, masked_moments, normalization
from .siblings import critic_loss, distillation_loss, m2po_mask, prox_logp_approximations, sapo_loss
from . import dpo  # noqa: F401  (DPO pair sums and loss)
from . import microbatch  # noqa: F401  (micro-batch allocation and split)
from . import sft  # noqa: F401  (supervised loss over a packed batch)
from .pipeline import lmhead_logits, logits_ppo_step

__all__ = [
    "logprobs",
    "logprobs_entropy",
    "logprobs_entropy_f64",
    "logprobs_entropy_grad_closed_form",
    "RejectionSamplingOutput",
    "kl_estimate",
    "ppo_actor_loss",
    "rejection_sampling",
    "sequence_level_ratio_and_advantages",
    "gae",
    "masked_moments",
    "normalization",
    "critic_loss",
    "distillation_loss",
    "m2po_mask",
    "prox_logp_approximations",
    "sapo_loss",
    "lmhead_logits",
    "logits_ppo_step",
]
