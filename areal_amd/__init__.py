"""MI355X-native kernels for AReaL's PPO/GRPO log-prob, entropy and actor-loss path.

Importing the package does not load the HIP library; the first op call does, and
raises ``NativeLibraryError`` if ``libareal_amd.so`` has not been built.
"""
from .actor_ops import (
    apply_m2po_masking,
    compute_prox_logp_approximations,
    distillation_terms,
    proximal_logging_stats,
)
from .advantages import (
    KLEstimator,
    Normalization,
    gae_advantages,
    kl_regularized_rewards,
    masked_moments,
    masked_normalization,
    reward_overlong_penalty,
)
from .dpo import dpo_loss, dpo_pair_logratios, dpo_preference_loss, rw_pair_loss
from .config import NormConfig, RejectionSamplingConfig
from .functional import (
    RejectionSamplingResult,
    apply_rejection_sampling,
    fused_lm_head_ppo_loss,
    fused_logprobs_ppo_loss,
    gather_logprobs,
    gather_logprobs_entropy,
    gather_logprobs_entropy_stats,
    lm_head_logprobs_entropy,
    lm_head_logprobs_entropy_stats,
    lm_head_chunk_tokens,
    lm_head_logprobs_entropy_static,
    ppo_actor_loss_fn,
    ppo_critic_loss_fn,
    sapo_loss_fn,
)
from .packing import pack_tensor_dict, pad_packed_tensor_dict, segment_copy, unpad_logits
from .tree import (
    gather_logprobs_entropy_pairs,
    gather_packed_tree_logprobs,
    gather_packed_tree_logprobs_entropy,
    gather_packed_tree_vocab_stats,
    merge_packed_tree_results,
    tree_sequence_pairs,
)
from .sapo import fused_lm_head_sapo_loss, fused_logprobs_sapo_loss
from .sft import fused_lm_head_sft_loss, fused_logprobs_sft_loss, sft_loss_fn
from ._native import NativeLibraryError

__version__ = "0.1.0"

__all__ = [
    "NativeLibraryError",
    "gather_packed_tree_vocab_stats",
    "merge_packed_tree_results",
    "KLEstimator",
    "fused_lm_head_sapo_loss",
    "fused_logprobs_sapo_loss",
    "fused_lm_head_sft_loss",
    "fused_logprobs_sft_loss",
    "sft_loss_fn",
    "proximal_logging_stats",
    "masked_normalization",
    "dpo_loss",
    "dpo_pair_logratios",
    "dpo_preference_loss",
    "rw_pair_loss",
    "NormConfig",
    "Normalization",
    "RejectionSamplingConfig",
    "RejectionSamplingResult",
    "apply_m2po_masking",
    "apply_rejection_sampling",
    "compute_prox_logp_approximations",
    "distillation_terms",
    "fused_lm_head_ppo_loss",
    "fused_logprobs_ppo_loss",
    "gae_advantages",
    "gather_logprobs",
    "gather_logprobs_entropy",
    "gather_logprobs_entropy_pairs",
    "gather_logprobs_entropy_stats",
    "gather_packed_tree_logprobs",
    "gather_packed_tree_logprobs_entropy",
    "kl_regularized_rewards",
    "lm_head_logprobs_entropy",
    "lm_head_logprobs_entropy_stats",
    "lm_head_chunk_tokens",
    "lm_head_logprobs_entropy_static",
    "masked_moments",
    "pack_tensor_dict",
    "pad_packed_tensor_dict",
    "ppo_actor_loss_fn",
    "ppo_critic_loss_fn",
    "reward_overlong_penalty",
    "sapo_loss_fn",
    "segment_copy",
    "tree_sequence_pairs",
    "unpad_logits",
]
