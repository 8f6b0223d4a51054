"""Drop-in counterparts of ``areal.utils.functional`` (``__init__.py:3-35`` of the reference)."""

from areal_amd.functional.functional import (
    RejectionSamplingResult,
    DeferredFloat,
    StatReduction,
    apply_rejection_sampling,
    cispo_loss_fn,
    masked_normalization,
    ppo_actor_loss_fn,
    reward_overlong_penalty,
)
from areal_amd.functional.aux_losses import (
    dpo_pair_logratios,
    dpo_preference_loss,
    ppo_critic_loss_fn,
    sapo_loss_fn,
)
from areal_amd.functional.lm_head import (
    ChunkedLMHeadOutput,
    chunked_lm_head_logprobs_entropy,
    fused_lm_head_logprobs_entropy,
)
from areal_amd.functional.vocab_parallel import (
    gather_logprobs,
    gather_logprobs_entropy,
)

__all__ = [
    "RejectionSamplingResult",
    "DeferredFloat",
    "StatReduction",
    "apply_rejection_sampling",
    "cispo_loss_fn",
    "masked_normalization",
    "ppo_actor_loss_fn",
    "reward_overlong_penalty",
    "sapo_loss_fn",
    "ppo_critic_loss_fn",
    "dpo_pair_logratios",
    "dpo_preference_loss",
    "gather_logprobs",
    "gather_logprobs_entropy",
    "ChunkedLMHeadOutput",
    "chunked_lm_head_logprobs_entropy",
    "fused_lm_head_logprobs_entropy",
]
