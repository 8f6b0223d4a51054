"""Drop-in counterparts of ``areal.utils.functional`` (``__init__.py:3-35`` of the reference)."""

from areal_amd.functional.lm_head import (
    ChunkedLMHeadOutput,
    fused_lm_head_logprobs_entropy,
)

__all__ = [
    "ChunkedLMHeadOutput",
    "fused_lm_head_logprobs_entropy",
]
