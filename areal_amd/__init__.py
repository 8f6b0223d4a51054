"""MI355X-native implementation of AReaL's per-token RL training hot path.

Fused lm_head -> log-softmax -> label log-prob + entropy, the PPO/GRPO/CISPO actor loss with
rejection-sampling masks, packed-sequence GAE and advantage normalisation, as hand-written
gfx950 HIP kernels behind the Python signatures of ``areal.utils.functional``.
"""

__version__ = "0.1.0"
