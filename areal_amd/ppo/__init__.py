"""PPO-side callers of the hot path (GAE, advantage shaping, the GRPO loss wrapper)."""
