"""MI355X-native quantized rollout decode for tunix-style QLoRA models.

Public surface (mirrors the reference's names for this path):
  tunix_amd.generate.Sampler / SamplerOutput / CacheConfig
  tunix_amd.rl.common.compute_per_token_logps / selective_log_softmax
  tunix_amd.rl.rollout.HipRollout (a BaseRollout-shaped engine)
"""
from .config import ModelConfig  # noqa: F401

__version__ = "0.1.0"
