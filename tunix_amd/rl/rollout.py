"""A rollout engine with the interface of the reference's BaseRollout
(tunix/rl/rollout/base_rollout.py:61-103) backed by the HIP sampler, shaped after
VanillaRollout (tunix/rl/rollout/vanilla_rollout.py:30-125): generate() forwards the
RolloutConfig fields to Sampler.__call__, get_per_token_logps() runs the fused
lm_head -> log-softmax -> gather pass, update_params() swaps the LoRA factors in place.
"""
from __future__ import annotations

import dataclasses
from typing import Any

import numpy as np
import torch

from ..generate import CacheConfig, Sampler
from ..model import QLoRAModel
from . import common


@dataclasses.dataclass
class RolloutConfig:
  """The sampling fields of tunix/common/configs.py:71-130 that the vanilla engine reads."""
  max_tokens_to_generate: int = 64
  temperature: float = 0.9
  top_p: float | None = 1.0
  top_k: int | None = None
  seed: int | None = None
  max_prompt_length: int = 64
  kv_cache_size: int = 1024
  eos_tokens: list[int] | None = None
  return_logprobs: bool = False


@dataclasses.dataclass
class RolloutOutput:
  """tunix/rl/rollout/base_rollout.py:35-58."""
  text: list[str]
  logits: list | None
  tokens: list[np.ndarray]
  left_padded_prompt_tokens: np.ndarray
  logprobs: list | None


class HipRollout:
  def __init__(self, model: QLoRAModel, tokenizer, cache_config_or_size: CacheConfig | int):
    cfg = model.cfg
    if isinstance(cache_config_or_size, int):
      cache_config_or_size = CacheConfig(cache_size=cache_config_or_size, num_layers=cfg.num_layers,
                                         num_kv_heads=cfg.num_kv_heads, head_dim=cfg.head_dim)
    self._sampler = Sampler(model, tokenizer, cache_config_or_size)

  def generate(self, prompts: list[str], rollout_config: RolloutConfig, **kwargs) -> RolloutOutput:
    rc = rollout_config
    out = self._sampler(
        input_strings=prompts,
        max_generation_steps=rc.max_tokens_to_generate,
        max_prompt_length=rc.max_prompt_length,
        echo=False,
        temperature=rc.temperature,
        top_p=rc.top_p,
        top_k=rc.top_k,
        seed=rc.seed,
        pad_output=False,
        eos_tokens=rc.eos_tokens,
        return_logprobs=rc.return_logprobs,
    )
    return RolloutOutput(text=out.text, logits=out.logits, tokens=out.tokens,
                         left_padded_prompt_tokens=out.padded_prompt_tokens, logprobs=out.logprobs)

  def get_per_token_logps(self, prompt_tokens, completion_tokens, temperature: float = 1.0,
                          chunk_size: int = 0) -> torch.Tensor:
    return common.compute_per_token_logps(self.model(), prompt_tokens, completion_tokens,
                                          pad_id=self.pad_id(), eos_id=self.eos_id(),
                                          temperature=temperature, chunk_size=chunk_size)

  def update_params(self, params: dict, filter_types: Any = None) -> None:
    """Weight sync between steps (tunix/rl/rollout/vanilla_rollout.py:92-121).  `params` maps flat
    names to new tensors.  Only '<linear>.lora_a' / '<linear>.lora_b' leaves: the LoRA-only swap,
    every adapter present (tunix/generate/sampler.py:333-352 requires the same structure as the
    old state).  With base parameters in it: those are replaced too, the linears re-quantised
    and re-packed in place (the full-state branch, sampler.py:322-325)."""
    self._sampler.update_params(params)

  def pad_id(self) -> int:
    return self._sampler.tokenizer.pad_id()

  def eos_id(self) -> int:
    return self._sampler.tokenizer.eos_id()

  def model(self) -> QLoRAModel:
    return self._sampler.transformer
