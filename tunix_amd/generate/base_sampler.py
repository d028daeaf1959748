"""Output contract of the sampler (tunix/generate/base_sampler.py:30-48)."""
from __future__ import annotations

import dataclasses
from typing import Optional

import numpy as np


@dataclasses.dataclass
class SamplerOutput:
  """Output of the sampler."""

  # Decoded samples from the model.
  text: list[str]
  # Per-step logits used during sampling (fp32 numpy arrays), [] unless return_logits.
  logits: Optional[list[np.ndarray]]
  # Tokens corresponding to the generated samples.
  tokens: list[np.ndarray]
  # Left padded prompt tokens.
  padded_prompt_tokens: np.ndarray
  logprobs: Optional[list[list[float]]]
