"""Mask / position / index helpers of the sampler, restated in numpy (oracle; tests only).

Follows tunix/generate/utils.py:34-298 and tunix/sft/utils.py:33-71.
"""
from __future__ import annotations

import numpy as np


def compute_attention_masks(time_step: int, seq_len: int, input_mask: np.ndarray) -> np.ndarray:
  """tunix/generate/utils.py:34-58.  `input_mask` is True where the token buffer holds pad.

  Returns [B, 1, seq_len] bool, True = attend.
  """
  input_mask = np.asarray(input_mask, dtype=bool)
  batch = input_mask.shape[0]
  causal_padding = np.arange(seq_len)[None, :] > np.full((batch, 1), time_step)
  max_seq_len = min(input_mask.shape[-1], seq_len)
  start = max(time_step - seq_len + 1, 0)
  # jax.lax.dynamic_slice clamps the start index so that the slice stays in bounds
  start = min(start, input_mask.shape[-1] - max_seq_len)
  sliced = input_mask[:, start:start + max_seq_len]
  padded = np.zeros((batch, seq_len), dtype=bool)
  padded[:, :max_seq_len] = sliced
  causal_padding = np.logical_or(causal_padding, padded)
  return ~causal_padding[:, None, :]


def make_causal_attn_mask(input_mask: np.ndarray, cache_size: int | None = None) -> np.ndarray:
  """tunix/generate/utils.py:61-83 (with cache_size) and tunix/sft/utils.py:33-56 (without)."""
  input_mask = np.asarray(input_mask).astype(bool)
  if input_mask.ndim != 2:
    raise ValueError(f"Input mask must be 2D (shape [B, L]), but got {input_mask.shape}.")
  seq_len = input_mask.shape[-1]
  causal = np.tril(np.ones((seq_len, seq_len), dtype=bool))
  attn = input_mask[:, None, :] & causal[None]
  if cache_size is not None:
    padding = cache_size - seq_len
    assert padding >= 0
    attn = np.pad(attn, ((0, 0), (0, 0), (0, padding)))
  return attn


def next_power_of_2(x: int) -> int:
  """tunix/generate/utils.py:86-90."""
  if x == 0:
    return 1
  return int(2 ** int(np.ceil(np.log2(x))))


def pad_to_length(x: np.ndarray, target_length: int, pad_value: int = 0, left: bool = False,
                  axis: int = 0) -> np.ndarray:
  """tunix/generate/utils.py:93-125."""
  length = x.shape[axis]
  if length >= target_length:
    return x
  shape = list(x.shape)
  shape[axis] = target_length - length
  padding = np.full(shape, pad_value, dtype=x.dtype)
  return np.concatenate([padding, x] if left else [x, padding], axis=axis)


def find_first_non_pad_idx(ids: np.ndarray, pad_id: int) -> int:
  """tunix/generate/utils.py:128-138, :152-156."""
  ids = np.asarray(ids)
  assert ids.ndim == 1
  mask = ids != pad_id
  return int(np.argmax(mask)) if mask.any() else 0


def find_first_eos_idx(ids: np.ndarray, eos_id) -> int:
  """tunix/generate/utils.py:141-149, :159-167."""
  ids = np.asarray(ids)
  assert ids.ndim == 1
  mask = np.isin(ids, np.atleast_1d(np.asarray(eos_id)))
  return int(np.argmax(mask)) if mask.any() else len(ids)


def find_last_non_pad_idx(ids: np.ndarray, pad_id: int) -> int:
  """tunix/generate/utils.py:170-181."""
  ids = np.asarray(ids)
  assert ids.ndim == 1
  mask = (ids != pad_id)[::-1]
  return int(ids.shape[-1] - np.argmax(mask) - 1) if mask.any() else int(ids.shape[-1])


def build_positions_from_mask(input_mask: np.ndarray) -> np.ndarray:
  """tunix/generate/utils.py:285-298 == tunix/sft/utils.py:59-71."""
  positions = np.cumsum(np.asarray(input_mask).astype(np.int32), axis=-1)
  return positions - (positions >= 1)


def create_sliding_window_mask(attn_mask: np.ndarray, sliding_window_size: int) -> np.ndarray:
  """tunix/models/gemma3/model.py:451-496 (decode: attn_mask [B, 1, cache_len])."""
  attn_mask = np.asarray(attn_mask).astype(bool)
  cache_len = attn_mask.shape[-1]
  all_zero = ~attn_mask.any(axis=-1)
  first_one_from_right = np.argmax(attn_mask[:, :, ::-1], axis=-1)
  upper = np.where(all_zero, 0, cache_len - 1 - first_one_from_right).squeeze(-1)
  window_start = upper - sliding_window_size + 1
  abs_pos = np.arange(cache_len)
  window = abs_pos[None, :] >= window_start[:, None]
  causal = abs_pos[None, :] <= upper[:, None]
  return (window & causal)[:, None, :]
