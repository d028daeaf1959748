"""Host-side helpers of the sampler (tunix/generate/utils.py:86-181, :285-298)."""
from __future__ import annotations

import numpy as np


def next_power_of_2(x: int) -> int:
  """Smallest power of two that is not smaller than x (utils.py:86-90)."""
  if x == 0:
    return 1
  return 1 << (int(x) - 1).bit_length()


def pad_to_length(x: np.ndarray, target_length: int, pad_value: int = 0, left: bool = False,
                  axis: int = 0) -> np.ndarray:
  """Pads `x` along `axis` up to `target_length` (utils.py:93-125); longer inputs pass through."""
  length = x.shape[axis]
  if length >= target_length:
    return x
  shape = list(x.shape)
  shape[axis] = target_length - length
  fill = np.full(shape, pad_value, dtype=x.dtype)
  return np.concatenate([fill, x] if left else [x, fill], axis=axis)


def np_find_first_non_pad_idx(ids: np.ndarray, pad_id: int) -> int:
  assert ids.ndim == 1, f"ids should be a 1d array. Got: {ids.shape}"
  hit = np.flatnonzero(ids != pad_id)
  return int(hit[0]) if hit.size else 0


def np_find_first_eos_idx(ids: np.ndarray, eos_id) -> int:
  assert ids.ndim == 1, f"ids should be a 1d array. Got: {ids.shape}"
  hit = np.flatnonzero(np.isin(ids, np.atleast_1d(np.asarray(eos_id))))
  return int(hit[0]) if hit.size else len(ids)


def build_positions_from_mask(input_mask: np.ndarray) -> np.ndarray:
  """RoPE positions that ignore pad tokens (utils.py:285-298): 0-based count of valid tokens."""
  running = np.cumsum(np.asarray(input_mask, dtype=np.int32), axis=-1)
  return (running - (running >= 1)).astype(np.int32)


def check_sampling_mode_conflict(current: list, new_mode: str) -> None:
  if current[0] is not None:
    raise ValueError(
        f"Conflicts setting sampling_mode, the current set sampling_mode is {current[0]} but"
        f" trying to override to {new_mode}. The rules are\n: 1. If top_p is provided, top_p will"
        " be used. 2. If beam_size is provided,beam_search will be used 3. If none of the above,"
        " greedy will be used.")
  current[0] = new_mode


class IdTokenizer:
  """Tokenizer stand-in for prompts given as token ids ("12 7 99" <-> [12, 7, 99])."""

  def __init__(self, vocab_size: int, pad_id: int = 0, eos_id: int = 1, bos_id: int | None = None):
    self.vocab_size, self._pad, self._eos, self._bos = vocab_size, pad_id, eos_id, bos_id

  def encode(self, s) -> list[int]:
    if isinstance(s, str):
      return [int(t) for t in s.split()]
    return [int(t) for t in s]

  def decode(self, ids) -> str:
    return " ".join(str(int(i)) for i in ids)

  def pad_id(self) -> int:
    return self._pad

  def eos_id(self) -> int:
    return self._eos

  def bos_id(self):
    return self._bos

  def dedup_bos_ids(self, ids: list[int]) -> list[int]:
    i = 0
    while i + 1 < len(ids) and ids[i] == self._bos and ids[i + 1] == self._bos:
      i += 1
    return ids[i:]
