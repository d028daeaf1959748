"""jax.random's default bit stream restated in numpy (oracle; tests only).

threefry2x32 (Salmon et al., SC'11; 20 rounds) as jax._src.prng uses it: PRNGKey(seed) =
(hi32, lo32) of the seed; fold_in(key, d) = threefry2x32(key, (0, d)); split; random_bits in
the "partitionable" layout (counter (hi, lo) = 64-bit index, output x0 ^ x1) and in the
original layout (counter array split in two halves); uniform / randint / gumbel / categorical.

jax is not importable in this build, so this file is pinned by the golden arrays the
reference's own tests hold for jax.random.PRNGKey(0) inputs (tests/rl/common_test.py:35-108);
see tests/test_oracle_rl.py (the threefry and golden-array tests) for which layout reproduces them.
"""
from __future__ import annotations

import numpy as np

_ROT = (13, 15, 26, 6, 17, 29, 16, 24)


def _rotl(x, r):
  return ((x << np.uint32(r)) | (x >> np.uint32(32 - r))).astype(np.uint32)


def threefry2x32(key, x0, x1):
  """key: (k0, k1) uint32 scalars; x0, x1: uint32 arrays of one shape."""
  with np.errstate(over="ignore"):
    k0, k1 = np.uint32(key[0]), np.uint32(key[1])
    ks = (k0, k1, np.uint32(k0 ^ k1 ^ np.uint32(0x1BD11BDA)))
    x0 = (np.asarray(x0, dtype=np.uint32) + ks[0]).astype(np.uint32)
    x1 = (np.asarray(x1, dtype=np.uint32) + ks[1]).astype(np.uint32)
    for g in range(5):
      for r in range(4):
        x0 = (x0 + x1).astype(np.uint32)
        x1 = _rotl(x1, _ROT[(g & 1) * 4 + r])
        x1 = x1 ^ x0
      x0 = (x0 + ks[(g + 1) % 3]).astype(np.uint32)
      x1 = (x1 + ks[(g + 2) % 3] + np.uint32(g + 1)).astype(np.uint32)
  return x0, x1


def prng_key(seed: int):
  seed = int(seed) & 0xFFFFFFFFFFFFFFFF
  return np.uint32(seed >> 32), np.uint32(seed & 0xFFFFFFFF)


def fold_in(key, data: int):
  a, b = threefry2x32(key, np.uint32([0]), np.uint32([int(data) & 0xFFFFFFFF]))
  return np.uint32(a[0]), np.uint32(b[0])


def random_bits(key, shape, partitionable: bool = True) -> np.ndarray:
  size = int(np.prod(shape)) if len(shape) else 1
  idx = np.arange(size, dtype=np.uint64)
  if partitionable:
    x0, x1 = threefry2x32(key, (idx >> np.uint64(32)).astype(np.uint32), idx.astype(np.uint32))
    bits = x0 ^ x1
  else:
    cnt = idx.astype(np.uint32)
    if size % 2:
      cnt = np.concatenate([cnt, np.uint32([0])])
    half = cnt.size // 2
    x0, x1 = threefry2x32(key, cnt[:half], cnt[half:])
    bits = np.concatenate([x0, x1])[:size]
  return bits.reshape(shape)


def split(key, num: int = 2, partitionable: bool = True):
  """jax.random.split: keys are the random bits of shape (num, 2)."""
  if partitionable:
    idx = np.arange(num, dtype=np.uint64)
    x0, x1 = threefry2x32(key, (idx >> np.uint64(32)).astype(np.uint32), idx.astype(np.uint32))
    return [(np.uint32(a), np.uint32(b)) for a, b in zip(x0, x1)]
  bits = random_bits(key, (num, 2), partitionable=False)
  return [(np.uint32(a), np.uint32(b)) for a, b in bits]


def uniform(key, shape, minval=0.0, maxval=1.0, partitionable: bool = True) -> np.ndarray:
  bits = random_bits(key, shape, partitionable)
  f = ((bits >> np.uint32(9)) | np.uint32(0x3F800000)).view(np.float32) - np.float32(1.0)
  lo, hi = np.float32(minval), np.float32(maxval)
  return np.maximum(lo, (f * (hi - lo) + lo).astype(np.float32))


def gumbel(key, shape, partitionable: bool = True) -> np.ndarray:
  tiny = np.finfo(np.float32).tiny
  u = uniform(key, shape, minval=tiny, maxval=1.0, partitionable=partitionable)
  return (-np.log(-np.log(u))).astype(np.float32)


def categorical(key, logits: np.ndarray, partitionable: bool = True) -> np.ndarray:
  """argmax(logits + gumbel) over the last axis (jax.random.categorical)."""
  g = gumbel(key, logits.shape, partitionable)
  return np.argmax(g + logits.astype(np.float32), axis=-1)


def randint(key, shape, minval, maxval, partitionable: bool = True) -> np.ndarray:
  """jax.random.randint for int32 ranges (two 32-bit draws combined, as jax does)."""
  k1, k2 = split(key, 2, partitionable)
  hi_bits = random_bits(k1, shape, partitionable).astype(np.uint64)
  lo_bits = random_bits(k2, shape, partitionable).astype(np.uint64)
  span = np.uint64(int(maxval) - int(minval))
  mult = np.uint64((1 << 32) % int(span))
  mult = (mult * mult) % span
  off = ((hi_bits % span) * mult + (lo_bits % span)) % span
  return (np.int64(minval) + off.astype(np.int64)).astype(np.int32)
