"""A packed batch shared by the CPU and the GPU test of the packed log-probability pass."""
import numpy as np


def packed_case(V, seed=11):
  """Three sequences in two rows of 24 slots: row 0 = A (10 tokens) | B (14), row 1 = C (8) |
  16 padding slots (segment 0, position 0)."""
  rng = np.random.default_rng(seed)
  A, Bq, Cq = (rng.integers(2, V, size=n).astype(np.int32) for n in (10, 14, 8))
  L = 24
  ids = np.zeros((2, L), np.int32)
  seg = np.zeros((2, L), np.int32)
  pos = np.zeros((2, L), np.int32)
  ids[0, :10], seg[0, :10], pos[0, :10] = A, 1, np.arange(10)
  ids[0, 10:], seg[0, 10:], pos[0, 10:] = Bq, 2, np.arange(14)
  ids[1, :8], seg[1, :8], pos[1, :8] = Cq, 1, np.arange(8)
  return (A, Bq, Cq), ids, seg, pos
