"""oracle/utils_ref.py against the literal vectors of the reference's own tests
(tests/generate/utils_test.py:91-168, tests/sft/sft_utils_test.py:22-68) and brute force."""
import numpy as np

from oracle import utils_ref as U


def test_compute_attention_masks_reference_vectors():
  # tests/generate/utils_test.py:91-115
  input_mask = np.array([[1, 1, 0, 0, 0], [1, 1, 0, 1, 0]], dtype=bool)
  got = U.compute_attention_masks(4, 8, input_mask)
  want = np.array([[0, 0, 1, 1, 1, 0, 0, 0], [0, 0, 1, 0, 1, 0, 0, 0]], dtype=bool)
  assert got.shape == (2, 1, 8)
  np.testing.assert_array_equal(got.squeeze(1), want)
  got = U.compute_attention_masks(4, 4, input_mask)
  want = np.array([[0, 1, 1, 1], [0, 1, 0, 1]], dtype=bool)
  np.testing.assert_array_equal(got.squeeze(1), want)


def test_make_causal_attn_mask_with_cache_size():
  # tests/generate/utils_test.py:117-136
  input_mask = np.array([[0, 1, 1, 0], [1, 1, 1, 0]])
  want = np.array([
      [[0, 0, 0, 0, 0], [0, 1, 0, 0, 0], [0, 1, 1, 0, 0], [0, 1, 1, 0, 0]],
      [[1, 0, 0, 0, 0], [1, 1, 0, 0, 0], [1, 1, 1, 0, 0], [1, 1, 1, 0, 0]],
  ])
  np.testing.assert_array_equal(U.make_causal_attn_mask(input_mask, 5), want)


def test_make_causal_attn_mask_sft():
  # tests/sft/sft_utils_test.py:22-50
  input_mask = np.array([[True, True, True, True], [True, True, True, False], [False, True, True, False]])
  want = np.array([
      [[1, 0, 0, 0], [1, 1, 0, 0], [1, 1, 1, 0], [1, 1, 1, 1]],
      [[1, 0, 0, 0], [1, 1, 0, 0], [1, 1, 1, 0], [1, 1, 1, 0]],
      [[0, 0, 0, 0], [0, 1, 0, 0], [0, 1, 1, 0], [0, 1, 1, 0]],
  ], dtype=bool)
  np.testing.assert_array_equal(U.make_causal_attn_mask(input_mask), want)


def test_build_positions_from_mask():
  # tests/sft/sft_utils_test.py:52-64
  input_mask = np.array([[1, 1, 1, 1], [0, 1, 1, 1], [1, 1, 1, 0], [0, 1, 1, 0]])
  want = np.array([[0, 1, 2, 3], [0, 0, 1, 2], [0, 1, 2, 2], [0, 0, 1, 1]])
  np.testing.assert_array_equal(U.build_positions_from_mask(input_mask), want)


def test_next_power_of_2():
  # tests/generate/utils_test.py:138-143
  assert [U.next_power_of_2(x) for x in (0, 2, 3, 4, 5)] == [1, 2, 4, 4, 8]


def test_find_indices():
  # tests/generate/utils_test.py:145-177
  for ids, want in (([1, 2, 3, 4, 5, 6], 0), ([0, 0, 1, 2, 3, 4], 2), ([0, 1, 2, 3, 0, 0], 1)):
    assert U.find_first_non_pad_idx(np.array(ids), 0) == want
  for ids, want in (([1, 2, 3, 4, 5, -1], 5), ([1, 2, -1, 4, -1, 0], 2), ([1, 2, 3, 4, 5, 6], 6)):
    assert U.find_first_eos_idx(np.array(ids), -1) == want
  for ids, want in (([1, 2, 3, 4, 5, 6], 5), ([1, 2, 3, 0, 0, 0], 2), ([0, 1, 2, 3, 0, 0], 3)):
    assert U.find_last_non_pad_idx(np.array(ids), 0) == want


def test_pad_to_length():
  x = np.array([1, 2, 3])
  np.testing.assert_array_equal(U.pad_to_length(x, 5, 0, left=True), [0, 0, 1, 2, 3])
  np.testing.assert_array_equal(U.pad_to_length(x, 5, 9, left=False), [1, 2, 3, 9, 9])
  np.testing.assert_array_equal(U.pad_to_length(x, 3, 0, left=True), [1, 2, 3])


def test_sliding_window_mask_brute_force():
  """Decode-time window of tunix/models/gemma3/model.py:476-496: keys (last - w, last]."""
  rng = np.random.default_rng(0)
  for w in (1, 3, 8):
    m = rng.random((4, 1, 12)) > 0.4
    m[1] = False  # an all-zero row selects index 0
    got = U.create_sliding_window_mask(m, w)
    for b in range(4):
      ones = np.nonzero(m[b, 0])[0]
      last = int(ones[-1]) if ones.size else 0
      want = np.array([(s <= last) and (s >= last - w + 1) for s in range(12)])
      np.testing.assert_array_equal(got[b, 0], want)
