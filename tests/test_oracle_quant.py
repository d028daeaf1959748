"""Closed-form and brute-force checks of oracle/quant_ref.py.

The quantised arithmetic of the reference lives in qwix, which is not in the reference tree and
not installed, and the reference holds no golden vector of a quantised result: parity with qwix
itself is UNPINNED.  What is pinned here is the format include/tunix_hip.h defines, by cases
where the right answer is known without running the code under test.
"""
import numpy as np
import torch

from oracle import quant_ref as Q


def test_int4_exact_roundtrip():
  """w = scale * q with |q| <= 7 and max |q| = 7 in every group: codes are q + 8, dequant exact."""
  rng = np.random.default_rng(0)
  K, N, g = 128, 16, 32
  q = rng.integers(-7, 8, size=(K, N))
  q.reshape(K // g, g, N)[:, 0, :] = 7
  scale = 2.0 ** rng.integers(-6, 3, size=(K // g, N))
  w = (q.reshape(K // g, g, N) * scale[:, None, :]).reshape(K, N).astype(np.float32)
  codes, s = Q.quantize(w, g, Q.INT4)
  np.testing.assert_array_equal(codes, q + 8)
  np.testing.assert_array_equal(s, scale.astype(np.float32))
  np.testing.assert_array_equal(Q.dequantize(codes, s, g, Q.INT4), w)


def test_int4_rounding_and_clamp():
  # absmax 7 -> scale 1: halves round to even, -8 is reachable only below -7.5 (clamped by absmax)
  col = np.array([7.0, 0.5, 1.5, 2.5, -0.5, -1.5, 3.49, -3.51] + [0.0] * 24, dtype=np.float32)
  codes, s = Q.quantize(col[:, None].repeat(16, 1), 32, Q.INT4)
  assert s[0, 0] == 1.0
  np.testing.assert_array_equal(codes[:8, 0].astype(np.int32) - 8, [7, 0, 2, 2, 0, -2, 3, -4])
  # scale is bf16(absmax / 7)
  col2 = np.array([1.0] + [0.0] * 31, dtype=np.float32)
  _, s2 = Q.quantize(col2[:, None].repeat(16, 1), 32, Q.INT4)
  assert s2[0, 0] == Q.rb_np(np.array([1.0 / 7.0], dtype=np.float32))[0]


def test_nf4_levels_recovered_and_ties():
  lv = Q.NF4_LEVELS
  K, N, g = 32, 16, 32
  col = np.zeros(K, dtype=np.float32)
  col[:16] = lv * 4.0           # absmax = 4 (power of two: bf16 scale is exact)
  col[16] = 4.0 * 0.5 * (lv[3] + lv[4])   # exact midpoint of two levels -> the lower code
  w = col[:, None].repeat(N, 1)
  codes, s = Q.quantize(w, g, Q.NF4)
  assert s[0, 0] == 4.0
  np.testing.assert_array_equal(codes[:16, 0], np.arange(16))
  mid = np.float32(np.float32(col[16]) / np.float32(4.0))
  mids = (np.float32(0.5) * (lv[:-1] + lv[1:])).astype(np.float32)
  assert codes[16, 0] == (3 if mid <= mids[3] else 4)
  deq = Q.dequantize(codes, s, g, Q.NF4)
  np.testing.assert_array_equal(deq[:16, 0], Q.rb_np(Q.rb_np(lv) * 4.0))
  # the unrounded reference mode keeps fp32 levels
  np.testing.assert_array_equal(Q.dequantize(codes, s, g, Q.NF4, round_levels=False)[:16, 0], lv * 4.0)


def test_nearest_level_brute_force():
  rng = np.random.default_rng(1)
  w = rng.normal(size=(64, 16)).astype(np.float32)
  for qtype in (Q.INT4, Q.NF4):
    codes, s = Q.quantize(w, 64, qtype)
    lv = Q.levels(qtype)
    x = w / s[0][None, :]
    if qtype == Q.INT4:
      best = np.clip(np.rint(x), -8, 7) + 8
    else:
      best = np.abs(x[..., None].astype(np.float64) - lv[None, None, :]).argmin(-1)
    np.testing.assert_array_equal(codes, best)


def test_zero_group_and_group_boundaries():
  K, N, g = 128, 16, 64
  w = np.zeros((K, N), dtype=np.float32)
  w[64:, :] = np.linspace(-3, 3, 64, dtype=np.float32)[:, None]
  for qtype in (Q.INT4, Q.NF4):
    codes, s = Q.quantize(w, g, qtype)
    assert (s[0] == 0).all() and (s[1] > 0).all()
    deq = Q.dequantize(codes, s, g, qtype)
    assert (deq[:64] == 0).all()
    assert np.abs(deq[64:] - w[64:]).max() <= (0.25 if qtype == Q.INT4 else 0.5)
  # scale linearity: doubling a group's weights doubles its scale and keeps the codes
  rng = np.random.default_rng(2)
  w = rng.normal(size=(K, N)).astype(np.float32)
  c1, s1 = Q.quantize(w, g, Q.NF4)
  w2 = w.copy()
  w2[:64] *= 2
  c2, s2 = Q.quantize(w2, g, Q.NF4)
  np.testing.assert_array_equal(c1, c2)
  np.testing.assert_array_equal(s2[0], 2 * s1[0])
  np.testing.assert_array_equal(s2[1], s1[1])


def test_qlinear_lora_closed_forms():
  rng = np.random.default_rng(3)
  M, K, N, r, g = 5, 128, 32, 8, 32
  w = rng.normal(size=(K, N)).astype(np.float32) * 0.05
  codes, s = Q.quantize(w, g, Q.INT4)
  x = Q.rb(torch.from_numpy(rng.normal(size=(M, K)).astype(np.float32)))
  a = Q.rb(torch.from_numpy(rng.normal(size=(K, r)).astype(np.float32) * 0.1))
  b = Q.rb(torch.from_numpy(rng.normal(size=(r, N)).astype(np.float32) * 0.1))
  wd = Q.dequantize(codes, s, g, Q.INT4).astype(np.float64)
  base = x.numpy().astype(np.float64) @ wd
  got = Q.qlinear_lora(x, codes, s, g, Q.INT4).numpy()
  np.testing.assert_allclose(got, base, rtol=1e-6, atol=1e-6)
  # B = 0: the adapter is a no-op
  got0 = Q.qlinear_lora(x, codes, s, g, Q.INT4, a, torch.zeros_like(b), 2.0).numpy()
  np.testing.assert_array_equal(got0, got)
  # fp32 reference mode equals the merged weight W + scale * A @ B (safetensors_saver.py:107)
  ref = Q.qlinear_lora(x, codes, s, g, Q.INT4, a, b, 0.5, bf16=False).numpy()
  wd32 = Q.dequantize(codes, s, g, Q.INT4, round_levels=False).astype(np.float64)
  merged = wd32 + 0.5 * (a.numpy().astype(np.float64) @ b.numpy().astype(np.float64))
  np.testing.assert_allclose(ref, x.numpy().astype(np.float64) @ merged, rtol=1e-5, atol=1e-6)
  # bf16 flow: t = bf16(x @ A) before the up-projection
  t = Q.rb(torch.from_numpy((x.numpy().astype(np.float64) @ a.numpy().astype(np.float64)).astype(np.float32)))
  want = base + 0.5 * (t.numpy().astype(np.float64) @ b.numpy().astype(np.float64))
  np.testing.assert_allclose(Q.qlinear_lora(x, codes, s, g, Q.INT4, a, b, 0.5).numpy(), want, rtol=1e-6, atol=1e-6)


def _unpack_brute(words, scales, K, N, group, interleave2):
  """Element-by-element reading of the QW layout as include/tunix_hip.h words it."""
  spt = max(2, 128 // group)
  ktiles = K // 128
  codes = np.zeros((K, N), dtype=np.uint8)
  sc = np.zeros((K // group, N), dtype=np.uint16)
  for c in range(N):
    pc = c
    if interleave2:
      half = N // 2
      h, cc = divmod(c, half)
      pc = (cc // 16) * 32 + h * 16 + cc % 16
    nt, lm = divmod(pc, 16)
    for k in range(K):
      kt, kk = divmod(k, 128)
      j, r = divmod(kk, 32)
      lq, i = divmod(r, 8)
      lane = lq * 16 + lm
      word = int(words[((nt * ktiles + kt) * 64 + lane) * 4 + j])
      codes[k, c] = (word >> (4 * i)) & 15
      slot = kk // (128 // spt)
      sc[k // group, c] = scales[((nt * ktiles + kt) * 16 + lm) * spt + slot]
  return codes, sc


def test_pack_qw_layout():
  rng = np.random.default_rng(4)
  for (K, N, group, il) in ((128, 32, 32, False), (256, 32, 64, True), (256, 16, 128, False), (512, 32, 256, True)):
    w = rng.normal(size=(K, N)).astype(np.float32)
    codes, s = Q.quantize(w, group, Q.NF4)
    words, sbits = Q.pack_qw(codes, s, group, il)
    assert words.size == K * N // 8
    c2, s2 = _unpack_brute(words, sbits, K, N, group, il)
    np.testing.assert_array_equal(c2, codes)
    want_bits = torch.from_numpy(s).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(s2, want_bits)


def test_int4_bound_parameter_closed_forms():
  """scale = bf16(absmax / bound): with bound 7 the group's extreme element maps to code 7 + 8 (or
  -7 + 8); with bound 8 a positive extreme would be 8 and clamps to 7 while a negative one uses
  the full -8; with 7.5 the scale rounds up to bf16(1 / 7.5) = 0.1337890625, so the extreme sits at
  7.47 and stays 7."""
  col = np.zeros((32, 1), dtype=np.float32)
  col[0, 0], col[1, 0], col[2, 0] = 1.0, -1.0, 0.5
  w = np.repeat(col, 16, axis=1)
  for bound, want_pos, want_neg, want_half in ((7.0, 7, -7, 4), (8.0, 7, -8, 4), (7.5, 7, -7, 4)):
    codes, s = Q.quantize(w, 32, Q.INT4, int4_bound=bound)
    np.testing.assert_array_equal(s, Q.rb_np(np.full((1, 16), 1.0 / bound, dtype=np.float32)))
    if bound == 7.5:
      assert float(s[0, 0]) == 0.1337890625
    q = codes.astype(np.int32) - 8
    # 0.5 / scale: 3.5 -> 4 (half to even), 4.0 -> 4, 3.75 -> 4 with the scales as rounded to bf16
    assert (q[0] == want_pos).all() and (q[1] == want_neg).all() and (q[2] == want_half).all(), (bound, q[:3, 0])
  a, _ = Q.quantize(w, 32, Q.INT4)
  b, _ = Q.quantize(w, 32, Q.INT4, int4_bound=7.0)
  np.testing.assert_array_equal(a, b)
  c_nf4, s_nf4 = Q.quantize(w, 32, Q.NF4, int4_bound=8.0)      # ignored for NF4
  np.testing.assert_array_equal(s_nf4, np.ones((1, 16), dtype=np.float32))
