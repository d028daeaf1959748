"""Group-quantised weights (int4 symmetric / NF4) and the quantised linear + LoRA (oracle).

The quantised arithmetic of the reference lives in the third-party package qwix
(pyproject.toml:43, reached from tunix/cli/utils/model.py:31-77); it is absent from the
reference tree, so this file restates the format that include/tunix_hip.h defines:

  scale[g, n] = bf16(absmax / 7)  (int4)   |  bf16(absmax)  (NF4), groups of `group`
                consecutive K indices per output column n
  code        = clamp(rint(w / f32(scale)), -8, 7) + 8   (int4, round-half-even)
              = index of the nearest NF4 level of w / f32(scale), ties to the lower code
  value       = w^[k, n] = bf16(bf16(level(code)) * scale): the weight "dequantised to bf16"
                (qvalue.astype(scale dtype) * scale), then a bf16 matmul with fp32 accumulation:
                y[m, n] = sum_k x[m, k] * w^[k, n]
  LoRA        y += (alpha / rank) * bf16(x @ A) @ B        (tunix/models/safetensors_saver.py:107
                                                            W_eff = W + (A @ B) * alpha / rank)

PARITY UNPINNED against qwix itself (no golden vector of a quantised result exists in the
reference tree); pinned by closed forms in tests/test_oracle_quant.py.
"""
from __future__ import annotations

import numpy as np
import torch

NF4_LEVELS = np.array(
    [-1.0, -0.6961928, -0.52507305, -0.39491749, -0.28444138, -0.18477343, -0.09105004, 0.0,
     0.0795803, 0.1609302, 0.2461123, 0.33791524, 0.44070983, 0.562617, 0.72295684, 1.0],
    dtype=np.float32)
INT4_LEVELS = np.arange(-8, 8, dtype=np.float32)
INT4, NF4 = 0, 1


def rb(x: torch.Tensor) -> torch.Tensor:
  """Round an fp32 tensor to bf16 precision (round-to-nearest-even), keeping fp32 storage."""
  return x.to(torch.float32).to(torch.bfloat16).to(torch.float32)


def rb_np(x: np.ndarray) -> np.ndarray:
  return rb(torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32))).numpy()


def levels(qtype: int) -> np.ndarray:
  return NF4_LEVELS if qtype == NF4 else INT4_LEVELS


def quantize(w: np.ndarray, group: int, qtype: int, int4_bound: float = 7.0) -> tuple[np.ndarray, np.ndarray]:
  """w fp32 [K, N] -> (codes uint8 [K, N] in 0..15, scales fp32 [K/group, N] holding bf16 values).
  int4_bound: the integer a group's absmax maps to (7 in the format's definition; a quantiser
  with another symmetric bound is mirrored by passing it, codes still clamp to [-8, 7])."""
  w = np.asarray(w, dtype=np.float32)
  K, N = w.shape
  assert K % group == 0
  wg = w.reshape(K // group, group, N)
  amax = np.abs(wg).max(axis=1)
  scale = rb_np(amax if qtype == NF4 else amax / np.float32(int4_bound))
  safe = np.where(scale == 0, np.float32(1.0), scale)
  xn = (wg / safe[:, None, :]).astype(np.float32)
  if qtype == NF4:
    mids = (np.float32(0.5) * (NF4_LEVELS[:-1] + NF4_LEVELS[1:])).astype(np.float32)
    # number of midpoints strictly below x == index of the nearest level, ties to the lower code
    codes = np.searchsorted(mids, xn, side="left").astype(np.uint8)
    codes = np.where(scale[:, None, :] == 0, np.uint8(7), codes)
  else:
    q = np.clip(np.rint(xn), -8, 7)
    codes = (q + 8).astype(np.uint8)
    codes = np.where(scale[:, None, :] == 0, np.uint8(8), codes)
  return codes.reshape(K, N), scale


def dequantize(codes: np.ndarray, scale: np.ndarray, group: int, qtype: int,
               round_levels: bool = True) -> np.ndarray:
  """fp32 [K, N]: bf16(bf16(level) * scale); round_levels=False is the fp32 reference mode
  (fp32 level * scale, no rounding)."""
  lv = levels(qtype)
  if round_levels:
    lv = rb_np(lv)
  K, N = codes.shape
  s = np.repeat(scale, group, axis=0)
  w = (lv[codes].astype(np.float64) * s.astype(np.float64)).astype(np.float32)
  return rb_np(w) if round_levels else w


def qlinear_lora(x: torch.Tensor, codes: np.ndarray, scale: np.ndarray, group: int, qtype: int,
                 lora_a: torch.Tensor | None = None, lora_b: torch.Tensor | None = None,
                 lora_scale: float = 1.0, acc=torch.float64, bf16: bool = True) -> torch.Tensor:
  """fp32 result (not yet rounded) of x[M,K] @ dequant(W)[K,N] + lora_scale * bf16(x@A) @ B.

  bf16=True follows the kernel's dtype flow (bf16 level, bf16 t); bf16=False is the
  fp32 reference mode (fp32 levels, no rounding of t).
  """
  wd = torch.from_numpy(dequantize(codes, scale, group, qtype, round_levels=bf16))
  y = x.to(acc) @ wd.to(acc)
  if lora_a is not None:
    t = (x.to(acc) @ lora_a.to(acc)).to(torch.float32)
    if bf16:
      t = rb(t)
    y = y + float(lora_scale) * (t.to(acc) @ lora_b.to(acc))
  return y.to(torch.float32)


# ---- the packed "QW" layout of include/tunix_hip.h, for checking tnx_quantize_pack ----------
def packed_col(c: np.ndarray, N: int, interleave2: bool) -> np.ndarray:
  if not interleave2:
    return c
  half = N // 2
  h, cc = c // half, c % half
  return (cc // 16) * 32 + h * 16 + (cc % 16)


def pack_qw(codes: np.ndarray, scale: np.ndarray, group: int, interleave2: bool = False):
  """codes uint8 [K,N], scale [K/group,N] -> (uint32 codes array, uint16 scales array)."""
  K, N = codes.shape
  assert K % 128 == 0 and N % 16 == 0
  ktiles, ntiles = K // 128, N // 16
  spt = 2 if group >= 64 else 128 // group   # scale slots per k-tile and column
  slot_w = 128 // spt
  pc = packed_col(np.arange(N), N, interleave2)
  cp = np.empty_like(codes)
  cp[:, pc] = codes
  # [kt, j, lq, i, nt, lm] -> [nt, kt, lq, lm, j, i]
  c6 = cp.reshape(ktiles, 4, 4, 8, ntiles, 16).transpose(4, 0, 2, 5, 1, 3).astype(np.uint32)
  shifts = (4 * np.arange(8, dtype=np.uint32))
  words = (c6 << shifts).sum(axis=-1, dtype=np.uint64).astype(np.uint32)  # [nt, kt, lq, lm, j]
  out_codes = words.reshape(-1)
  sbits = torch.from_numpy(np.ascontiguousarray(scale, dtype=np.float32)).to(
      torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
  sp = np.empty_like(sbits)
  sp[:, pc] = sbits
  per_slot = np.repeat(sp, group, axis=0)[::slot_w]      # [K / slot_w, N]
  st = per_slot.reshape(ktiles, spt, ntiles, 16)
  out_scales = st.transpose(2, 0, 3, 1).reshape(-1)       # [nt][kt][16][spt]
  return out_codes, np.ascontiguousarray(out_scales)
