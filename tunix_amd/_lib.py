"""ctypes binding of libtunix_hip.so (the C ABI declared in include/tunix_hip.h).

The library is the product: there is no CPU or eager-PyTorch fallback.  If the shared object
is missing or fails to load, importing a kernel wrapper raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtunix_hip.so")

# the ABI this binding was written against (TNX_ABI_VERSION_MAJOR / _MINOR of include/tunix_hip.h)
ABI_VERSION = (3, 1)

TNX_Q_INT4, TNX_Q_NF4 = 0, 1
TNX_NORM_LLAMA, TNX_NORM_QWEN3, TNX_NORM_GEMMA3 = 0, 1, 2
TNX_ROPE_LLAMA, TNX_ROPE_QWEN3, TNX_ROPE_GEMMA3 = 0, 1, 2
TNX_EPI_STORE, TNX_EPI_RESIDUAL, TNX_EPI_SILU_MUL, TNX_EPI_GELU_MUL, TNX_EPI_F32 = 0, 1, 2, 3, 4

_p = C.c_void_p
_i64 = C.c_int64
_i32 = C.c_int
_f32 = C.c_float


class QLinearDesc(C.Structure):
  _fields_ = [
      ("M", _i64), ("K", _i64), ("N", _i64),
      ("group", _i32), ("qtype", _i32),
      ("x", _p), ("codes", _p), ("scales", _p),
      ("lora_rank", _i32), ("lora_nseg", _i32),
      ("lora_seg_end", _i64 * 4), ("lora_seg_toff", _i32 * 4),
      ("t_ld", _i64), ("t", _p), ("lora_b", _p), ("lora_scale", _f32),
      ("epilogue", _i32), ("residual", _p), ("y", _p),
      ("split_k", _i32), ("ws", _p),
      ("next_a_t", _p), ("next_rank", _i32), ("next_tpart", _p),
      ("w_expanded", _p),
  ]


class RopeDesc(C.Structure):
  _fields_ = [
      ("B", _i64), ("T", _i64), ("S", _i64),
      ("Hq", _i32), ("Hkv", _i32), ("dh", _i32),
      ("rope_flavor", _i32), ("rope_scale", _f32), ("timescale", _p),
      ("qk_norm", _i32), ("norm_eps", _f32),
      ("q_norm_w", _p), ("k_norm_w", _p), ("q_prescale", _f32),
      ("qkv", _p), ("positions", _p), ("pos_ld", _i64), ("col_ptr", _p),
      ("q_out", _p), ("kcache", _p), ("vcache", _p),
      ("qkv_ws", _p), ("split_k", _i32),
  ]


class AttnDesc(C.Structure):
  _fields_ = [
      ("B", _i64), ("T", _i64), ("S", _i64),
      ("Hq", _i32), ("Hkv", _i32), ("dh", _i32),
      ("scale", _f32), ("window", _i32), ("pad_id", C.c_int32),
      ("q", _p), ("kcache", _p), ("vcache", _p),
      ("tokens", _p), ("tok_ld", _i64), ("col_ptr", _p),
      ("kv_chunk", _i32), ("ws", _p), ("out", _p),
      ("qkv_ws", _p), ("qkv", _p), ("qkv_split", _i32), ("rope_sin", _p), ("rope_cos", _p),
      ("segment_ids", _p),
  ]


class LmHeadDesc(C.Structure):
  _fields_ = [
      ("M", _i64), ("D", _i64), ("V", _i64),
      ("x", _p), ("w_bf16", _p), ("codes", _p), ("scales", _p),
      ("group", _i32), ("qtype", _i32), ("lora_rank", _i32),
      ("t", _p), ("t_ld", _i64), ("lora_b", _p), ("lora_scale", _f32),
      ("temperature", _f32), ("forbidden", _p), ("n_forbidden", _i32),
      ("targets", _p), ("part", _p), ("best_id", _p), ("best_logp", _p),
      ("target_logp", _p), ("lse", _p), ("logits_out", _p),
      ("part_entropy", _p), ("entropy", _p),
      ("part_draw", _p), ("draw_key0", C.c_uint32), ("draw_key1", C.c_uint32), ("draw_rng_variant", _i32),
      ("draw_step_ptr", _p), ("draw_id", _p), ("draw_logp", _p), ("logits_fp32", _i32),
      ("w_expanded", _p),
  ]


class MoeGmmDesc(C.Structure):
  _fields_ = [
      ("n_routes", _i64), ("E", _i32), ("k", _i32), ("K", _i64), ("N", _i64),
      ("group", _i32), ("qtype", _i32), ("x", _p), ("x_div", _i32),
      ("codes", _p), ("scales", _p), ("offsets", _p), ("sorted_route", _p),
      ("epilogue", _i32), ("y", _p),
  ]


# name -> (restype, argtypes); every symbol include/tunix_hip.h declares.
SIGNATURES = {
    "tnx_last_error": (C.c_char_p, []),
    "tnx_version": (_i32, []),
    "tnx_qw_sizes": (_i32, [_i64, _i64, _i32, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "tnx_quantize_pack": (_i32, [_p, _p, _i32, _i64, _i64, _i32, _i32, _i32, _f32, _p, _p]),
    "tnx_qw_dequant": (_i32, [_p, _p, _p, _i64, _i64, _i32, _i32, _i32, _p]),
    "tnx_qw_expanded_bytes": (C.c_size_t, [_i64, _i64]),
    "tnx_qw_expand": (_i32, [_p, _p, _p, _i64, _i64, _i32, _i32, _p]),
    "tnx_dense_expand": (_i32, [_p, _p, _i64, _i64, _p]),
    "tnx_qlinear_lora": (_i32, [_p, C.POINTER(QLinearDesc)]),
    "tnx_splitk_finish": (_i32, [_p, C.POINTER(QLinearDesc)]),
    "tnx_lora_reduce": (_i32, [_p, _p, _i64, _i64, _i32, _p, _i64]),
    "tnx_lora_down": (_i32, [_p, _p, _i64, _i64, _p, _i32, _p, _i64]),
    "tnx_embed": (_i32, [_p, _p, _i64, _i64, _p, _i64, _p, _i64, _i64, _f32, _p]),
    "tnx_rmsnorm": (_i32, [_p, _p, _p, _p, _p, _p, _p, _i64, _i64, _f32, _i32]),
    "tnx_rmsnorm_splitk": (_i32, [_p, _p, _i32, _p, _p, _p, _p, _p, _i64, _i64, _f32, _i32]),
    "tnx_rmsnorm_moe_combine": (_i32, [_p, _p, _p, _i32, _p, _p, _p, _p, _p, _i64, _i64, _f32, _i32]),
    "tnx_rmsnorm_pair": (_i32, [_p, _p, _p, _i32, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _f32, _i32]),
    "tnx_qknorm_rope_kvwrite": (_i32, [_p, C.POINTER(RopeDesc)]),
    "tnx_rope_table": (_i32, [_p, _p, _i64, _p, _i64, _p, _i32, _p, _p]),
    "tnx_attn_ws_bytes": (C.c_size_t, [_i64, _i64, _i64, _i32, _i32, _i32]),
    "tnx_gqa_attn": (_i32, [_p, C.POINTER(AttnDesc)]),
    "tnx_lmhead_nblocks": (_i64, [_i64]),
    "tnx_lmhead_logp": (_i32, [_p, C.POINTER(LmHeadDesc)]),
    "tnx_sample_topk_ws_bytes": (C.c_size_t, [_i64, _i64, _i32]),
    "tnx_sample_fullsort_ws_bytes": (C.c_size_t, [_i64, _i64]),
    "tnx_sample_topk": (_i32, [_p, _p, _i64, _i64, _i32, _f32, _f32, C.c_uint32, C.c_uint32, _i32,
                               _p, _i32, _p, _p, _p, _p]),
    "tnx_sample_topk_head_ok": (_i32, [_i64, _i32]),
    "tnx_sample_topk_head": (_i32, [_p, _p, _p, _p, _i64, _i64, _i32, _f32, _f32, C.c_uint32, C.c_uint32, _i32,
                                    _p, _i32, _p, _p, _p]),
    "tnx_sample_commit": (_i32, [_p, _p, _p, _i64, _p, _i64, _p, _p, _p, _i32, _p]),
    "tnx_moe_route_topk": (_i32, [_p, _p, _i64, _i32, _i32, _p, _p]),
    "tnx_moe_sort_routes": (_i32, [_p, _p, _i64, _i32, _i32, _p, _p, _p]),
    "tnx_moe_int4_gmm": (_i32, [_p, C.POINTER(MoeGmmDesc)]),
    "tnx_moe_combine": (_i32, [_p, _p, _p, _i64, _i32, _i64, _p, _p]),
    "tnx_grpo_ratio": (_i32, [_p, _p, _p, _p, _i64, _i64, _f32, _f32, _p, _p, _p]),
    "tnx_kl_divergence": (_i32, [_p, _p, _p, _i64, _i32, _f32, _p]),
    "tnx_aggregate_loss": (_i32, [_p, _p, _p, _i64, _i64, _i32, _f32, _p, _p]),
    "tnx_aggregate_loss_segmented_ws_bytes": (C.c_size_t, [_i64, _i32]),
    "tnx_aggregate_loss_segmented": (_i32, [_p, _p, _p, _p, _i64, _i64, _i32, _i32, _f32, _p, _p]),
    "tnx_logp_drift_ws_bytes": (C.c_size_t, [_i64]),
    "tnx_logp_drift": (_i32, [_p, _p, _p, _p, _i64, _i64, _p, _p]),
    "tnx_logp_drift_static_max_rows": (_i64, []),
    "tnx_logp_drift_static": (_i32, [_p, _p, _p, _p, _i64, _i64, _p]),
    "tnx_fill_u32": (_i32, [_p, _p, _i64, C.c_uint32]),
}

_lib = None


class TnxError(RuntimeError):
  """A libtunix_hip.so entry point returned a negative code."""


def lib() -> C.CDLL:
  """Loads libtunix_hip.so once; raises if it was not built (no fallback exists)."""
  global _lib
  if _lib is None:
    if not os.path.exists(LIB_PATH):
      raise ImportError(
          f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; "
          "g.build()'` (hipcc --offload-arch=gfx950); there is no CPU fallback"
      )
    handle = C.CDLL(LIB_PATH)
    handle.tnx_version.restype = _i32
    v = handle.tnx_version()
    if (v >> 16) != ABI_VERSION[0] or (v & 0xffff) < ABI_VERSION[1]:
      raise ImportError(f"{LIB_PATH} has ABI version {v >> 16}.{v & 0xffff}; this binding needs "
                        f"{ABI_VERSION[0]}.x with x >= {ABI_VERSION[1]} (rebuild the library)")
    for name, (res, args) in SIGNATURES.items():
      fn = getattr(handle, name)
      fn.restype = res
      fn.argtypes = args
    _lib = handle
  return _lib


def check(rc: int, what: str) -> None:
  if rc != 0:
    msg = lib().tnx_last_error().decode("utf-8", "replace")
    if rc == -22:
      raise ValueError(f"{what}: {msg}")
    raise TnxError(f"{what} failed with code {rc}: {msg}")
