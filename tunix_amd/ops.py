"""Thin Python wrappers over the C ABI: torch tensors in, kernels launched on torch's current
stream.  torch is used for device memory and streams only; every computation below happens in
libtunix_hip.so.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib as L


def _stream() -> int:
  return torch.cuda.current_stream().cuda_stream


def _ptr(t: torch.Tensor | None) -> int | None:
  if t is None:
    return None
  if not t.is_cuda:
    raise ValueError("expected a tensor on the GPU")
  if not t.is_contiguous():
    raise ValueError("expected a contiguous tensor")
  return t.data_ptr()


def _expect(t: torch.Tensor, dtype, what: str):
  if t.dtype != dtype:
    raise ValueError(f"{what}: expected {dtype}, got {t.dtype}")


def qw_sizes(K: int, N: int, group: int) -> tuple[int, int]:
  cb, sb = C.c_size_t(0), C.c_size_t(0)
  L.check(L.lib().tnx_qw_sizes(K, N, group, C.byref(cb), C.byref(sb)), "tnx_qw_sizes")
  return cb.value, sb.value


def quantize_pack(w: torch.Tensor, group: int, qtype: int, interleave2: bool = False, int4_bound: float = 7.0):
  """w [K,N] bf16 or fp32 on the GPU -> (codes int32 [K*N/8], scales bf16 [...]).  int4_bound: the
  integer a group's absmax maps to (scale = absmax / bound; ignored for NF4)."""
  K, N = w.shape
  cb, sb = qw_sizes(K, N, group)
  codes = torch.empty(cb // 4, dtype=torch.int32, device=w.device)
  scales = torch.empty(sb // 2, dtype=torch.bfloat16, device=w.device)
  scales[-8:] = 0   # the 16 bytes of tail padding the packer does not write
  is_f32 = 1 if w.dtype == torch.float32 else 0
  if not is_f32:
    _expect(w, torch.bfloat16, "quantize_pack")
  L.check(L.lib().tnx_quantize_pack(_stream(), _ptr(w), is_f32, K, N, group, qtype,
                                    1 if interleave2 else 0, float(int4_bound), _ptr(codes), _ptr(scales)),
          "tnx_quantize_pack")
  return codes, scales


def qw_dequant(codes, scales, K, N, group, qtype, interleave2=False) -> torch.Tensor:
  out = torch.empty(K, N, dtype=torch.float32, device=codes.device)
  L.check(L.lib().tnx_qw_dequant(_stream(), _ptr(codes), _ptr(scales), K, N, group, qtype,
                                 1 if interleave2 else 0, _ptr(out)), "tnx_qw_dequant")
  return out


def make_qlinear_desc(*, M, K, N, group, qtype, x, codes, scales, y, epilogue=L.TNX_EPI_STORE,
                      residual=None, lora_rank=0, lora_nseg=1, lora_seg_end=(), lora_seg_toff=(),
                      t=None, t_ld=0, lora_b=None, lora_scale=0.0, split_k=1, ws=None,
                      next_a_t=None, next_rank=0, next_tpart=None, w_expanded=None):
  d = L.QLinearDesc()
  d.M, d.K, d.N, d.group, d.qtype = M, K, N, group, qtype
  d.x, d.codes, d.scales, d.y = _ptr(x), _ptr(codes), _ptr(scales), _ptr(y)
  d.epilogue, d.residual = epilogue, _ptr(residual)
  d.lora_rank, d.lora_nseg = lora_rank, lora_nseg
  for i, v in enumerate(lora_seg_end):
    d.lora_seg_end[i] = v
  for i, v in enumerate(lora_seg_toff):
    d.lora_seg_toff[i] = v
  d.t, d.t_ld, d.lora_b, d.lora_scale = _ptr(t), t_ld, _ptr(lora_b), lora_scale
  d.split_k, d.ws = split_k, _ptr(ws)
  d.next_a_t, d.next_rank, d.next_tpart = _ptr(next_a_t), next_rank, _ptr(next_tpart)
  d.w_expanded = _ptr(w_expanded)
  return d


def qw_expand(codes, scales, K, N, group, qtype):
  """The second, converted copy of a packed weight for calls with many rows (tnx_qw_expand):
  bf16, 2 bytes per weight, in the many-row kernel's fragment order."""
  import torch
  n = int(L.lib().tnx_qw_expanded_bytes(K, N)) // 2
  out = torch.empty(n, dtype=torch.bfloat16, device=codes.device)
  L.check(L.lib().tnx_qw_expand(_stream(), _ptr(codes), _ptr(scales), K, N, group, qtype, _ptr(out)),
          "tnx_qw_expand")
  return out


def dense_expand(w):
  """The same copy for a dense bf16 matrix w [N, K] (an unquantised or tied lm_head [V, D])."""
  import torch
  N, K = w.shape
  out = torch.empty(int(L.lib().tnx_qw_expanded_bytes(K, N)) // 2, dtype=torch.bfloat16, device=w.device)
  L.check(L.lib().tnx_dense_expand(_stream(), _ptr(w), K, N, _ptr(out)), "tnx_dense_expand")
  return out


def qlinear(desc: L.QLinearDesc, finish: bool = True):
  """finish=False leaves the split-k partial planes in desc.ws for a consumer that sums them
  itself (rmsnorm_splitk)."""
  L.check(L.lib().tnx_qlinear_lora(_stream(), C.byref(desc)), "tnx_qlinear_lora")
  if desc.split_k > 1 and finish:
    L.check(L.lib().tnx_splitk_finish(_stream(), C.byref(desc)), "tnx_splitk_finish")


def lora_reduce(tpart, M, n_col_blocks, R, t):
  """t[M, :R] = bf16(sum of the fragment planes a *_MUL linear left in tpart)."""
  L.check(L.lib().tnx_lora_reduce(_stream(), _ptr(tpart), M, n_col_blocks, R, _ptr(t), t.shape[1]),
          "tnx_lora_reduce")


def lora_down(x, a_t, t, M=None):
  """t[M, :R] = bf16(x @ a_t.T); x [M,K], a_t [R,K], t [M, t_ld]."""
  M = x.shape[0] if M is None else M
  K = x.shape[1]
  R = a_t.shape[0]
  L.check(L.lib().tnx_lora_down(_stream(), _ptr(x), M, K, _ptr(a_t), R, _ptr(t), t.shape[1]),
          "tnx_lora_down")


def embed(table, ids, col_ptr, B, T, scale, out):
  V, D = table.shape
  L.check(L.lib().tnx_embed(_stream(), _ptr(table), V, D, _ptr(ids), ids.shape[1], _ptr(col_ptr),
                            B, T, float(scale), _ptr(out)), "tnx_embed")


def rmsnorm(x, w, y, eps, flavor, M=None, res_pre=None, h_out=None, res_post=None):
  M = x.shape[0] if M is None else M
  D = x.shape[1]
  L.check(L.lib().tnx_rmsnorm(_stream(), _ptr(x), _ptr(res_pre), _ptr(h_out), _ptr(w),
                              _ptr(res_post), _ptr(y), M, D, float(eps), flavor), "tnx_rmsnorm")


def rmsnorm_splitk(ws, split_k, w, y, eps, flavor, M, D, res_pre=None, h_out=None, res_post=None):
  """y = norm(h), h = bf16(bf16(sum_z ws[z]) + res_pre): the finishing pass of a split-k linear
  (N == D) folded into the residual add + norm that consumes it."""
  L.check(L.lib().tnx_rmsnorm_splitk(_stream(), _ptr(ws), split_k, _ptr(res_pre), _ptr(h_out), _ptr(w),
                                     _ptr(res_post), _ptr(y), M, D, float(eps), flavor),
          "tnx_rmsnorm_splitk")


def rmsnorm_moe_combine(y_route, topk_w, k, w, y, eps, flavor, M, D, res_pre=None, h_out=None, res_post=None):
  """y = norm(h), h = bf16(bf16(sum_j topk_w[m, j] * y_route[m * k + j]) + res_pre): the weighted
  combine of an MoE layer folded into the residual add + norm that consumes it."""
  L.check(L.lib().tnx_rmsnorm_moe_combine(_stream(), _ptr(y_route), _ptr(topk_w), k, _ptr(res_pre), _ptr(h_out),
                                          _ptr(w), _ptr(res_post), _ptr(y), M, D, float(eps), flavor),
          "tnx_rmsnorm_moe_combine")


def rmsnorm_pair(w, y, w2, y2, eps, flavor, M, D, x=None, ws=None, split_k=0, res_pre=None, h_out=None,
                 res_post=None):
  """y = [res_post +] norm(h) . w with h from x (or the split-k planes ws) [+ res_pre]; y2 = norm(y) . w2."""
  L.check(L.lib().tnx_rmsnorm_pair(_stream(), _ptr(x), _ptr(ws), split_k, _ptr(res_pre), _ptr(h_out),
                                   _ptr(w), _ptr(res_post), _ptr(y), _ptr(w2), _ptr(y2), M, D, float(eps),
                                   flavor), "tnx_rmsnorm_pair")


def rope_kvwrite(desc: L.RopeDesc):
  L.check(L.lib().tnx_qknorm_rope_kvwrite(_stream(), C.byref(desc)), "tnx_qknorm_rope_kvwrite")


def rope_table(positions, col_ptr, B, timescale, dh, sin_out, cos_out):
  L.check(L.lib().tnx_rope_table(_stream(), _ptr(positions), positions.shape[1], _ptr(col_ptr), B,
                                 _ptr(timescale), dh, _ptr(sin_out), _ptr(cos_out)), "tnx_rope_table")


def attn_ws_bytes(B, T, S, Hq, dh, kv_chunk) -> int:
  return int(L.lib().tnx_attn_ws_bytes(B, T, S, Hq, dh, kv_chunk))


def gqa_attn(desc: L.AttnDesc):
  L.check(L.lib().tnx_gqa_attn(_stream(), C.byref(desc)), "tnx_gqa_attn")


def lmhead_nblocks(V: int) -> int:
  return int(L.lib().tnx_lmhead_nblocks(V))


def lmhead(desc: L.LmHeadDesc):
  L.check(L.lib().tnx_lmhead_logp(_stream(), C.byref(desc)), "tnx_lmhead_logp")


def sample_topk_ws_bytes(M, V, k) -> int:
  return int(L.lib().tnx_sample_topk_ws_bytes(M, V, 0 if k is None else int(k)))


def sample_fullsort_ws_bytes(M, V) -> int:
  return int(L.lib().tnx_sample_fullsort_ws_bytes(M, V))


def sample_topk(logits, k, top_p, temperature, key, rng_variant, step_ptr, ws, ids_out, logp_out,
                forbidden=None):
  """logits: raw fp32 [M,V]; they are divided by `temperature` inside the kernel."""
  M, V = logits.shape
  L.check(L.lib().tnx_sample_topk(_stream(), _ptr(logits), M, V, k, float(top_p),
                                  float(temperature), key[0], key[1], rng_variant,
                                  _ptr(forbidden), 0 if forbidden is None else forbidden.numel(),
                                  _ptr(step_ptr), _ptr(ws), _ptr(ids_out), _ptr(logp_out)),
          "tnx_sample_topk")


def sample_topk_head_ok(V, k) -> bool:
  """Whether tnx_sample_topk_head takes this vocabulary size and top_k."""
  return bool(L.lib().tnx_sample_topk_head_ok(int(V), int(k)))


def sample_topk_head(logits, part, lse, k, top_p, temperature, key, rng_variant, step_ptr, ids_out, logp_out,
                     forbidden=None):
  """The top-k / top-p draw from the statistics a head call left behind (tnx_sample_topk_head):
  logits, part and lse are that call's logits_out, workspace and lse output, and the call used
  the same temperature and forbidden list."""
  M, V = logits.shape
  L.check(L.lib().tnx_sample_topk_head(_stream(), _ptr(logits), _ptr(part), _ptr(lse), M, V, int(k), float(top_p),
                                       float(temperature), key[0], key[1], rng_variant,
                                       _ptr(forbidden), 0 if forbidden is None else forbidden.numel(),
                                       _ptr(step_ptr), _ptr(ids_out), _ptr(logp_out)),
          "tnx_sample_topk_head")


def sample_commit(ids, logp, tokens, logprobs, done, eos, step_ptr):
  B = ids.shape[0]
  L.check(L.lib().tnx_sample_commit(_stream(), _ptr(ids), _ptr(logp), B, _ptr(tokens),
                                    tokens.shape[1], _ptr(logprobs), _ptr(done), _ptr(eos),
                                    0 if eos is None else eos.numel(), _ptr(step_ptr)),
          "tnx_sample_commit")


def moe_route_topk(scores, k, topk_w, topk_id):
  M, E = scores.shape
  L.check(L.lib().tnx_moe_route_topk(_stream(), _ptr(scores), M, E, k, _ptr(topk_w),
                                     _ptr(topk_id)), "tnx_moe_route_topk")


def moe_sort_routes(topk_id, E, counts, offsets, sorted_route):
  M, k = topk_id.shape
  L.check(L.lib().tnx_moe_sort_routes(_stream(), _ptr(topk_id), M, k, E, _ptr(counts),
                                      _ptr(offsets), _ptr(sorted_route)), "tnx_moe_sort_routes")


def moe_gmm(desc: L.MoeGmmDesc):
  L.check(L.lib().tnx_moe_int4_gmm(_stream(), C.byref(desc)), "tnx_moe_int4_gmm")


def moe_combine(y, topk_w, M, k, D, residual, out):
  L.check(L.lib().tnx_moe_combine(_stream(), _ptr(y), _ptr(topk_w), M, k, D, _ptr(residual),
                                  _ptr(out)), "tnx_moe_combine")


def grpo_ratio(logp, old_logp, adv, tokens_per_seq, eps_lo, eps_hi, ratio=None, loss=None,
               clipped=None):
  N = logp.numel()
  L.check(L.lib().tnx_grpo_ratio(_stream(), _ptr(logp), _ptr(old_logp), _ptr(adv), N,
                                 tokens_per_seq, float(eps_lo), float(eps_hi), _ptr(ratio),
                                 _ptr(loss), _ptr(clipped)), "tnx_grpo_ratio")


KL_METHODS = {"kl": 0, "mse_kl": 1, "low_var_kl": 2}
AGG_MODES = {"token-mean": 0, "sequence-mean-token-mean": 1, "sequence-mean-token-scale": 2,
             "seq-mean-token-sum": 3, "sequence-mean-token-sum-norm": 4}


def kl_divergence(logp, ref_logp, method: int, clamp: float, out):
  L.check(L.lib().tnx_kl_divergence(_stream(), _ptr(logp), _ptr(ref_logp), logp.numel(), method,
                                    float(clamp), _ptr(out)), "tnx_kl_divergence")


def aggregate_loss(per_token_loss, mask, mode: int, norm: float, row_ws, out):
  B, T = per_token_loss.shape
  L.check(L.lib().tnx_aggregate_loss(_stream(), _ptr(per_token_loss), _ptr(mask), B, T, mode,
                                     float(norm), _ptr(row_ws), _ptr(out)), "tnx_aggregate_loss")


def aggregate_loss_segmented(per_token_loss, mask, segment_ids, num_segments: int, mode: int, norm: float, out):
  B, T = per_token_loss.shape
  nb = int(L.lib().tnx_aggregate_loss_segmented_ws_bytes(B, num_segments))
  ws = torch.empty(nb // 4, dtype=torch.float32, device=out.device)
  L.check(L.lib().tnx_aggregate_loss_segmented(_stream(), _ptr(per_token_loss), _ptr(mask), _ptr(segment_ids), B, T,
                                               int(num_segments), mode, float(norm), _ptr(ws), _ptr(out)),
          "tnx_aggregate_loss_segmented")


def logp_drift(rollout_logp, trainer_logp, mask, out5):
  B, T = rollout_logp.shape
  ws = torch.empty(int(L.lib().tnx_logp_drift_ws_bytes(B)) // 8, dtype=torch.float64, device=out5.device)
  L.check(L.lib().tnx_logp_drift(_stream(), _ptr(rollout_logp), _ptr(trainer_logp), _ptr(mask), B, T,
                                 _ptr(ws), _ptr(out5)), "tnx_logp_drift")


def logp_drift_static(rollout_logp, trainer_logp, mask, out5):
  """tnx_logp_drift with the library's built-in scratch: no workspace, nothing allocated."""
  B, T = rollout_logp.shape
  L.check(L.lib().tnx_logp_drift_static(_stream(), _ptr(rollout_logp), _ptr(trainer_logp), _ptr(mask), B, T,
                                        _ptr(out5)), "tnx_logp_drift_static")


def fill_u32(t: torch.Tensor, value: int = 0):
  assert t.element_size() == 4
  L.check(L.lib().tnx_fill_u32(_stream(), _ptr(t), t.numel(), value), "tnx_fill_u32")
