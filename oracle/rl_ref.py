"""Per-token log-probabilities, KL estimators, loss aggregation and the GRPO clipped ratio
(oracle; tests only).

Follows tunix/rl/common.py:135-203, :234-291, :326-571, :704-760 (segment sums), :763-940,
tunix/rl/algo_core.py:440-489 and tunix/rl/grpo/grpo_learner.py:405-440.
"""
from __future__ import annotations

import numpy as np
import torch

from . import utils_ref as U


def compute_kl_divergence(logps, ref_logps, method="low_var_kl", clamp_value=None):
  """tunix/rl/common.py:135-184."""
  logps = np.asarray(logps, dtype=np.float32)
  ref = np.asarray(ref_logps, dtype=np.float32)
  if method == "kl":
    kl = logps - ref
  elif method == "mse_kl":
    kl = 0.5 * np.square(logps - ref)
  elif method == "low_var_kl":
    diff = ref - logps
    kl = np.exp(diff) - diff - 1
  else:
    raise ValueError("`method` must be one of 'kl', 'mse_kl', 'low_var_kl'. Received:"
                     f" {method}")
  if clamp_value is not None:
    kl = np.clip(kl, -clamp_value, clamp_value)
  return kl


def selective_log_softmax(logits: torch.Tensor, input_ids: torch.Tensor) -> torch.Tensor:
  """tunix/rl/common.py:187-203: f32(logit[target]) - logsumexp(f32(logits))."""
  lg = logits.to(torch.float32)
  tgt = torch.gather(lg, -1, input_ids.long()[..., None]).squeeze(-1)
  return tgt - torch.logsumexp(lg, dim=-1)


def segment_attn_mask(segment_ids: np.ndarray) -> np.ndarray:
  """[B, L, L] bool: query i attends key j iff j <= i and both carry the same segment id -- what the
  splash-attention path of the packed mode computes from a causal mask kernel plus
  SegmentIds(q, kv) (tunix/models/qwen3/model.py:622-655)."""
  seg = np.asarray(segment_ids)
  L = seg.shape[1]
  causal = np.tril(np.ones((L, L), dtype=bool))
  return (seg[:, :, None] == seg[:, None, :]) & causal[None]


def process_ids(prompt_tokens: np.ndarray, completion_tokens: np.ndarray, pad_id: int,
                segment_ids=None, segment_positions=None):
  """tunix/rl/common.py:234-291.  Packed branch (:260-271): positions are the caller's
  segment_positions (required), no padding mask; the model separates sequences by segment id."""
  ids = np.concatenate([prompt_tokens, completion_tokens], axis=1)
  if segment_ids is not None:
    if segment_positions is None:
      raise ValueError("segment_positions must be explicitly provided for packed sequences. ")
    return ids, np.asarray(segment_positions), segment_attn_mask(segment_ids)
  mask = np.concatenate([prompt_tokens != pad_id, completion_tokens != pad_id], axis=-1)
  positions = U.build_positions_from_mask(mask)
  attn_mask = U.make_causal_attn_mask(mask)
  return ids, positions, attn_mask


def compute_entropy_from_logits(logits: torch.Tensor) -> torch.Tensor:
  """tunix/rl/common.py:1136-1148: log_probs = log_softmax(logits); probs = softmax(log_probs);
  entropy = -sum(probs * log_probs) over the last axis."""
  lp = torch.log_softmax(logits.to(torch.float32), dim=-1)
  pr = torch.softmax(lp, dim=-1)
  return -(pr * lp).sum(-1)


def compute_per_token_logps(ref_model, prompt_tokens, completion_tokens, pad_id,
                            temperature: float = 1.0, chunk_size: int = 0, return_entropy: bool = False,
                            segment_ids=None, segment_positions=None):
  """tunix/rl/common.py:326-482: one full forward without cache, logits[:, -T-1:-1],
  optional temperature, gather - logsumexp.  chunk_size > 0 follows compute_chunked_logps
  (:485-571): the head is applied per sequence chunk.  Packed mode (segment_ids, :408-418): the
  whole buffer is scored, logits_to_keep = L - 1, and the result is padded in front with one 0.0
  so that logp[i] belongs to token[i] (:440-443, :468-472)."""
  ids, positions, attn_mask = process_ids(np.asarray(prompt_tokens), np.asarray(completion_tokens),
                                          pad_id, segment_ids, segment_positions)
  B, Ltot = ids.shape
  T = completion_tokens.shape[1] if segment_ids is None else Ltot - 1
  inner = _logps_of_last(ref_model, ids, positions, attn_mask, T, temperature, chunk_size, return_entropy)
  if segment_ids is None:
    return inner
  pad = lambda x: torch.cat([torch.zeros(B, 1, dtype=x.dtype), x], dim=1)
  return (pad(inner[0]), pad(inner[1])) if return_entropy else pad(inner)


def _logps_of_last(ref_model, ids, positions, attn_mask, T, temperature, chunk_size, return_entropy):
  """Shared tail of compute_per_token_logps: forward, keep logits[:, -T-1:-1], gather."""
  B, Ltot = ids.shape
  cache = ref_model.init_cache(B, Ltot)
  tok = torch.from_numpy(ids.astype(np.int64))
  h = ref_model.hidden(tok, torch.from_numpy(positions.astype(np.int64)), cache,
                       torch.from_numpy(attn_mask), 0)
  hk = h[:, -T - 1:-1]
  targets = tok[:, -T:]

  def head(hh):
    lg = ref_model.logits(hh).to(torch.float32)
    if temperature != 0.0 and temperature != 1.0:
      lg = lg / np.float32(temperature)
    return lg

  if chunk_size > 0:
    outs = []
    for s in range(0, T, chunk_size):
      outs.append(selective_log_softmax(head(hk[:, s:s + chunk_size]), targets[:, s:s + chunk_size]))
    return torch.cat(outs, dim=1)
  if return_entropy:  # :479-481, on the same (temperature-scaled) logits
    lg = head(hk)
    return selective_log_softmax(lg, targets), compute_entropy_from_logits(lg)
  return selective_log_softmax(head(hk), targets)


def grpo_ratio(logp, old_logp, adv, eps_lo, eps_hi):
  """tunix/rl/algo_core.py:440-489: clipped importance ratio and per-token loss."""
  logp = np.asarray(logp, dtype=np.float32)
  old = logp if old_logp is None else np.asarray(old_logp, dtype=np.float32)
  lr = np.clip(logp - old, -20.0, 20.0).astype(np.float32)
  ratio = np.exp(lr).astype(np.float32)
  a = np.asarray(adv, dtype=np.float32)
  a = a if a.ndim == logp.ndim else a[..., None]
  l1 = -a * ratio
  l2 = -a * np.clip(ratio, np.float32(1 - eps_lo), np.float32(1 + eps_hi))
  return ratio, np.maximum(l1, l2).astype(np.float32), (l2 > l1)


def aggregate_loss(per_token_loss, completion_mask, loss_agg_mode, **kwargs):
  """tunix/rl/common.py:763-854 without packing segments, in float64:
  (unreduced_sum, denominator, min_denom)."""
  loss = np.asarray(per_token_loss, dtype=np.float64)
  mask = np.asarray(completion_mask, dtype=np.float64)

  def get_norm(default):  # tunix/rl/common.py:1151-1177
    if "norm" in kwargs:
      try:
        norm = float(kwargs["norm"])
      except (ValueError, TypeError):
        raise ValueError(f"Invalid 'norm' value: {kwargs['norm']}. Must be a positive number.")
      if norm <= 0:
        raise ValueError(f"Invalid 'norm' value: {norm}. Must be a positive number.")
      return norm
    return default

  if loss_agg_mode == "token-mean":
    return (loss * mask).sum(), mask.sum(), 1.0
  if loss_agg_mode == "sequence-mean-token-mean":
    seq_mask = mask.sum(axis=-1)
    seq_loss = (loss * mask).sum(axis=-1) / np.clip(seq_mask, 1.0, None)
    return seq_loss.sum(), float((seq_mask > 0).sum()), 1.0
  if loss_agg_mode == "sequence-mean-token-scale":
    norm = get_norm(loss.shape[-1])
    seq_loss = (loss * mask).sum(axis=-1) / max(norm, 1e-6)
    return seq_loss.sum(), float((mask.sum(axis=-1) > 0).sum()), 1.0
  if loss_agg_mode == "seq-mean-token-sum":
    seq_loss = (loss * mask).sum(axis=-1)
    seq_mask = (mask.sum(axis=-1) > 0).astype(np.float64)
    return (seq_loss * seq_mask).sum(), seq_mask.sum(), 1e-6
  if loss_agg_mode == "sequence-mean-token-sum-norm":
    norm = get_norm(loss.shape[0])
    return (loss * mask).sum(), float(norm), 1e-6
  raise ValueError(f"Unsupported loss aggregation mode: {loss_agg_mode}.")


def segmented_sum(values, segment_ids, num_segments):
  """tunix/rl/common.py:704-735: per-row sums of `values` grouped by segment id -> [B, S]; ids
  outside [0, S) are dropped, as jax.ops.segment_sum drops them."""
  values = np.asarray(values, dtype=np.float64)
  seg = np.asarray(segment_ids).astype(np.int64)
  out = np.zeros((values.shape[0], num_segments), dtype=np.float64)
  for b in range(values.shape[0]):
    for t in range(values.shape[1]):
      s = seg[b, t]
      if 0 <= s < num_segments:
        out[b, s] += values[b, t]
  return out


def aggregate_loss_segmented(per_token_loss, completion_mask, loss_agg_mode, segment_ids, num_segments,
                             **kwargs):
  """tunix/rl/common.py:857-940 (_aggregate_loss_segmented), in float64: per-sequence reductions
  group by packing segment instead of by row, segment 0 (padding) is excluded, a segment counts
  when it has at least one scored token.  Returns (unreduced_sum, denominator, min_denom)."""
  if num_segments is None:
    raise ValueError("num_segments must be provided when segment_ids is not None.")
  loss = np.asarray(per_token_loss, dtype=np.float64)
  mask = np.asarray(completion_mask, dtype=np.float64)
  masked = loss * mask
  l_seg = segmented_sum(masked, segment_ids, num_segments)
  c_seg = segmented_sum(mask, segment_ids, num_segments)
  a_seg = (c_seg > 0).astype(np.float64)
  a_seg[:, 0] = 0.0
  n_act = a_seg.sum()

  def get_norm(default):
    if "norm" in kwargs:
      try:
        norm = float(kwargs["norm"])
      except (ValueError, TypeError):
        raise ValueError(f"Invalid 'norm' value: {kwargs['norm']}. Must be a positive number.")
      if norm <= 0:
        raise ValueError(f"Invalid 'norm' value: {norm}. Must be a positive number.")
      return norm
    return default

  if loss_agg_mode == "token-mean":
    return masked.sum(), mask.sum(), 1.0
  if loss_agg_mode == "sequence-mean-token-mean":
    return ((l_seg / np.clip(c_seg, 1.0, None)) * a_seg).sum(), n_act, 1.0
  if loss_agg_mode == "sequence-mean-token-scale":
    if "norm" not in kwargs:
      raise ValueError("sequence-mean-token-scale under sequence packing requires an explicit 'norm'")
    norm = get_norm(loss.shape[-1])
    return ((l_seg / max(norm, 1e-6)) * a_seg).sum(), n_act, 1.0
  if loss_agg_mode == "seq-mean-token-sum":
    return (l_seg * a_seg).sum(), n_act, 1e-6
  if loss_agg_mode == "sequence-mean-token-sum-norm":
    return masked.sum(), float(get_norm(n_act)), 1e-6
  raise ValueError(f"Unsupported loss aggregation mode: {loss_agg_mode}.")


def weighted_metric_compute(unreduced_sum, denominator, min_denom=None, eps=None):
  """WeightedMetric.compute, tunix/sft/utils.py:201-219."""
  denom = float(denominator)
  if eps is not None:
    denom = denom + eps
  if min_denom is not None:
    denom = max(denom, min_denom)
  return 0.0 if denom == 0 else float(unreduced_sum) / denom


def sampler_trainer_agreement(rollout_logps, trainer_logps, completion_mask):
  """tunix/rl/grpo/grpo_learner.py:405-440, fp32 as there: how far the log-probabilities recorded
  by the rollout are from the ones the trainer recomputes, over the completion tokens."""
  a = np.asarray(rollout_logps, dtype=np.float32)
  b = np.asarray(trainer_logps, dtype=np.float32)
  mask = np.asarray(completion_mask).astype(bool)
  mask_f = mask.astype(np.float32)
  mask_sum = np.maximum(mask_f.sum(dtype=np.float32), np.float32(1.0))
  diff = np.abs(a - b)
  rp, tp = np.exp(a), np.exp(b)
  prob_diff = np.abs(rp - tp)
  rp_flat, tp_flat, mf = rp.reshape(-1), tp.reshape(-1), mask_f.reshape(-1)
  rp_mean = (rp_flat * mf).sum(dtype=np.float32) / mask_sum
  tp_mean = (tp_flat * mf).sum(dtype=np.float32) / mask_sum
  rp_d = (rp_flat - rp_mean) * mf
  tp_d = (tp_flat - tp_mean) * mf
  cov = (rp_d * tp_d).sum(dtype=np.float32) / mask_sum
  rp_var = (rp_d * rp_d).sum(dtype=np.float32) / mask_sum
  tp_var = (tp_d * tp_d).sum(dtype=np.float32) / mask_sum
  return {
      "sampler_trainer/logp_diff_mean": float((diff * mask_f).sum(dtype=np.float32) / mask_sum),
      "sampler_trainer/logp_diff_max": float(np.where(mask, diff, 0.0).max()),
      "sampler_trainer/prob_diff_mean": float((prob_diff * mask_f).sum(dtype=np.float32) / mask_sum),
      "sampler_trainer/prob_diff_max": float(np.where(mask, prob_diff, 0.0).max()),
      "sampler_trainer/probs_pearson_corr": float(cov / np.sqrt(np.maximum(rp_var * tp_var, np.float32(1e-12)))),
  }
