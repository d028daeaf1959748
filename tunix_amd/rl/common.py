"""Per-token log-probabilities, the GRPO clipped ratio, KL estimators and loss aggregation on
the quantized model (mirrors tunix/rl/common.py:187-203 selective_log_softmax, :326-482
compute_per_token_logps, :485-571 compute_chunked_logps, :135-184 compute_kl_divergence,
:763-854 aggregate_loss, the ratio of tunix/rl/algo_core.py:440-489 and the rollout-against-trainer
agreement figures of tunix/rl/grpo/grpo_learner.py:405-440).

compute_per_token_logps runs one full forward over prompt + completion (no cache reuse, the
reference does the same), then feeds the hidden states of the positions that predict the
completion tokens to the fused lm_head -> log-softmax -> gather kernel: full-vocabulary logits
are never written to HBM, so `chunk_size` only bounds the number of rows per launch.
"""
from __future__ import annotations

import dataclasses
from typing import Any

import numpy as np
import torch

from .. import ops
from ..model import QLoRAModel, Runner


def selective_log_softmax(logits: torch.Tensor, input_ids: torch.Tensor) -> torch.Tensor:
  """log_softmax(logits)[..., input_ids] for logits that already exist as a tensor
  (tunix/rl/common.py:187-203).  A convenience for callers that already hold a logits tensor,
  written with torch tensor methods: it is NOT one of this package's HIP kernels and nothing on
  the rollout or log-probability path calls it (those go through the fused head kernel,
  tnx_lmhead_logp, and never materialise logits)."""
  lg = logits.to(torch.float32)
  tgt = torch.gather(lg, -1, input_ids.long().unsqueeze(-1)).squeeze(-1)
  return tgt - torch.logsumexp(lg, dim=-1)


def process_ids(prompt_tokens: torch.Tensor, completion_tokens: torch.Tensor, pad_id: int):
  """tunix/rl/common.py:234-291 (unpacked): concatenated ids and positions counted over
  non-pad tokens.  The attention kernels derive the causal + padding mask from the ids
  themselves (key != pad_id and key <= query), which is make_causal_attn_mask of that mask."""
  ids = torch.cat([prompt_tokens, completion_tokens], dim=1).to(torch.int32).contiguous()
  mask = ids != pad_id
  run = torch.cumsum(mask.to(torch.int32), dim=-1)
  positions = (run - (run >= 1).to(torch.int32)).to(torch.int32).contiguous()
  return ids, positions


def compute_per_token_logps(model: QLoRAModel, prompt_tokens, completion_tokens, pad_id: int,
                            eos_id: int | None = None, *, temperature: float = 1.0,
                            chunk_size: int = 0, return_entropy: bool = False,
                            segment_ids=None, segment_positions=None,
                            max_rows: int = 16384, logits_fp32: bool = False) -> torch.Tensor:
  """fp32 [B, completion_len]: log p(completion token | everything before it).

  Packed batches (tunix/rl/common.py:260-271, :408-418, :440-443, :468-472): with `segment_ids`
  [B, L] a row of completion_tokens holds several prompt + completion sequences one after the
  other (prompt_tokens is then [B, 0]), `segment_positions` [B, L] gives every token its position
  inside its own sequence (required, as in the reference), a token attends the earlier tokens of
  its own segment only (the causal mask combined with equal segment ids, what the reference's
  flash-attention path computes from SegmentIds: tunix/models/qwen3/model.py:622-655), no padding
  mask is applied, every position but the first is scored and the result is [B, L] with 0.0 in
  column 0, so that logp[i] belongs to token[i].

  prompt_tokens [B, P] (left padded) and completion_tokens [B, T] (right padded) are integer
  arrays or tensors.  `temperature` divides the logits as in the reference (:431-436: ignored
  when 0 or 1).  `max_rows` bounds the token rows of one forward pass.  With return_entropy the
  result is (logps, entropy), entropy = -sum p log p of the same (temperature-scaled) logits
  (compute_entropy_from_logits, :1136-1148), also from the fused head kernel.  logits_fp32: the
  head's fp32-accumulate reference mode (the logits keep their fp32 accumulators instead of being
  rounded to bf16 as the reference's bf16 einsum output is).
  """
  dev = model.device
  pt = torch.as_tensor(np.asarray(prompt_tokens) if not isinstance(prompt_tokens, torch.Tensor)
                       else prompt_tokens).to(dev)
  ct = torch.as_tensor(np.asarray(completion_tokens) if not isinstance(completion_tokens, torch.Tensor)
                       else completion_tokens).to(dev)
  if pt.ndim != 2 or ct.ndim != 2 or pt.shape[0] != ct.shape[0]:
    raise ValueError(f"prompt_tokens {tuple(pt.shape)} and completion_tokens {tuple(ct.shape)} "
                     "must be [B, P] and [B, T]")
  B, T = ct.shape
  seg = None
  if segment_ids is not None:
    if segment_positions is None:
      raise ValueError("segment_positions must be explicitly provided for packed sequences. ")
    ids = torch.cat([pt, ct], dim=1).to(torch.int32).contiguous()
    as_i32 = lambda a: torch.as_tensor(np.asarray(a) if not isinstance(a, torch.Tensor) else a).to(dev, torch.int32).contiguous()
    seg, positions = as_i32(segment_ids), as_i32(segment_positions)
    if tuple(seg.shape) != tuple(ids.shape) or tuple(positions.shape) != tuple(ids.shape):
      raise ValueError(f"segment_ids {tuple(seg.shape)} and segment_positions {tuple(positions.shape)} must "
                       f"have the shape of the token buffer {tuple(ids.shape)}")
    T = ids.shape[1] - 1          # every position but the first is scored (:440-443)
    pad_front = True
  else:
    ids, positions = process_ids(pt, ct, pad_id)
    pad_front = False
  Ltot = ids.shape[1]
  if T <= 0:
    empty = torch.zeros(B, Ltot if pad_front else 0, dtype=torch.float32, device=dev)
    return (empty, torch.zeros_like(empty)) if return_entropy else empty
  if Ltot < T + 1:
    raise ValueError("the first completion token needs at least one token before it")
  cfg = model.cfg
  temp = 1.0 if temperature in (0.0, 1.0) else float(temperature)
  rows_b = max(1, min(B, max_rows // Ltot))
  runner = Runner(model, rows_b, Ltot, Ltot, pad_id, kv_chunk=0)
  # the cache is scratch here: every layer writes its keys / values and reads them back
  # within the same pass, so one pair of buffers serves all layers
  kc = torch.empty(rows_b, cfg.num_kv_heads, Ltot, cfg.head_dim, dtype=torch.bfloat16, device=dev)
  vc = torch.empty_like(kc)
  head_rows = rows_b * T if chunk_size <= 0 else rows_b * min(T, chunk_size)
  head_rows = min(head_rows, 8192)
  part = torch.empty(head_rows * runner.nvb * 4, dtype=torch.float32, device=dev)
  runner.part = part
  xsel = torch.empty(rows_b * T, cfg.embed_dim, dtype=torch.bfloat16, device=dev)
  out = torch.empty(B, T, dtype=torch.float32, device=dev)
  ent = torch.empty(B, T, dtype=torch.float32, device=dev) if return_entropy else None
  part_ent = torch.empty(head_rows * runner.nvb, dtype=torch.float32, device=dev) if return_entropy else None
  for b0 in range(0, B, rows_b):
    nb = min(rows_b, B - b0)
    xn = runner.forward_hidden(ids[b0:b0 + nb], positions[b0:b0 + nb], runner.zero,
                               [kc[:nb]] * cfg.num_layers, [vc[:nb]] * cfg.num_layers, B=nb, T=Ltot,
                               segment_ids=None if seg is None else seg[b0:b0 + nb])
    # logits[:, -T-1:-1] predict the completion tokens (:462-467)
    xs = xsel[: nb * T]
    xs.view(nb, T, -1).copy_(xn[: nb * Ltot].view(nb, Ltot, -1)[:, Ltot - T - 1: Ltot - 1])
    tg = ids[b0:b0 + nb, Ltot - T:].contiguous().view(-1)
    lp = out[b0:b0 + nb].view(-1)
    for r0 in range(0, nb * T, head_rows):
      nr = min(head_rows, nb * T - r0)
      kw = {}
      if return_entropy:  # entropy of the temperature-scaled distribution (:479-481)
        kw = dict(entropy=ent[b0:b0 + nb].view(-1)[r0:r0 + nr], part_entropy=part_ent)
      runner.run_head(xs[r0:r0 + nr], nr, temperature=temp, targets=tg[r0:r0 + nr],
                      target_logp=lp[r0:r0 + nr], logits_fp32=logits_fp32, **kw)
  if pad_front:   # one 0.0 in front: logp[i] belongs to token[i] (:468-472)
    front = lambda x: torch.cat([torch.zeros(B, 1, dtype=torch.float32, device=dev), x], dim=1)
    return (front(out), front(ent)) if return_entropy else front(out)
  return (out, ent) if return_entropy else out


def grpo_clipped_ratio(logp: torch.Tensor, old_logp: torch.Tensor | None, advantages: torch.Tensor,
                       epsilon: float = 0.2, epsilon_high: float | None = None):
  """(ratio, per-token loss, clipped flag) of tunix/rl/algo_core.py:440-489:
  ratio = exp(logp - old_logp) (old_logp None: the on-policy case, ratio 1),
  loss = max(-A * ratio, -A * clip(ratio, 1 - eps, 1 + eps_high)); A is per sequence."""
  B, T = logp.shape
  eps_hi = epsilon if epsilon_high is None else epsilon_high
  lp = logp.to(torch.float32).contiguous()
  old = None if old_logp is None else old_logp.to(torch.float32).contiguous()
  adv = advantages.to(torch.float32).contiguous().view(-1)
  if adv.numel() != B:
    raise ValueError("advantages must hold one value per sequence")
  ratio = torch.empty_like(lp)
  loss = torch.empty_like(lp)
  clipped = torch.empty(B, T, dtype=torch.int32, device=lp.device)
  ops.grpo_ratio(lp, old, adv, T, epsilon, eps_hi, ratio=ratio, loss=loss, clipped=clipped)
  return ratio, loss, clipped.bool()


def compute_kl_divergence(per_token_logps: torch.Tensor, ref_per_token_logps: torch.Tensor,
                          method: str = "low_var_kl", clamp_value: float | None = None) -> torch.Tensor:
  """Per-token KL between the trained and the reference policy (tunix/rl/common.py:135-184):
  "kl" logp - ref, "mse_kl" 0.5 (logp - ref)^2, "low_var_kl" exp(d) - d - 1 with d = ref - logp;
  clamp_value clips the result symmetrically."""
  if method not in ops.KL_METHODS:
    raise ValueError("`method` must be one of 'kl', 'mse_kl', 'low_var_kl'. Received:"
                     f" {method}")
  if clamp_value is not None and clamp_value < 0:
    raise ValueError("clamp_value must not be negative")  # clip(x, c, -c) with c < 0 has no meaning
  lp = per_token_logps.to(torch.float32).contiguous()
  ref = ref_per_token_logps.to(torch.float32).contiguous()
  if lp.shape != ref.shape:
    raise ValueError(f"shapes differ: {tuple(lp.shape)} vs {tuple(ref.shape)}")
  out = torch.empty_like(lp)
  if lp.numel():
    ops.kl_divergence(lp, ref, ops.KL_METHODS[method], -1.0 if clamp_value is None else clamp_value, out)
  return out


@dataclasses.dataclass
class WeightedMetric:
  """A sum and the weight to divide it by (tunix/sft/utils.py:185-219); both stay on the device."""
  unreduced_sum: torch.Tensor
  denominator: torch.Tensor
  eps: float | None = None
  min_denom: float | None = None

  def compute_scale(self) -> torch.Tensor:
    denom = self.denominator
    if self.eps is not None:
      denom = denom + self.eps
    if self.min_denom is not None:
      denom = torch.clamp(denom, min=self.min_denom)
    safe = torch.where(denom == 0, torch.ones_like(denom), denom)
    return torch.where(denom == 0, torch.zeros_like(denom), 1.0 / safe)

  def compute(self) -> torch.Tensor:
    return self.unreduced_sum * self.compute_scale()


def _check_get_norm(arguments: dict[str, Any], default: float) -> float:
  """The `norm` keyword or its default (tunix/rl/common.py:1151-1177)."""
  if "norm" in arguments:
    try:
      norm = float(arguments["norm"])
    except (ValueError, TypeError):
      raise ValueError(f"Invalid 'norm' value: {arguments['norm']}. Must be a positive number.")
    if norm <= 0:
      raise ValueError(f"Invalid 'norm' value: {norm}. Must be a positive number.")
    return norm
  return float(default)


def aggregate_loss(per_token_loss: torch.Tensor, completion_mask: torch.Tensor, loss_agg_mode: str,
                   segment_ids=None, num_segments=None, **kwargs: Any) -> WeightedMetric:
  """Aggregates a [B, T] per-token loss under its completion mask (tunix/rl/common.py:763-940).
  With `segment_ids` ([B, T], 0 = padding) the batch is packed: the per-sequence modes reduce per
  segment instead of per row (the segment branch, :857-940); `num_segments` bounds the ids."""
  if loss_agg_mode not in ops.AGG_MODES:
    raise ValueError(
        f"Unsupported loss aggregation mode: {loss_agg_mode}. Supported modes:"
        " 'token-mean', 'sequence-mean-token-mean',"
        " 'sequence-mean-token-scale', 'seq-mean-token-sum',"
        " 'sequence-mean-token-sum-norm'.")
  if per_token_loss.dim() != 2 or per_token_loss.shape != completion_mask.shape:
    raise ValueError("per_token_loss and completion_mask must both be [batch_size, sequence_len]")
  B, T = per_token_loss.shape
  min_denom = 1e-6 if loss_agg_mode in ("seq-mean-token-sum", "sequence-mean-token-sum-norm") else 1.0
  loss = per_token_loss.to(torch.float32).contiguous()
  mask = completion_mask.to(torch.float32).contiguous()
  out = torch.zeros(2, dtype=torch.float32, device=loss.device)
  if segment_ids is not None:
    if num_segments is None:
      raise ValueError("num_segments must be provided when segment_ids is not None.")
    if tuple(segment_ids.shape) != (B, T):
      raise ValueError("segment_ids must be [batch_size, sequence_len]")
    norm = -1.0   # sum-norm: the number of active segments unless the caller names a norm
    if loss_agg_mode == "sequence-mean-token-scale":
      if "norm" not in kwargs:
        raise ValueError(
            "sequence-mean-token-scale under sequence packing requires an"
            " explicit 'norm' (e.g. max_response_length); the default row-width"
            " norm is the pack budget, which dilutes every sequence.")
      norm = _check_get_norm(kwargs, T)
    elif loss_agg_mode == "sequence-mean-token-sum-norm" and "norm" in kwargs:
      norm = _check_get_norm(kwargs, 1.0)
    if B and T:
      seg = segment_ids.to(device=loss.device, dtype=torch.int32).contiguous()
      ops.aggregate_loss_segmented(loss, mask, seg, int(num_segments), ops.AGG_MODES[loss_agg_mode], norm, out)
    elif loss_agg_mode == "sequence-mean-token-sum-norm" and norm > 0:
      out[1] = norm
    return WeightedMetric(out[0], out[1], min_denom=min_denom)
  norm = 1.0
  if loss_agg_mode == "sequence-mean-token-scale":
    norm = _check_get_norm(kwargs, T)
  elif loss_agg_mode == "sequence-mean-token-sum-norm":
    norm = _check_get_norm(kwargs, B)
  if B and T:
    row_ws = torch.empty(B, 2, dtype=torch.float32, device=loss.device)
    ops.aggregate_loss(loss, mask, ops.AGG_MODES[loss_agg_mode], norm, row_ws, out)
  elif loss_agg_mode == "sequence-mean-token-sum-norm":
    out[1] = norm
  return WeightedMetric(out[0], out[1], min_denom=min_denom)


DRIFT_METRICS = ("sampler_trainer/logp_diff_mean", "sampler_trainer/logp_diff_max",
                 "sampler_trainer/prob_diff_mean", "sampler_trainer/prob_diff_max",
                 "sampler_trainer/probs_pearson_corr")


def sampler_trainer_agreement(rollout_per_token_logps: torch.Tensor, trainer_per_token_logps: torch.Tensor,
                              completion_mask: torch.Tensor) -> dict[str, float]:
  """How far the log-probabilities the rollout recorded are from the ones recomputed for the same
  tokens, over the completion positions (tunix/rl/grpo/grpo_learner.py:405-440, same metric
  names): mean / max |dlogp|, mean / max |dp| and the Pearson correlation of the probabilities.
  With the rollout's own log-probabilities and compute_per_token_logps of this package it is the
  running check that the decode path and the many-row path agree."""
  a = rollout_per_token_logps.to(torch.float32).contiguous()
  b = trainer_per_token_logps.to(torch.float32).contiguous()
  if a.dim() != 2 or a.shape != b.shape or a.shape != completion_mask.shape:
    raise ValueError("log-probabilities and mask must share one [batch_size, sequence_len] shape")
  out = torch.zeros(5, dtype=torch.float32, device=a.device)
  if a.numel():
    ops.logp_drift(a, b, completion_mask.to(torch.bool).to(torch.float32).contiguous(), out)
  return dict(zip(DRIFT_METRICS, out.tolist()))
