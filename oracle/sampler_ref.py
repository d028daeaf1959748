"""The sampler's prefill + decode loop (oracle; tests only).

Follows tunix/generate/sampler.py:105-161 (sample_top_p, sample_best), :362-463
(init_sample_state), :474-552 (_sample), :554-673 (_prefill_fn), :675-736 (_decode_fn,
_sample_step): dense boolean masks over the whole cache, full [B,V] fp32 logits per step.
"""
from __future__ import annotations

import numpy as np
import torch

from . import threefry as TF
from . import utils_ref as U


def sample_best(logits_last: torch.Tensor):
  """sampler.py:151-161: first maximal index; logp from the fp32 log-softmax."""
  lg = logits_last.to(torch.float32)
  tok = torch.from_numpy(np.argmax(lg.numpy(), axis=-1))
  lp = torch.log_softmax(lg, dim=-1).gather(-1, tok[:, None]).squeeze(-1)
  return tok, lp


def sample_top_p(logits_last: torch.Tensor, key, temperature, top_p, top_k, partitionable=False):
  """sampler.py:105-148 with jax.random.categorical restated by oracle.threefry."""
  lg = (logits_last.to(torch.float32) / np.float32(temperature)).numpy()
  V = lg.shape[-1]
  no_topk = top_k is None or top_k <= 0
  if top_p >= 1.0 and no_topk:
    tok = TF.categorical(key, lg, partitionable)
  else:
    k = V if no_topk else int(top_k)
    order = np.argsort(-lg, axis=-1, kind="stable")[:, :k]        # descending, lower index first
    srt = np.take_along_axis(lg, order, axis=-1)
    ex = np.exp(srt - srt[:, :1])
    probs = (ex / ex.sum(-1, keepdims=True)).astype(np.float32)
    cum = np.cumsum(probs, axis=-1, dtype=np.float32)
    srt = np.where(cum - probs > np.float32(top_p), -np.inf, srt).astype(np.float32)
    idx = TF.categorical(key, srt, partitionable)
    tok = np.take_along_axis(order, idx[:, None], axis=-1)[:, 0]
  lp = torch.log_softmax(torch.from_numpy(lg), dim=-1).numpy()
  return torch.from_numpy(tok.astype(np.int64)), torch.from_numpy(
      np.take_along_axis(lp, tok[:, None].astype(np.int64), axis=-1)[:, 0])


def run(ref_model, all_input_ids: np.ndarray, max_generation_steps: int, pad_id: int,
        cache_size: int, eos_ids, temperature: float = 0.0, top_p=None, top_k=None, seed: int = 0,
        forbidden=None, keep_logits: bool = False, partitionable: bool = False):
  """Returns dict(token_buffer [B,L], logprobs [B,L], logits list per generated column)."""
  B, P = all_input_ids.shape
  L = P + max_generation_steps
  assert L <= cache_size
  tb = np.full((B, L), pad_id, dtype=np.int64)
  tb[:, :P] = all_input_ids
  in_mask = np.ones((B, L), dtype=bool)
  in_mask[:, :P] = all_input_ids != pad_id
  positions = U.build_positions_from_mask(in_mask)
  done = np.zeros(B, dtype=bool)
  lpbuf = np.zeros((B, L), dtype=np.float32)
  cache = ref_model.init_cache(B, cache_size)
  key = TF.prng_key(seed)
  logits_log = []

  def sample(logits_last, step):
    lg = logits_last.clone()
    if forbidden:
      lg[:, list(forbidden)] = -np.inf
    if top_p is None:
      tok, lp = sample_best(lg)
    else:
      tok, lp = sample_top_p(lg, TF.fold_in(key, step), temperature, top_p, top_k, partitionable)
    tb[:, step + 1] = tok.numpy()
    lpbuf[:, step + 1] = lp.numpy()
    if keep_logits:
      logits_log.append(lg.numpy().copy())
    return np.isin(tb[:, step + 1], np.asarray(eos_ids))

  # prefill
  pmask = U.make_causal_attn_mask(tb[:, :P] != pad_id, cache_size)
  logits = ref_model(torch.from_numpy(tb[:, :P]), torch.from_numpy(positions[:, :P]), cache,
                     torch.from_numpy(pmask), 0)
  done |= sample(logits[:, -1], P - 1)
  step = P
  while step < L - 1 and (~done).any():
    amask = U.compute_attention_masks(step, cache_size, tb == pad_id)
    logits = ref_model(torch.from_numpy(tb[:, step:step + 1]),
                       torch.from_numpy(positions[:, step:step + 1]), cache,
                       torch.from_numpy(amask), step)
    done |= sample(logits[:, -1], step)
    step += 1
  return {"token_buffer": tb, "logprobs": lpbuf, "logits": logits_log, "steps": step - P}
