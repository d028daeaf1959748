"""Sampler for QLoRA decoders on MI355X: the host driver of tunix/generate/sampler.py:198-1011
with the jitted prefill / while_loop decode replaced by libtunix_hip.so kernels.

Same call contract as the reference: `Sampler(transformer, tokenizer, cache_config)` and
`sampler(input_strings, max_generation_steps, ...) -> SamplerOutput`.  `transformer` is a
`tunix_amd.model.QLoRAModel`.  One decode step is captured into a HIP graph and replayed: the
step counter, positions and token buffer live in device memory, so no host round trip happens
inside the loop.
"""
from __future__ import annotations

import dataclasses
from typing import Iterable, Optional, Sequence

import numpy as np
import torch

from .. import ops
from ..model import QLoRAModel, Runner
from . import utils
from .base_sampler import SamplerOutput


@dataclasses.dataclass(frozen=True)
class CacheConfig:
  """Configuration for the KV cache (tunix/common/configs.py:60-67)."""

  cache_size: int
  num_layers: int
  num_kv_heads: int
  head_dim: int


def _threefry_seed(seed: int) -> tuple[int, int]:
  """jax.random.PRNGKey(seed) for the threefry2x32 implementation: (high word, low word).  With
  jax's default 32-bit integers the seed is an int32 (wider Python ints wrap), its logical shift
  right by 32 gives 0, and the low word is the seed's two's-complement bit pattern: PRNGKey(-1)
  is (0, 0xFFFFFFFF)."""
  return 0, int(seed) & 0xFFFFFFFF


def sampling_plan(top_k: int | None, top_p: float, vocab_size: int) -> tuple[int, str]:
  """(k passed to tnx_sample_topk, which path it takes there) for a top_p-mode call
  (sampler.py:105-148).  top_k None or <= 0 means "no top-k" (:118): then top_p >= 1 is the
  categorical draw inside the head ("head_draw", noise per vocabulary id) and top_p < 1 sorts whole
  rows ("fullsort", workspace of tnx_sample_fullsort_ws_bytes).  top_k == vocab_size is a real
  top-k in the reference -- jax.lax.top_k(k = V) sorts the row and the draw runs over sorted
  positions, whatever top_p -- so it takes the full sort too; top_k > vocab_size raises as
  jax.lax.top_k does.  Any other top_k uses the segmented selection ("topk", workspace of
  tnx_sample_topk_ws_bytes) or, for the shapes tnx_sample_topk_head_ok accepts (top_k <= 64), the
  one-launch draw from the head's block statistics, which selects the same candidates.  One
  predicate decides both the path and the workspace size."""
  if top_k is None or top_k <= 0:
    return 0, ("head_draw" if top_p >= 1.0 else "fullsort")
  if top_k > vocab_size:
    raise ValueError(f"top_k={top_k} must be at most the vocabulary size {vocab_size}")
  if top_k == vocab_size:
    return int(top_k), "fullsort"
  return int(top_k), "topk"


class _SamplingState:
  """Device-resident counterpart of _SamplingState (tunix/generate/sampler.py:49-102)."""

  def __init__(self, model: QLoRAModel, all_input_ids: np.ndarray, total_sampling_steps: int,
               cache_size: int, pad_id: int, include_logits: bool, include_logprobs: bool):
    cfg, dev = model.cfg, model.device
    B, P = all_input_ids.shape
    L = total_sampling_steps
    tb = np.full((B, L), pad_id, dtype=np.int32)
    tb[:, :P] = all_input_ids
    mask = np.ones((B, L), dtype=bool)
    mask[:, :P] = all_input_ids != pad_id
    self.num_input_tokens = P
    self.total_sampling_steps = L
    self.token_buffer = torch.from_numpy(tb).to(dev)
    self.positions = torch.from_numpy(utils.build_positions_from_mask(mask)).to(dev)
    self.done = torch.zeros(B, dtype=torch.int32, device=dev)
    # decoding_step: column of the last committed token
    self.step = torch.full((1,), P - 1, dtype=torch.int32, device=dev)
    shape = (B, cfg.num_kv_heads, cache_size, cfg.head_dim)
    self.kcache = [torch.zeros(shape, dtype=torch.bfloat16, device=dev) for _ in range(cfg.num_layers)]
    self.vcache = [torch.zeros(shape, dtype=torch.bfloat16, device=dev) for _ in range(cfg.num_layers)]
    self.logits_buffer = (torch.zeros(B, L, cfg.vocab_size, dtype=torch.float32, device=dev)
                          if include_logits else None)
    self.logprobs_buffer = (torch.zeros(B, L, dtype=torch.float32, device=dev)
                            if include_logprobs else None)


class Sampler:
  """Sampler for transformer model."""

  def __init__(self, transformer: QLoRAModel, tokenizer, cache_config: CacheConfig,
               use_graph: bool = True, prefill_rows: int = 16384):
    self._transformer = transformer
    self.tokenizer = tokenizer
    self.cache_config = cache_config
    self.use_graph = use_graph
    self.prefill_rows = prefill_rows
    self.rng_variant = 0  # threefry random_bits layout that reproduces the reference's golden arrays
    self.last_stats: dict = {}

  @property
  def transformer(self) -> QLoRAModel:
    return self._transformer

  @property
  def transformer_state(self):
    return self._transformer

  def update_lora(self, lora_state: dict) -> None:
    """LoRA-only state replacement (sampler.py:333-352)."""
    self._transformer.update_lora(lora_state)

  def update_params(self, state: dict) -> None:
    """Full or LoRA-only state replacement (sampler.py:265-352), by flat parameter name."""
    self._transformer.update_params(state)

  @property
  def dtype(self):
    return torch.bfloat16

  def tokenize(self, input_string) -> np.ndarray:
    """BOS + ids of one prompt (sampler.py:465-472); id sequences pass through unchanged."""
    if not isinstance(input_string, str):
      return np.asarray(input_string, dtype=np.int32)
    input_ids = list(self.tokenizer.encode(input_string))
    bos = self.tokenizer.bos_id()
    bos_tok = [bos] if bos else []
    ids = bos_tok + input_ids
    if hasattr(self.tokenizer, "dedup_bos_ids"):
      ids = self.tokenizer.dedup_bos_ids(ids)
    return np.asarray(ids, dtype=np.int32)

  # ---- one sampling step on the device -------------------------------------------------------
  def _sample(self, runner: Runner, x, st: _SamplingState, mode: dict):
    """lm_head + sampling + bookkeeping for the B rows in x (sampler.py:474-552)."""
    want_lp = st.logprobs_buffer is not None
    if mode["name"] == "greedy":
      runner.run_head(x, runner.B, best_id=runner.best_id, best_logp=runner.best_logp,
                      forbidden=mode["forbidden"], logits_out=runner.logits)
      ids, lp = runner.best_id, (runner.best_logp if want_lp else None)
    elif mode["top_k"] == 0 and mode["top_p"] >= 1.0:
      # the plain categorical draw (the reference's default rollout configuration) happens inside
      # the head kernel: no logits in HBM, no sampling launch
      runner.run_head(x, runner.B, temperature=mode["temperature"], forbidden=mode["forbidden"],
                      logits_out=runner.logits,
                      draw=dict(part=mode["part_draw"], key=mode["key"], variant=self.rng_variant,
                                step=st.step, ids=mode["ids"], logp=mode["logp"]))
      ids, lp = mode["ids"], (mode["logp"] if want_lp else None)
    elif mode.get("head_lse") is not None:
      # top-k of at most 64: the head runs at the sampling temperature and leaves per-block
      # maxima and the row's log-sum-exp; the draw then reads only the k best blocks' logits
      runner.run_head(x, runner.B, temperature=mode["temperature"], forbidden=mode["forbidden"],
                      lse=mode["head_lse"], logits_out=runner.logits)
      ops.sample_topk_head(runner.logits, runner.part, mode["head_lse"], mode["top_k"], mode["top_p"],
                           mode["temperature"], mode["key"], self.rng_variant, st.step, mode["ids"],
                           mode["logp"], forbidden=mode["forbidden"])
      ids, lp = mode["ids"], (mode["logp"] if want_lp else None)
    else:
      runner.run_head(x, runner.B, best_id=runner.best_id, logits_out=runner.logits)
      ops.sample_topk(runner.logits, mode["top_k"], mode["top_p"], mode["temperature"], mode["key"],
                      self.rng_variant, st.step, mode["ws"], mode["ids"], mode["logp"],
                      forbidden=mode["forbidden"])
      ids, lp = mode["ids"], (mode["logp"] if want_lp else None)
    ops.sample_commit(ids, lp, st.token_buffer, st.logprobs_buffer, st.done, mode["eos"], st.step)

  def _prefill(self, st: _SamplingState, runner_dec: Runner, mode: dict, return_logits: bool):
    """sampler.py:554-673: forward over the padded prompts, fill the cache, sample one token."""
    model = self._transformer
    B, P = st.token_buffer.shape[0], st.num_input_tokens
    S = self.cache_config.cache_size
    rows = max(1, min(B, self.prefill_rows // max(P, 1)))
    pad = self.tokenizer.pad_id()
    runner = Runner(model, rows, P, S, pad, kv_chunk=0)
    D = model.cfg.embed_dim
    for b0 in range(0, B, rows):
      nb = min(rows, B - b0)
      kc = [k[b0:b0 + nb] for k in st.kcache]
      vc = [v[b0:b0 + nb] for v in st.vcache]
      xn = runner.forward_hidden(st.token_buffer[b0:b0 + nb], st.positions[b0:b0 + nb],
                                 runner.zero, kc, vc, B=nb, T=P)
      runner_dec.xlast[b0:b0 + nb].copy_(xn[: nb * P].view(nb, P, D)[:, P - 1])
      if return_logits:
        # logits of every prompt position go to logits_buffer[:, 1:P+1] (sampler.py:617-625)
        part = torch.empty(nb * P * runner.nvb * 4, dtype=torch.float32, device=model.device)
        lg = torch.empty(nb * P, model.cfg.vocab_size, dtype=torch.float32, device=model.device)
        runner.part = part
        runner.run_head(xn, nb * P, logits_out=lg)
        lg = lg.view(nb, P, -1)
        L = st.total_sampling_steps
        n_fit = min(P, L - 1)
        st.logits_buffer[b0:b0 + nb, 1:1 + n_fit].copy_(lg[:, :n_fit])
    del runner
    self._sample(runner_dec, runner_dec.xlast, st, mode)

  def _decode_step(self, runner: Runner, st: _SamplingState, mode: dict):
    """sampler.py:692-736: one token per row from the cached state."""
    xn = runner.forward_hidden(st.token_buffer, st.positions, st.step, st.kcache, st.vcache)
    self._sample(runner, xn, st, mode)

  # ---- public entry --------------------------------------------------------------------------
  def __call__(
      self,
      input_strings,
      max_generation_steps: int,
      max_prompt_length: int | None = None,
      echo: bool = False,
      return_logits: bool = False,
      return_logprobs: bool = False,
      eos_tokens: Sequence[int] | None = None,
      forbidden_tokens: Iterable[int] | None = None,
      temperature: float = 0.0,
      top_p: Optional[float] = None,
      top_k: Optional[int] = None,
      beam_size: Optional[int] = None,
      seed: int | None = None,
      pad_output: bool = False,
  ) -> SamplerOutput:
    """Samples a completion of the input prompts (sampler.py:738-1011).

    If top_p is provided the sampling mode is top_p (top_k alone does not enable sampling);
    otherwise greedy.  Beam search is not part of this build.
    """
    model, dev = self._transformer, self._transformer.device
    cfg = model.cfg
    eos_ids = list(eos_tokens) if eos_tokens else [self.tokenizer.eos_id()]
    if isinstance(input_strings, str):
      input_strings = [input_strings]
    forbidden = tuple(forbidden_tokens) if forbidden_tokens else None
    tokens = [self.tokenize(x) for x in input_strings]
    max_tokens_length = max(len(x) for x in tokens)
    if max_prompt_length is None or max_prompt_length < max_tokens_length:
      max_prompt_length = utils.next_power_of_2(max_tokens_length)
    pad = self.tokenizer.pad_id()
    all_input_ids = np.array([
        utils.pad_to_length(x, target_length=max_prompt_length, pad_value=pad, left=True)
        for x in tokens])
    total_sampling_steps = max_prompt_length + max_generation_steps
    if total_sampling_steps > self.cache_config.cache_size:
      raise ValueError(
          f"Total sampling steps {total_sampling_steps} must be less than the"
          f" cache size {self.cache_config.cache_size}.")
    if beam_size is not None:
      if top_p is not None:
        utils.check_sampling_mode_conflict(["beam_search"], "top_p")
      raise NotImplementedError("beam search is outside the rollout decode path of this build")
    key = _threefry_seed(0 if seed is None else seed)

    B = all_input_ids.shape[0]
    S = self.cache_config.cache_size
    st = _SamplingState(model, all_input_ids, total_sampling_steps, S, pad, return_logits,
                        return_logprobs)
    mode = {"name": "greedy", "forbidden": None,
            "eos": torch.tensor(eos_ids, dtype=torch.int32, device=dev)}
    if forbidden:
      mode["forbidden"] = torch.tensor(forbidden, dtype=torch.int32, device=dev)
    if top_p is not None:
      k, path = sampling_plan(top_k, float(top_p), cfg.vocab_size)
      ws_bytes = (ops.sample_fullsort_ws_bytes(B, cfg.vocab_size) if path == "fullsort"
                  else ops.sample_topk_ws_bytes(B, cfg.vocab_size, k))
      if path == "fullsort" and ws_bytes == 0:
        raise ValueError("top_p < 1 without top_k sorts whole rows: batch x vocabulary must stay below 2^31")
      mode.update(name="top_p", temperature=float(temperature), top_p=float(top_p), top_k=k,
                  key=key,
                  ws=torch.empty(max(ws_bytes // 4, 1), dtype=torch.float32, device=dev),
                  ids=torch.empty(B, dtype=torch.int32, device=dev),
                  logp=torch.empty(B, dtype=torch.float32, device=dev))
      if path == "topk" and ops.sample_topk_head_ok(cfg.vocab_size, k):
        mode["head_lse"] = torch.empty(B, dtype=torch.float32, device=dev)
      if k == 0 and top_p >= 1.0:
        mode["part_draw"] = torch.empty(B * ops.lmhead_nblocks(cfg.vocab_size) * 3, dtype=torch.float32,
                                        device=dev)
    in_head_draw = mode["name"] == "top_p" and mode["top_k"] == 0 and mode["top_p"] >= 1.0
    need_logits = return_logits or (mode["name"] == "top_p" and not in_head_draw)
    runner = Runner(model, B, 1, S, pad, want_logits=need_logits)

    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    ev[0].record()
    self._prefill(st, runner, mode, return_logits)
    ev[1].record()

    n_decode = total_sampling_steps - 1 - max_prompt_length
    steps_run = 0
    if n_decode > 0:
      if return_logits or not self.use_graph:
        for i in range(n_decode):
          self._decode_step(runner, st, mode)
          if return_logits:
            st.logits_buffer[:, max_prompt_length + i + 1].copy_(runner.logits)
          steps_run += 1
          if (i & 15) == 15 and bool(st.done.all()):
            break
      else:
        # the first step runs eagerly (lazy module load, attribute set-up), then one captured
        # step is replayed; `done` is polled every 32 steps like the while_loop condition
        self._decode_step(runner, st, mode)
        steps_run = 1
        if n_decode > 1:
          graph = torch.cuda.CUDAGraph()
          side = torch.cuda.Stream()
          side.wait_stream(torch.cuda.current_stream())
          with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
              self._decode_step(runner, st, mode)
          torch.cuda.current_stream().wait_stream(side)
          # capture does not execute: replay n_decode - 1 times
          while steps_run < n_decode:
            burst = min(32, n_decode - steps_run)
            for _ in range(burst):
              graph.replay()
            steps_run += burst
            if bool(st.done.all()):
              break
    ev[2].record()
    torch.cuda.synchronize(dev)
    self.last_stats = {
        "prefill_ms": ev[0].elapsed_time(ev[1]), "decode_ms": ev[1].elapsed_time(ev[2]),
        "decode_steps": steps_run, "batch": B, "prompt_len": max_prompt_length}

    token_buffers = st.token_buffer.cpu().numpy()
    logprobs_np = st.logprobs_buffer.cpu().numpy() if return_logprobs else None
    logits_np = st.logits_buffer.cpu().numpy() if return_logits else None
    eos_arr = np.asarray(eos_ids)
    out_tokens, out_logits, out_logprobs = [], [], []
    max_len = total_sampling_steps if echo else max_generation_steps
    for i in range(B):
      tb = token_buffers[i]
      start_idx = utils.np_find_first_non_pad_idx(tb, pad) if echo else max_prompt_length
      end_idx = utils.np_find_first_eos_idx(tb[max_prompt_length:], eos_arr) + max_prompt_length
      toks = tb[start_idx:end_idx]
      if pad_output:
        length = end_idx - start_idx
        toks = utils.pad_to_length(toks, max_len, pad)[:max_len]
        if return_logits:
          lg = np.zeros((max_len, cfg.vocab_size), dtype=np.float32)
          lg[:length] = logits_np[i][start_idx:end_idx]
          out_logits.append(lg)
        if return_logprobs:
          lp = np.zeros(max_len, dtype=np.float32)
          lp[:length] = logprobs_np[i][start_idx:end_idx]
          out_logprobs.append(lp.tolist())
      else:
        if return_logits:
          out_logits.append(logits_np[i][start_idx:end_idx])
        if return_logprobs:
          out_logprobs.append(logprobs_np[i][start_idx:end_idx].tolist())
      out_tokens.append(toks)
    if pad_output:
      lengths = [utils.np_find_first_eos_idx(token_buffers[i][max_prompt_length:], eos_arr)
                 + max_prompt_length
                 - (utils.np_find_first_non_pad_idx(token_buffers[i], pad) if echo
                    else max_prompt_length) for i in range(B)]
      decoded = [self.tokenizer.decode(t[:n].tolist()) for t, n in zip(out_tokens, lengths)]
    else:
      decoded = [self.tokenizer.decode(t.tolist()) for t in out_tokens]
    self._last_state = st
    return SamplerOutput(
        text=decoded,
        logits=out_logits if return_logits else [],
        tokens=out_tokens,
        padded_prompt_tokens=all_input_ids,
        logprobs=out_logprobs if return_logprobs else None,
    )
