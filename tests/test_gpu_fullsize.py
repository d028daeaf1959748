"""The benchmark workload (Llama-3.1-8B shape, NF4 g64, LoRA r64, batch 128) at its real sizes.

The CPU oracle cannot run 32 layers of this width in test time, so full size is covered two ways:
one layer at full width (every kernel at the shapes, k splits and fused epilogues of the real
step) against the oracle, and the whole 32-layer model through properties that do not need the
oracle: the log-probabilities the decode path reports for its own tokens equal the ones the
whole-sequence pass (`compute_per_token_logps`: other tile shapes, no KV cache, causal prefill
attention) assigns to the same tokens, and a replayed HIP graph equals eager execution bit for
bit.
"""
import numpy as np
import pytest
import torch

from oracle import model_ref as MR
from test_gpu_sampler import _check_greedy, _oracle_full_logits, _prompts

pytestmark = pytest.mark.gpu


def test_full_width_layer_matches_oracle(gpu):
  """1 layer of the 8B shape (D 4096, 32q/8kv heads of 128, MLP 14336), batch 128: greedy ids and
  log-probabilities against the teacher-forced oracle."""
  from tunix_amd import config, dummy_model
  from tunix_amd.generate import CacheConfig, Sampler
  from tunix_amd.generate.utils import IdTokenizer
  from tunix_amd.model import QLoRAModel
  cfg = config.llama31_8b(num_layers=1, vocab_size=4096)
  w = dummy_model.create_dummy_weights(cfg, seed=20256)
  model = QLoRAModel(cfg, w, gpu)
  B, P, T = 128, 12, 4
  tok = IdTokenizer(cfg.vocab_size, pad_id=0, eos_id=1)
  sampler = Sampler(model, tok, CacheConfig(64, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim))
  prompts = _prompts(B, P, cfg.vocab_size, 20256)
  out = sampler(prompts, max_generation_steps=T, max_prompt_length=P, return_logprobs=True, eos_tokens=[-1])
  st = sampler._last_state
  tb = st.token_buffer.cpu().numpy()[:, :P + T]
  assert all(len(t) == T for t in out.tokens)
  ref = MR.RefModel(cfg, {k: v.cpu() for k, v in w.items()})
  logits = _oracle_full_logits(ref, tb, 0)
  report, n = _check_greedy(tb, logits, P, st.logprobs_buffer.cpu().numpy(), label="llama-8B width, 1 layer, batch 128")
  print(f"full-width layer: {n - len(report)}/{n} ids equal the oracle arg-max; near-ties: {report}")
  assert len(report) <= n // 20


def test_full_size_decode_agrees_with_whole_sequence_pass(gpu):
  """32 layers, batch 128, prompt 512, 1024-slot cache: decode log-probabilities against
  compute_per_token_logps over the generated tokens, and graph replay against eager."""
  from tunix_amd import config, dummy_model
  from tunix_amd.generate import CacheConfig, Sampler
  from tunix_amd.generate.utils import IdTokenizer
  from tunix_amd.model import QLoRAModel
  from tunix_amd.rl.common import compute_per_token_logps
  cfg = config.llama31_8b()
  model = QLoRAModel(cfg, dummy_model.create_dummy_weights(cfg, seed=20257, device=gpu), gpu)
  B, P, T = 128, 512, 6
  tok = IdTokenizer(cfg.vocab_size, pad_id=0, eos_id=1)
  cc = CacheConfig(1024, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim)
  prompts = _prompts(B, P, cfg.vocab_size, 20257)
  outs = []
  for use_graph in (True, False):
    out = Sampler(model, tok, cc, use_graph=use_graph)(prompts, T, max_prompt_length=P, return_logprobs=True,
                                                        return_logits=not use_graph, eos_tokens=[-1])
    outs.append(out)
    torch.cuda.empty_cache()
  a, b = outs
  for x, y in zip(a.tokens, b.tokens):
    np.testing.assert_array_equal(x, y)
  np.testing.assert_array_equal(np.asarray(a.logprobs), np.asarray(b.logprobs))
  comp = np.stack(a.tokens).astype(np.int32)
  lps = compute_per_token_logps(model, a.padded_prompt_tokens, comp, 0, max_rows=16 * (P + T)).cpu().numpy()
  got = np.asarray(a.logprobs, dtype=np.float32)
  assert np.isfinite(got).all() and np.isfinite(lps).all()
  # Both are bf16-flow evaluations of the same network through different kernels and tilings.
  # The logits are bf16 values of magnitude 4-8 here, so a log-probability moves in steps of one
  # logit ulp (2^-5); through 32 layers the two accumulation orders drift apart by a few such
  # steps (measured: mean error 0.004 / 0.012 / 0.033 at 2 / 8 / 32 layers, i.e. rounding noise
  # growing with depth, median one ulp at 32 layers).  The bound is stated in those ulps.
  lg = np.asarray(b.logits)                                  # [B, T, V] raw logits of the eager run
  chosen = np.take_along_axis(lg, comp[:, :, None].astype(np.int64), -1)[..., 0]
  ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(chosen), 2.0 ** -20))) - 7)
  err = np.abs(lps - got)
  print(f"full size: decode vs whole-sequence logp, max {err.max():.3e} ({(err / ulp).max():.1f} ulp), "
        f"mean {err.mean():.3e}, median {np.median(err / ulp):.2f} ulp")
  assert np.median(err / ulp) <= 2.0
  assert (err <= 8.0 * ulp + 2e-2).all()


def test_gemma3_1b_full_size_decode_agrees_with_whole_sequence_pass(gpu):
  """The Gemma3-1B workload at its real sizes (26 layers, head_dim 256, one KV head, sliding
  window 512, 262144-entry tied head, int4 g128, LoRA r16, batch 64, prompt 256): greedy decode
  log-probabilities against compute_per_token_logps, graph replay against eager."""
  from tunix_amd import config, dummy_model
  from tunix_amd.generate import CacheConfig, Sampler
  from tunix_amd.generate.utils import IdTokenizer
  from tunix_amd.model import QLoRAModel
  from tunix_amd.rl.common import compute_per_token_logps
  cfg = config.gemma3_1b()
  model = QLoRAModel(cfg, dummy_model.create_dummy_weights(cfg, seed=20258, device=gpu), gpu)
  B, P, T = 64, 256, 6
  tok = IdTokenizer(cfg.vocab_size, pad_id=0, eos_id=1)
  cc = CacheConfig(512, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim)
  prompts = _prompts(B, P, cfg.vocab_size, 20258)
  a = Sampler(model, tok, cc, use_graph=True)(prompts, T, max_prompt_length=P, return_logprobs=True, eos_tokens=[-1])
  b = Sampler(model, tok, cc, use_graph=False)(prompts, T, max_prompt_length=P, return_logprobs=True,
                                               return_logits=True, eos_tokens=[-1])
  for x, y in zip(a.tokens, b.tokens):
    np.testing.assert_array_equal(x, y)
  np.testing.assert_array_equal(np.asarray(a.logprobs), np.asarray(b.logprobs))
  comp = np.stack(a.tokens).astype(np.int32)
  lps = compute_per_token_logps(model, a.padded_prompt_tokens, comp, 0, max_rows=16 * (P + T)).cpu().numpy()
  got = np.asarray(a.logprobs, dtype=np.float32)
  lg = np.asarray(b.logits)
  chosen = np.take_along_axis(lg, comp[:, :, None].astype(np.int64), -1)[..., 0]
  ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(chosen), 2.0 ** -20))) - 7)
  err = np.abs(lps - got)
  print(f"gemma3-1b full size: max {err.max():.3e} ({(err / ulp).max():.1f} ulp), mean {err.mean():.3e}, "
        f"median {np.median(err / ulp):.2f} ulp")
  assert np.isfinite(got).all() and np.isfinite(lps).all()
  assert np.median(err / ulp) <= 2.0
  assert (err <= 8.0 * ulp + 2e-2).all()


def test_gemma3_top_k_draw_over_the_full_vocabulary(gpu):
  """temperature 1.0, top-k 50 over the 262144-entry vocabulary of the Gemma3-1B workload (batch
  64): the segmented top-k selection (32 segments of 8192 per row) and the draw, ids exact
  against the oracle's sample_top_p on the logits the GPU itself produced, log-probabilities
  against the full-vocabulary log-softmax of those logits."""
  from oracle import sampler_ref as SR
  from oracle import threefry as TF
  from tunix_amd import config, dummy_model
  from tunix_amd.generate import CacheConfig, Sampler
  from tunix_amd.generate.utils import IdTokenizer
  from tunix_amd.model import QLoRAModel
  cfg = config.gemma3_1b(num_layers=2)
  assert cfg.vocab_size == 262144
  model = QLoRAModel(cfg, dummy_model.create_dummy_weights(cfg, seed=20259, device=gpu), gpu)
  B, P, T = 64, 16, 3
  tok = IdTokenizer(cfg.vocab_size, pad_id=0, eos_id=1)
  sampler = Sampler(model, tok, CacheConfig(32, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim))
  prompts = _prompts(B, P, cfg.vocab_size, 20259)
  out = sampler(prompts, T, max_prompt_length=P, temperature=1.0, top_p=1.0, top_k=50, seed=11, return_logprobs=True,
                return_logits=True, eos_tokens=[-1])
  tb = sampler._last_state.token_buffer.cpu().numpy()
  lps = sampler._last_state.logprobs_buffer.cpu().numpy()
  key = TF.prng_key(11)
  for c in range(P, P + T):
    gpu_lg = torch.from_numpy(np.stack([out.logits[b][c - P] for b in range(B)]))
    t_ref, lp_ref = SR.sample_top_p(gpu_lg, TF.fold_in(key, c - 1), 1.0, 1.0, 50)
    np.testing.assert_array_equal(t_ref.numpy(), tb[:, c])
    np.testing.assert_allclose(lps[:, c], lp_ref.numpy(), rtol=0, atol=2e-5)
  assert len({int(x) for x in tb[:, P:].reshape(-1)}) > B     # the draws differ from row to row


def test_qwen3_30b_a3b_width_decode(gpu):
  """Two layers of the Qwen3-30B-A3B workload at full width (D 2048, 32q / 4kv heads of 128, 128
  experts with top-8 routing, expert MLP 768, vocabulary 151936, int4 g128, LoRA r16 on the
  attention projections), batch 64: graph replay equals eager execution bit for bit, and the
  decode path's log-probabilities agree with compute_per_token_logps over the same tokens (the
  whole-sequence pass: other GEMM tiles, causal attention, 64 x more rows per expert)."""
  from tunix_amd import config, dummy_model
  from tunix_amd.generate import CacheConfig, Sampler
  from tunix_amd.generate.utils import IdTokenizer
  from tunix_amd.model import QLoRAModel
  from tunix_amd.rl.common import compute_per_token_logps
  cfg = config.qwen3_30b_a3b(num_layers=2)
  assert cfg.num_experts == 128 and cfg.num_experts_per_tok == 8 and cfg.hidden_dim == 768
  model = QLoRAModel(cfg, dummy_model.create_dummy_weights(cfg, seed=20260, device=gpu), gpu)
  B, P, T = 64, 32, 6
  tok = IdTokenizer(cfg.vocab_size, pad_id=0, eos_id=1)
  cc = CacheConfig(64, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim)
  prompts = _prompts(B, P, cfg.vocab_size, 20260)
  a = Sampler(model, tok, cc, use_graph=True)(prompts, T, max_prompt_length=P, return_logprobs=True, eos_tokens=[-1])
  b = Sampler(model, tok, cc, use_graph=False)(prompts, T, max_prompt_length=P, return_logprobs=True,
                                               return_logits=True, eos_tokens=[-1])
  for x, y in zip(a.tokens, b.tokens):
    np.testing.assert_array_equal(x, y)
  np.testing.assert_array_equal(np.asarray(a.logprobs), np.asarray(b.logprobs))
  comp = np.stack(a.tokens).astype(np.int32)
  lps = compute_per_token_logps(model, a.padded_prompt_tokens, comp, 0).cpu().numpy()
  got = np.asarray(a.logprobs, dtype=np.float32)
  assert np.isfinite(got).all() and np.isfinite(lps).all()
  lg = np.asarray(b.logits)
  chosen = np.take_along_axis(lg, comp[:, :, None].astype(np.int64), -1)[..., 0]
  ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(chosen), 2.0 ** -20))) - 7)
  err = np.abs(lps - got)
  print(f"qwen3-30b-a3b width: max {err.max():.3e} ({(err / ulp).max():.1f} ulp), mean {err.mean():.3e}, "
        f"median {np.median(err / ulp):.2f} ulp")
  # a routing near-tie (k-th against (k+1)-th router score within bf16 resolution) may send a token
  # to another expert in one of the two passes; such tokens move by more than rounding noise, the
  # bulk does not
  assert np.median(err / ulp) <= 2.0
  assert (err <= 8.0 * ulp + 2e-2).mean() >= 0.97
  assert err.max() <= 0.25


def _rollout_mode(sampler, model, B, seed):
  """The sampling-mode record Sampler.__call__ builds for temperature 1.0, top_p 1.0, no top-k (the
  categorical draw inside the head): every step commits freshly drawn tokens."""
  from tunix_amd import ops
  from tunix_amd.generate.sampler import _threefry_seed
  dev = model.device
  return {"name": "top_p", "forbidden": None, "eos": torch.tensor([-1], dtype=torch.int32, device=dev),
          "temperature": 1.0, "top_p": 1.0, "top_k": 0, "key": _threefry_seed(seed), "ws": None,
          "ids": torch.empty(B, dtype=torch.int32, device=dev),
          "logp": torch.empty(B, dtype=torch.float32, device=dev),
          "part_draw": torch.empty(B * ops.lmhead_nblocks(model.cfg.vocab_size) * 3, dtype=torch.float32, device=dev)}


def test_chain_handoffs_are_visible(gpu):
  """Every producer -> consumer hand-over of the decode chain crosses a kernel boundary inside
  one captured graph: the gate|up epilogue's activation tile -> the down GEMM's loads straight
  into LDS, the split-k partial planes -> the norm / the attention kernel that sums them, the
  adapter planes -> their reduce -> the t block of the next GEMM.  264 replays of the captured
  32-layer step at the benchmark's sizes (batch 128, contexts 760..1023, the last 32 slots of the
  1024-slot cache included), every one on freshly drawn tokens, each compared bit for bit with an
  eager execution of the same step on a second copy of the state: a consumer that saw a stale
  line of the previous step's data would differ."""
  from tunix_amd import config, dummy_model
  from tunix_amd.generate import CacheConfig, Sampler
  from tunix_amd.generate.sampler import _SamplingState
  from tunix_amd.generate.utils import IdTokenizer
  from tunix_amd.model import QLoRAModel, Runner
  cfg = config.llama31_8b()
  model = QLoRAModel(cfg, dummy_model.create_dummy_weights(cfg, seed=20261, device=gpu), gpu)
  B, P, S = 128, 760, 1024
  n_steps = S - P - 1                                         # the last one fills slot 1023
  tok = IdTokenizer(cfg.vocab_size, pad_id=0, eos_id=1)
  sampler = Sampler(model, tok, CacheConfig(S, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim))
  ids = np.stack([np.pad(p, (P - len(p), 0)) for p in _prompts(B, P, cfg.vocab_size, 20261)]).astype(np.int32)
  st_e = _SamplingState(model, ids, S, S, 0, False, True)
  st_g = _SamplingState(model, ids, S, S, 0, False, True)
  mode = _rollout_mode(sampler, model, B, seed=5)
  runner = Runner(model, B, 1, S, 0)
  sampler._prefill(st_e, runner, mode, False)
  sampler._decode_step(runner, st_e, mode)                    # lazy set-up happens outside the capture
  for name in ("token_buffer", "logprobs_buffer", "done", "step"):
    getattr(st_g, name).copy_(getattr(st_e, name))
  for dst, src in zip(st_g.kcache + st_g.vcache, st_e.kcache + st_e.vcache):
    dst.copy_(src)
  torch.cuda.synchronize()
  graph = torch.cuda.CUDAGraph()
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    with torch.cuda.graph(graph, stream=side):
      sampler._decode_step(runner, st_g, mode)
  torch.cuda.current_stream().wait_stream(side)
  bad = []
  seen = set()
  for i in range(n_steps - 1):
    graph.replay()
    torch.cuda.synchronize()
    xn_g, act_g, t_g = runner.xn.clone(), runner.act.clone(), runner.t.clone()
    sampler._decode_step(runner, st_e, mode)
    torch.cuda.synchronize()
    col = int(st_e.step.item())
    assert int(st_g.step.item()) == col == P + 1 + i + 1
    same = (torch.equal(xn_g, runner.xn), torch.equal(act_g, runner.act), torch.equal(t_g, runner.t),
            torch.equal(st_g.token_buffer[:, col], st_e.token_buffer[:, col]),
            torch.equal(st_g.logprobs_buffer[:, col], st_e.logprobs_buffer[:, col]))
    if not all(same):
      bad.append((i, col, same, int((xn_g != runner.xn).sum())))
      break
    seen.update(st_e.token_buffer[:, col].tolist())
  assert not bad, f"graph replay and eager execution differ (step, column, [xn, act, t, ids, logp] equal, differing elements): {bad}"
  assert int(st_e.step.item()) == S - 1                       # the rollout ran to the end of the cache
  assert torch.equal(st_g.kcache[-1], st_e.kcache[-1]) and torch.equal(st_g.vcache[0], st_e.vcache[0])
  assert len(seen) > 20 * B                                   # the draws really were fresh every step


def test_qwen3_30b_a3b_bench_prompt_and_cache(gpu):
  """The Qwen3-30B-A3B workload at the benchmark's prompt and cache (prompt 1024, 1280-slot cache,
  batch 64; three of the 48 layers): the split key range of decode attention with its combine
  launch at that cache size, the grouped GEMM at 64 x top-8 routes, prefill over 65536 rows.  Graph
  replay equals eager execution bit for bit; the decode path's log-probabilities agree with
  compute_per_token_logps over the same tokens."""
  from tunix_amd import config, dummy_model
  from tunix_amd.generate import CacheConfig, Sampler
  from tunix_amd.generate.utils import IdTokenizer
  from tunix_amd.model import QLoRAModel, Runner
  from tunix_amd.rl.common import compute_per_token_logps
  cfg = config.qwen3_30b_a3b(num_layers=3)
  model = QLoRAModel(cfg, dummy_model.create_dummy_weights(cfg, seed=20262, device=gpu), gpu)
  B, P, T, S = 64, 1024, 8, 1280
  assert Runner(model, B, 1, S, 0).kv_chunk > 0               # the key range is split at this size
  tok = IdTokenizer(cfg.vocab_size, pad_id=0, eos_id=1)
  cc = CacheConfig(S, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim)
  prompts = _prompts(B, P, cfg.vocab_size, 20262)
  a = Sampler(model, tok, cc, use_graph=True)(prompts, T, max_prompt_length=P, return_logprobs=True, eos_tokens=[-1])
  b = Sampler(model, tok, cc, use_graph=False)(prompts, T, max_prompt_length=P, return_logprobs=True,
                                               return_logits=True, eos_tokens=[-1])
  for x, y in zip(a.tokens, b.tokens):
    np.testing.assert_array_equal(x, y)
  np.testing.assert_array_equal(np.asarray(a.logprobs), np.asarray(b.logprobs))
  comp = np.stack(a.tokens).astype(np.int32)
  lps = compute_per_token_logps(model, a.padded_prompt_tokens, comp, 0).cpu().numpy()
  got = np.asarray(a.logprobs, dtype=np.float32)
  assert np.isfinite(got).all() and np.isfinite(lps).all()
  lg = np.stack([np.asarray(x) for x in b.logits])
  chosen = np.take_along_axis(lg, comp[:, :, None].astype(np.int64), -1)[..., 0]
  ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(chosen), 2.0 ** -20))) - 7)
  err = np.abs(lps - got)
  print(f"qwen3-30b-a3b prompt 1024 / cache 1280: max {err.max():.3e} ({(err / ulp).max():.1f} ulp), "
        f"mean {err.mean():.3e}, median {np.median(err / ulp):.2f} ulp")
  # (routing near-ties may send a token to another expert in one of the two passes: the bulk
  # agrees to rounding noise, as at the short prompt)
  assert np.median(err / ulp) <= 2.0
  assert (err <= 8.0 * ulp + 2e-2).mean() >= 0.97
  assert err.max() <= 0.25


def test_fused_logps_at_the_bench_launch_size(gpu):
  """One launch of the standalone fused log-probability pass at the benchmark's size: 16384 rows
  x 4096 -> 128256 (int4 g128 + LoRA r64), the many-row kernel with the head-statistics epilogue.
  Its statistics are checked against the logits of eight rows (first, last, both sides of row
  8192, others) materialised by the small-batch head kernel: logsumexp, the target's
  log-probability, normalisation; and every row's result is a finite log-probability."""
  from oracle import quant_ref as Q
  from tunix_amd import _lib as L
  from tunix_amd import ops
  D, V, r, group, rows = 4096, 128256, 64, 128, 16384
  g = torch.Generator(device=gpu).manual_seed(20263)
  x = torch.randn(rows, D, generator=g, device=gpu).to(torch.bfloat16)
  w = (torch.randn(D, V, generator=g, device=gpu) * 0.02).to(torch.bfloat16)
  a_t = (torch.randn(r, D, generator=g, device=gpu) * 0.02).to(torch.bfloat16)
  b_t = (torch.randn(V, r, generator=g, device=gpu) * 0.01).to(torch.bfloat16)
  targets = torch.randint(0, V, (rows,), generator=g, device=gpu, dtype=torch.int32)
  c, s = ops.quantize_pack(w, group, Q.INT4)
  del w
  t = torch.zeros(rows, r, dtype=torch.bfloat16, device=gpu)
  ops.lora_down(x, a_t, t)
  nvb = ops.lmhead_nblocks(V)

  def head(xx, tt, tg, n, logits=None):
    d = L.LmHeadDesc()
    d.M, d.D, d.V = n, D, V
    d.x, d.codes, d.scales, d.group, d.qtype = xx.data_ptr(), c.data_ptr(), s.data_ptr(), group, Q.INT4
    d.lora_rank, d.t, d.t_ld, d.lora_b, d.lora_scale = r, tt.data_ptr(), r, b_t.data_ptr(), 1.0
    d.temperature = 1.0
    part = torch.empty(n * nvb * 4, dtype=torch.float32, device=gpu)
    tlp = torch.empty(n, dtype=torch.float32, device=gpu)
    lse = torch.empty(n, dtype=torch.float32, device=gpu)
    d.targets, d.part, d.target_logp, d.lse = tg.data_ptr(), part.data_ptr(), tlp.data_ptr(), lse.data_ptr()
    if logits is not None:
      d.logits_out = logits.data_ptr()
    ops.lmhead(d)
    torch.cuda.synchronize()
    return tlp, lse

  tlp, lse = head(x, t, targets, rows)
  assert torch.isfinite(tlp).all() and (tlp <= 0).all() and torch.isfinite(lse).all()
  idx = torch.tensor([0, 1, 4095, 8191, 8192, 12001, 16382, 16383], device=gpu)
  lg = torch.empty(len(idx), V, dtype=torch.float32, device=gpu)
  tlp8, lse8 = head(x[idx].contiguous(), t[idx].contiguous(), targets[idx].contiguous(), len(idx), logits=lg)
  ref_lse = torch.logsumexp(lg, -1)
  torch.testing.assert_close(lse8, ref_lse, rtol=0, atol=2e-5)          # the small kernel against its own logits
  torch.testing.assert_close(lse[idx], ref_lse, rtol=0, atol=2e-3)      # the many-row launch: bf16 logits that may
  sel = lg[torch.arange(len(idx)), targets[idx].long()] - ref_lse       # round apart by one ulp in a few places
  torch.testing.assert_close(tlp[idx], sel, rtol=0, atol=1e-2)
  torch.testing.assert_close(torch.exp(lg - ref_lse[:, None]).sum(-1), torch.ones(len(idx), device=gpu), rtol=0, atol=1e-4)
  # logits of a random target are N(0, sigma^2) with sigma^2 = D * 0.02^2, so the mean
  # log-probability is -(log V + sigma^2 / 2) up to the quantisation of the weights
  assert abs(float(tlp.mean()) + np.log(V) + D * 0.02 ** 2 / 2) < 0.1


def test_expanded_weight_copy_gives_the_same_whole_sequence_pass(gpu):
  """One layer of the 8B shape, 32 x 96 tokens (3072 rows: every linear on the many-row GEMM): the model that keeps
  the converted second copy of its NF4 weights and the one that converts codes in the loop give
  bit-identical per-token log-probabilities, and a base-weight update refreshes the copy."""
  from tunix_amd import config, dummy_model
  from tunix_amd.model import QLoRAModel
  from tunix_amd.rl.common import compute_per_token_logps
  cfg = config.llama31_8b(num_layers=1, vocab_size=4096)
  w = dummy_model.create_dummy_weights(cfg, seed=20261, device=gpu)
  packed = QLoRAModel(cfg, w, gpu, expand_many_rows=False)
  expanded = QLoRAModel(cfg, w, gpu, expand_many_rows=True)
  assert all(f.expanded is None for f in packed._linears()) and packed.head_expanded is None
  assert all(f.expanded is not None for f in expanded._linears()) and expanded.head_expanded is not None
  # (the dense head's copy sends the head itself to another kernel, with another summation order:
  # checked on its own below; the linears' copies change no bit)
  head_copy, expanded.head_expanded = expanded.head_expanded, None
  g = np.random.Generator(np.random.PCG64(20261))
  prompt = torch.from_numpy(g.integers(2, cfg.vocab_size, size=(32, 32)).astype(np.int32)).to(gpu)
  completion = torch.from_numpy(g.integers(2, cfg.vocab_size, size=(32, 64)).astype(np.int32)).to(gpu)
  a = compute_per_token_logps(packed, prompt, completion, pad_id=0, eos_id=1)
  b = compute_per_token_logps(expanded, prompt, completion, pad_id=0, eos_id=1)
  assert torch.isfinite(a).all() and torch.equal(a, b)
  # new base weights for one projection: both models re-quantise, the copy follows
  w2 = dict(w)
  w2["l0.wo"] = (w["l0.wo"].float() * 1.5).to(w["l0.wo"].dtype)
  packed.update_params(w2)
  expanded.update_params(w2)
  a2 = compute_per_token_logps(packed, prompt, completion, pad_id=0, eos_id=1)
  b2 = compute_per_token_logps(expanded, prompt, completion, pad_id=0, eos_id=1)
  assert torch.equal(a2, b2) and not torch.equal(a, a2)
  # the dense head through its copy (the many-row kernel's statistics epilogue instead of the
  # 128 x 128 head kernel): same logits up to the rounding of a bf16 logit whose fp32 sum came
  # out in another order
  expanded.head_expanded = head_copy
  c2 = compute_per_token_logps(expanded, prompt, completion, pad_id=0, eos_id=1)
  assert torch.isfinite(c2).all() and not torch.equal(c2, b2)
  assert (c2 - b2).abs().max().item() < 2e-2 and (c2 - b2).abs().mean().item() < 2e-3
  # ... and an update of the head refreshes the copy
  w3 = dict(w2)
  w3["lm_head"] = (w["lm_head"].float() * 0.5).to(w["lm_head"].dtype)
  expanded.update_params(w3)
  packed.update_params(w3)
  c3 = compute_per_token_logps(expanded, prompt, completion, pad_id=0, eos_id=1)
  a3 = compute_per_token_logps(packed, prompt, completion, pad_id=0, eos_id=1)
  assert (c3 - a3).abs().max().item() < 2e-2 and (c3 - c2).abs().max().item() > 0.05
