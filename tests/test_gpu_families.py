"""End-to-end GPU parity of the sampler for the other model families of the path, at shapes the
CPU oracle finishes in seconds (same architecture rules as the full-size configurations:
Llama-3 NF4 g64 + LoRA, Gemma-3 int4 g128 with sliding-window layers, tied embeddings and
GeGLU, Qwen3-MoE int4 g128 with top-k routing).  Same bar as test_gpu_sampler.py: greedy ids
equal the teacher-forced oracle arg-max except at listed near-ties (<= 2 bf16 ulps), and
log-probabilities <= 2e-2."""
import numpy as np
import pytest
import torch

from oracle import model_ref as MR
from test_gpu_sampler import _check_greedy, _oracle_full_logits, _prompts

pytestmark = pytest.mark.gpu


def _run(cfg, gpu, B, P, T, wseed, **call_kw):
  from tunix_amd import dummy_model
  from tunix_amd.generate import CacheConfig, Sampler
  from tunix_amd.generate.utils import IdTokenizer
  from tunix_amd.model import QLoRAModel
  w = dummy_model.create_dummy_weights(cfg, seed=wseed)
  model = QLoRAModel(cfg, w, gpu)
  tok = IdTokenizer(cfg.vocab_size, pad_id=0, eos_id=1)
  sampler = Sampler(model, tok, CacheConfig(P + T, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim))
  prompts = _prompts(B, P, cfg.vocab_size, wseed)
  out = sampler(prompts, max_generation_steps=T, max_prompt_length=P, return_logprobs=True, eos_tokens=[-1],
                **call_kw)
  st = sampler._last_state
  return w, out, st.token_buffer.cpu().numpy(), st.logprobs_buffer.cpu().numpy()


def _greedy_case(cfg, gpu, B, P, T, seed, lp_tol=2e-2):
  w, out, tb, lps = _run(cfg, gpu, B, P, T, seed)
  assert all(len(t) == T for t in out.tokens)
  ref = MR.RefModel(cfg, w)
  logits = _oracle_full_logits(ref, tb, 0)
  report, n = _check_greedy(tb, logits, P, lps, lp_tol=lp_tol, label=f"{cfg.family} small shape, greedy")
  print(f"{cfg.family}: {n - len(report)}/{n} greedy ids equal the oracle arg-max; near-ties: {report}")
  assert len(report) <= max(1, n // 20)


def test_llama3_nf4_greedy(gpu):
  from tunix_amd import config
  cfg = config.llama31_8b(num_layers=2, vocab_size=8192, embed_dim=512, hidden_dim=1024, num_heads=8,
                          num_kv_heads=2, head_dim=64, lora_rank=32, lora_alpha=32.0)
  assert cfg.qtype == config.Q_NF4 and cfg.group == 64
  _greedy_case(cfg, gpu, B=6, P=32, T=24, seed=31)


def test_gemma3_sliding_window_greedy(gpu):
  from tunix_amd import config
  # 7 layers = 5 local + 1 global + 1 local; the 16-token window is shorter than prompt + output
  cfg = config.gemma3_1b(num_layers=7, vocab_size=8192, embed_dim=512, hidden_dim=1024, num_heads=4,
                         num_kv_heads=1, head_dim=128, sliding_window=16)
  assert cfg.tied_embedding and cfg.group == 128
  # Gemma-3 multiplies the embeddings by sqrt(D) and ties the head to them, so its logits reach
  # 2-4 in magnitude where one bf16 ulp is 0.008-0.016; seven layers of all-bf16 norms leave the
  # chosen logit up to four of those ulps from the oracle's, hence 4e-2 here
  _greedy_case(cfg, gpu, B=4, P=24, T=24, seed=32, lp_tol=4e-2)


def test_qwen3_moe_greedy(gpu):
  from tunix_amd import config
  cfg = config.qwen3_30b_a3b(num_layers=2, vocab_size=8192, embed_dim=512, hidden_dim=256, num_heads=8,
                             num_kv_heads=2, head_dim=64, num_experts=16, num_experts_per_tok=4)
  assert cfg.group == 128 and cfg.lora_targets == config.ATTN_LINEARS
  B, P, T = 6, 24, 16
  w, out, tb, lps = _run(cfg, gpu, B, P, T, 33)
  ref = MR.RefModel(cfg, w)
  logits = _oracle_full_logits(ref, tb, 0)
  # Top-k routing is a discontinuity: where the k-th and (k+1)-th router scores of a token lie
  # within two bf16 ulps, a different summation order selects another expert.  The strict
  # check covers every position whose own token has no such near-tie in any layer; the others
  # are counted and bounded loosely.
  tie = torch.zeros(B, P + T, dtype=torch.bool)
  for i in range(cfg.num_layers):
    tie |= ref.route_near_tie[i]
  tainted = tie  # the token's own routing; earlier tokens' flips reach it only through attention
  lp = torch.log_softmax(logits.float(), -1)
  strict = loose = 0
  for b in range(B):
    for c in range(P, P + T):
      lg = logits[b, c - 1]
      best, tok = int(torch.argmax(lg)), int(tb[b, c])
      err = abs(float(lps[b, c]) - float(lp[b, c - 1, tok]))
      ulp = 2.0 ** (np.floor(np.log2(max(abs(float(lg[best])), 2.0 ** -120))) - 7)
      if not bool(tainted[b, c - 1]):
        strict += 1
        assert err <= 2e-2, (b, c, err)
        assert tok == best or float(lg[best] - lg[tok]) <= 2 * ulp, (b, c, tok, best)
      else:
        loose += 1
        assert err <= 0.25, (b, c, err)
  print(f"qwen3-moe: {strict} positions checked strictly, {loose} after a routing near-tie")
  assert strict >= (B * T) // 3


def test_gemma3_temperature_topk_sampling(gpu):
  """temperature 1.0, top-k 50 from a fixed seed (the Gemma-3 parity configuration): the ids
  are the oracle's draw from the logits the GPU produced, and those logits match the
  teacher-forced oracle to bf16 resolution."""
  from oracle import sampler_ref as SR
  from oracle import threefry as TF
  from tunix_amd import config
  cfg = config.gemma3_1b(num_layers=3, vocab_size=8192, embed_dim=512, hidden_dim=1024, num_heads=4,
                         num_kv_heads=1, head_dim=128, sliding_window=512)
  B, P, T = 4, 16, 10
  w, out, tb, lps = _run(cfg, gpu, B, P, T, 34, temperature=1.0, top_p=1.0, top_k=50, seed=7, return_logits=True)
  ref = MR.RefModel(cfg, w)
  logits = _oracle_full_logits(ref, tb, 0)
  key = TF.prng_key(7)
  for c in range(P, P + T):
    gpu_lg = torch.from_numpy(np.stack([out.logits[b][c - P] for b in range(B)]))
    t_ref, lp_ref = SR.sample_top_p(gpu_lg, TF.fold_in(key, c - 1), 1.0, 1.0, 50)
    np.testing.assert_array_equal(t_ref.numpy(), tb[:, c])
    diff = (gpu_lg - logits[:, c - 1]).abs().max().item()
    assert diff <= 2.0 ** -6 * max(1.0, logits[:, c - 1].abs().max().item())
    lp_full = torch.log_softmax(logits[:, c - 1].float(), -1)
    for b in range(B):
      mag = max(abs(float(logits[b, c - 1, tb[b, c]])), 1e-30)
      tol = max(4e-2, 2.0 * 2.0 ** (np.floor(np.log2(mag)) - 7))
      assert abs(lps[b, c] - float(lp_full[b, tb[b, c]])) <= tol
