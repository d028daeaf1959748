"""Pins oracle/model_ref.py (fp32 reference mode) against transformers' implementations of the
same architectures on random weights: the equivalence the reference asserts for its own models
in tests/model_alignment/qwen_align_test.py:113-200 (logits of the HF torch model vs the JAX
model, atol/rtol 1e-3).  The HF model receives the oracle's effective weights
W_eff = dequant(quant(W)) + (alpha / r) * A @ B (tunix/models/safetensors_saver.py:107), so a
wrong norm, RoPE pairing, GQA grouping, mask, activation or LoRA merge shows up as a logit
mismatch; the quantiser itself cancels out here and is pinned in test_oracle_quant.py.
"""
import numpy as np
import pytest
import torch

from oracle import model_ref as MR
from oracle import utils_ref as U
from tunix_amd import config, dummy_model

transformers = pytest.importorskip("transformers")


def _effective(ref: MR.RefModel, name: str) -> torch.Tensor:
  w = ref.q[name] if name in ref.q else ref.w[name].float()
  if name in ref.lora:
    a, b = ref.lora[name]
    w = w + (ref.cfg.lora_alpha / ref.cfg.lora_rank) * (a.double() @ b.double()).float()
  return w


def _oracle_logits(cfg, w, ids):
  ref = MR.RefModel(cfg, w, bf16=False, acc=torch.float64)
  B, L = ids.shape
  mask = torch.from_numpy(U.make_causal_attn_mask(np.ones((B, L), dtype=bool)))
  pos = torch.arange(L)[None].repeat(B, 1)
  cache = ref.init_cache(B, L)
  return ref, ref(torch.from_numpy(ids).long(), pos, cache, mask, 0)


def _fill_common(sd, ref, cfg, prefix="model."):
  sd[prefix + "embed_tokens.weight"] = ref.w["embed"].float()
  sd[prefix + "norm.weight"] = ref.w["final_norm"].float()
  for i in range(cfg.num_layers):
    p, s = f"l{i}.", f"{prefix}layers.{i}."
    for ours, theirs in (("wq", "q_proj"), ("wk", "k_proj"), ("wv", "v_proj"), ("wo", "o_proj")):
      sd[s + f"self_attn.{theirs}.weight"] = _effective(ref, p + ours).t().contiguous()
    if cfg.family in ("qwen3", "gemma3"):
      sd[s + "self_attn.q_norm.weight"] = ref.w[p + "q_norm"].float()
      sd[s + "self_attn.k_norm.weight"] = ref.w[p + "k_norm"].float()
    if not cfg.num_experts:
      for ours, theirs in (("w_gate", "gate_proj"), ("w_up", "up_proj"), ("w_down", "down_proj")):
        sd[s + f"mlp.{theirs}.weight"] = _effective(ref, p + ours).t().contiguous()


def _randomize_norms(w, seed):
  g = torch.Generator().manual_seed(seed)
  for k in w:
    if k.endswith("norm"):
      w[k] = (w[k].float() + 0.2 * torch.randn(w[k].shape, generator=g)).to(torch.bfloat16)
  return w


def _check(hf, sd, ids, got, tol=1e-3):
  missing, unexpected = hf.load_state_dict(sd, strict=False)
  assert not unexpected, unexpected
  assert all("rotary" in m or "inv_freq" in m for m in missing), missing
  hf.eval()
  with torch.no_grad():
    want = hf(torch.from_numpy(ids).long()).logits.float()
  err = (got - want).abs().max().item()
  assert err <= tol, f"max |logit diff| {err}"
  # the comparison has teeth: logits are not all alike
  assert want.std().item() > 10 * tol


def test_llama_matches_transformers():
  cfg = config.llama31_8b(num_layers=2, vocab_size=160, embed_dim=64, hidden_dim=128, num_heads=4,
                          num_kv_heads=2, head_dim=16, lora_rank=8, lora_alpha=16.0, group=32,
                          rope_theta=500000.0)
  w = _randomize_norms(dummy_model.create_dummy_weights(cfg, seed=1, scale=0.2, lora_b_scale=0.1), 1)
  ids = np.random.default_rng(1).integers(0, cfg.vocab_size, size=(2, 12))
  ref, got = _oracle_logits(cfg, w, ids)
  hc = transformers.LlamaConfig(vocab_size=cfg.vocab_size, hidden_size=cfg.embed_dim,
                                intermediate_size=cfg.hidden_dim, num_hidden_layers=cfg.num_layers,
                                num_attention_heads=cfg.num_heads, num_key_value_heads=cfg.num_kv_heads,
                                head_dim=cfg.head_dim, rms_norm_eps=cfg.norm_eps, rope_theta=cfg.rope_theta,
                                tie_word_embeddings=False, attention_bias=False, mlp_bias=False)
  hf = transformers.LlamaForCausalLM(hc).float()
  sd = {}
  _fill_common(sd, ref, cfg)
  for i in range(cfg.num_layers):
    sd[f"model.layers.{i}.input_layernorm.weight"] = ref.w[f"l{i}.attn_norm"].float()
    sd[f"model.layers.{i}.post_attention_layernorm.weight"] = ref.w[f"l{i}.mlp_norm"].float()
  sd["lm_head.weight"] = ref.w["lm_head"].float().t().contiguous()
  _check(hf, sd, ids, got)


def test_qwen3_matches_transformers():
  cfg = config.tiny_qwen3(vocab_size=160, embed_dim=64, hidden_dim=96, num_heads=4, num_kv_heads=2,
                          head_dim=32, group=32, lora_rank=8, lora_alpha=8.0)
  w = _randomize_norms(dummy_model.create_dummy_weights(cfg, seed=2, scale=0.2, lora_b_scale=0.1), 2)
  ids = np.random.default_rng(2).integers(0, cfg.vocab_size, size=(2, 10))
  ref, got = _oracle_logits(cfg, w, ids)
  hc = transformers.Qwen3Config(vocab_size=cfg.vocab_size, hidden_size=cfg.embed_dim,
                                intermediate_size=cfg.hidden_dim, num_hidden_layers=cfg.num_layers,
                                num_attention_heads=cfg.num_heads, num_key_value_heads=cfg.num_kv_heads,
                                head_dim=cfg.head_dim, rms_norm_eps=cfg.norm_eps, rope_theta=cfg.rope_theta,
                                tie_word_embeddings=False, attention_bias=False, use_sliding_window=False)
  hf = transformers.Qwen3ForCausalLM(hc).float()
  sd = {}
  _fill_common(sd, ref, cfg)
  for i in range(cfg.num_layers):
    sd[f"model.layers.{i}.input_layernorm.weight"] = ref.w[f"l{i}.attn_norm"].float()
    sd[f"model.layers.{i}.post_attention_layernorm.weight"] = ref.w[f"l{i}.mlp_norm"].float()
  sd["lm_head.weight"] = ref.w["lm_head"].float().t().contiguous()
  _check(hf, sd, ids, got)


def test_qwen3_moe_matches_transformers():
  cfg = config.qwen3_30b_a3b(num_layers=2, vocab_size=96, embed_dim=64, hidden_dim=32, num_heads=4,
                             num_kv_heads=2, head_dim=16, group=32, lora_rank=8, lora_alpha=8.0,
                             num_experts=8, num_experts_per_tok=2)
  w = _randomize_norms(dummy_model.create_dummy_weights(cfg, seed=3, scale=0.2, lora_b_scale=0.1), 3)
  ids = np.random.default_rng(3).integers(0, cfg.vocab_size, size=(2, 9))
  ref, got = _oracle_logits(cfg, w, ids)
  hc = transformers.Qwen3MoeConfig(
      vocab_size=cfg.vocab_size, hidden_size=cfg.embed_dim, intermediate_size=4 * cfg.hidden_dim,
      moe_intermediate_size=cfg.hidden_dim, num_hidden_layers=cfg.num_layers,
      num_attention_heads=cfg.num_heads, num_key_value_heads=cfg.num_kv_heads, head_dim=cfg.head_dim,
      rms_norm_eps=cfg.norm_eps, rope_theta=cfg.rope_theta, tie_word_embeddings=False,
      num_experts=cfg.num_experts, num_experts_per_tok=cfg.num_experts_per_tok, norm_topk_prob=True,
      decoder_sparse_step=1, mlp_only_layers=[], use_sliding_window=False)
  hf = transformers.Qwen3MoeForCausalLM(hc).float()
  sd = {}
  _fill_common(sd, ref, cfg)
  for i in range(cfg.num_layers):
    p, s = f"l{i}.", f"model.layers.{i}."
    sd[s + "input_layernorm.weight"] = ref.w[p + "attn_norm"].float()
    sd[s + "post_attention_layernorm.weight"] = ref.w[p + "mlp_norm"].float()
    sd[s + "mlp.gate.weight"] = ref.w[p + "router"].float().t().contiguous()
    g, u, d = ref.q[p + "e_gate"], ref.q[p + "e_up"], ref.q[p + "e_down"]     # [E,D,F] / [E,F,D]
    sd[s + "mlp.experts.gate_up_proj"] = torch.cat([g, u], dim=2).transpose(1, 2).contiguous()
    sd[s + "mlp.experts.down_proj"] = d.transpose(1, 2).contiguous()
  sd["lm_head.weight"] = ref.w["lm_head"].float().t().contiguous()
  _check(hf, sd, ids, got)


def test_gemma3_matches_transformers():
  cfg = config.gemma3_1b(num_layers=7, vocab_size=128, embed_dim=64, hidden_dim=96, num_heads=4,
                         num_kv_heads=1, head_dim=16, group=32, lora_rank=8, lora_alpha=8.0,
                         sliding_window=64)
  w = _randomize_norms(dummy_model.create_dummy_weights(cfg, seed=4, scale=0.2, lora_b_scale=0.1), 4)
  ids = np.random.default_rng(4).integers(0, cfg.vocab_size, size=(2, 11))
  ref, got = _oracle_logits(cfg, w, ids)
  kw = dict(vocab_size=cfg.vocab_size, hidden_size=cfg.embed_dim, intermediate_size=cfg.hidden_dim,
            num_hidden_layers=cfg.num_layers, num_attention_heads=cfg.num_heads,
            num_key_value_heads=cfg.num_kv_heads, head_dim=cfg.head_dim, rms_norm_eps=1e-6,
            query_pre_attn_scalar=cfg.head_dim, sliding_window=cfg.sliding_window,
            tie_word_embeddings=True, attention_bias=False, final_logit_softcapping=None,
            attn_logit_softcapping=None)
  try:
    hc = transformers.Gemma3TextConfig(
        **kw, rope_parameters={
            "full_attention": {"rope_type": "default", "rope_theta": cfg.global_base_frequency},
            "sliding_attention": {"rope_type": "default", "rope_theta": cfg.local_base_frequency}})
  except TypeError:
    hc = transformers.Gemma3TextConfig(**kw, rope_theta=cfg.global_base_frequency,
                                       rope_local_base_freq=cfg.local_base_frequency)
  assert [t == "sliding_attention" for t in hc.layer_types] == [cfg.is_local_layer(i) for i in range(cfg.num_layers)]
  hf = transformers.Gemma3ForCausalLM(hc).float()
  sd = {}
  _fill_common(sd, ref, cfg)
  for i in range(cfg.num_layers):
    p, s = f"l{i}.", f"model.layers.{i}."
    sd[s + "input_layernorm.weight"] = ref.w[p + "attn_norm"].float()
    sd[s + "post_attention_layernorm.weight"] = ref.w[p + "post_attn_norm"].float()
    sd[s + "pre_feedforward_layernorm.weight"] = ref.w[p + "mlp_norm"].float()
    sd[s + "post_feedforward_layernorm.weight"] = ref.w[p + "post_ffw_norm"].float()
  sd["lm_head.weight"] = ref.w["embed"].float()
  _check(hf, sd, ids, got, tol=2e-3)


def test_attention_brute_force_fp64():
  """GQA grouping, masking and the softmax against an explicit per-head loop in float64."""
  cfg = config.tiny_qwen3(num_layers=1, vocab_size=64)
  B, T, S, Hq, Hkv, dh = 2, 3, 7, 4, 2, 8
  g = torch.Generator().manual_seed(0)
  q = torch.randn(B, T, Hq, dh, generator=g)
  k = torch.randn(B, S, Hkv, dh, generator=g)
  v = torch.randn(B, S, Hkv, dh, generator=g)
  mask = torch.rand(B, T, S, generator=g) > 0.3
  mask[..., 0] = True
  m = MR.RefModel.__new__(MR.RefModel)
  m.cfg, m.bf16, m.acc = cfg, False, torch.float64
  got = m.attention(q, k, v, mask, dh ** -0.5)
  want = torch.zeros(B, T, Hq, dh, dtype=torch.float64)
  for b in range(B):
    for t in range(T):
      for h in range(Hq):
        kv = h // (Hq // Hkv)
        s = (k[b, :, kv].double() @ q[b, t, h].double()) * dh ** -0.5
        s = torch.where(mask[b, t], s, torch.tensor(-1e30, dtype=torch.float64))
        p = torch.softmax(s, 0)
        want[b, t, h] = p @ v[b, :, kv].double()
  assert (got.double() - want).abs().max().item() < 1e-5
