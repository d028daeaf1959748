"""from_reference_tree: arrays laid out like the reference's nnx parameter tree -> the flat names
QLoRAModel consumes.  The inverse map below is written from the shapes the reference documents
(llama3/model.py:311-334, :461-487; gemma3/model.py:527-565; LoRA leaves:
tunix/models/llama3/mapping_sglang_jax.py:64-145, gemma3/params.py:301-318 with the merge at
tunix/models/safetensors_saver.py:88-107), independently of the function under test: a round trip
must reproduce every tensor, and the effective weight W + A B of each projection, formed in the
tree's own layout the way the reference's merge does, must equal the flat one."""
import numpy as np
import pytest
import torch

from tunix_amd import config, dummy_model


def _to_tree(cfg, w):
  D, H, K, dh, r = cfg.embed_dim, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim, cfg.lora_rank
  t = {"embedder.input_embedding": w["embed"]}
  nk = "scale" if cfg.family == "gemma3" else "w"
  t[f"final_norm.{nk}"] = w["final_norm"]
  if "lm_head" in w:
    t["lm_head.w"] = w["lm_head"]
  for i in range(cfg.num_layers):
    s, p = f"layers.{i}.", f"l{i}."
    if cfg.family == "gemma3":
      t[s + "pre_attention_norm.scale"] = w[p + "attn_norm"]
      t[s + "post_attention_norm.scale"] = w[p + "post_attn_norm"]
      t[s + "pre_ffw_norm.scale"] = w[p + "mlp_norm"]
      t[s + "post_ffw_norm.scale"] = w[p + "post_ffw_norm"]
      t[s + "attn._query_norm.scale"] = w[p + "q_norm"]
      t[s + "attn._key_norm.scale"] = w[p + "k_norm"]
      t[s + "attn.q_einsum.w"] = w[p + "wq"].reshape(D, H, dh).permute(1, 0, 2)          # [N,D,H]
      t[s + "attn.kv_einsum.w"] = torch.stack([w[p + "wk"].reshape(D, K, dh).permute(1, 0, 2),
                                               w[p + "wv"].reshape(D, K, dh).permute(1, 0, 2)])  # [2,K,D,H]
      t[s + "attn.attn_vec_einsum.w"] = w[p + "wo"].reshape(H, dh, D)
      if p + "wq.lora_a" in w:
        t[s + "attn.q_einsum.w_lora_a"] = w[p + "wq.lora_a"]
        t[s + "attn.q_einsum.w_lora_b"] = w[p + "wq.lora_b"].reshape(r, H, dh)
        t[s + "attn.kv_einsum.w_lora_a"] = w[p + "wk.lora_a"]                            # one A for k and v
        t[s + "attn.kv_einsum.w_lora_b"] = torch.stack([w[p + "wk.lora_b"].reshape(r, K, dh),
                                                        w[p + "wv.lora_b"].reshape(r, K, dh)], dim=1)
        t[s + "attn.attn_vec_einsum.w_lora_a"] = w[p + "wo.lora_a"].reshape(H, dh, r)
        t[s + "attn.attn_vec_einsum.w_lora_b"] = w[p + "wo.lora_b"]
    else:
      t[s + "input_layernorm.w"] = w[p + "attn_norm"]
      t[s + "post_attention_layernorm.w"] = w[p + "mlp_norm"]
      if cfg.family == "qwen3":
        t[s + "attn.q_norm.w"] = w[p + "q_norm"]
        t[s + "attn.k_norm.w"] = w[p + "k_norm"]
      for src, dst, heads in (("q_proj", "wq", H), ("k_proj", "wk", K), ("v_proj", "wv", K)):
        t[s + f"attn.{src}.w"] = w[p + dst].reshape(D, heads, dh)
        if p + dst + ".lora_a" in w:
          t[s + f"attn.{src}.w_lora_a"] = w[p + dst + ".lora_a"]
          t[s + f"attn.{src}.w_lora_b"] = w[p + dst + ".lora_b"].reshape(r, heads, dh)
      t[s + "attn.o_proj.w"] = w[p + "wo"].reshape(H, dh, D)
      if p + "wo.lora_a" in w:
        t[s + "attn.o_proj.w_lora_a"] = w[p + "wo.lora_a"].reshape(H, dh, r)
        t[s + "attn.o_proj.w_lora_b"] = w[p + "wo.lora_b"]
    if cfg.num_experts:
      t[s + "mlp.router.kernel"] = w[p + "router"]
      for src, dst in (("gate_proj", "e_gate"), ("up_proj", "e_up"), ("down_proj", "e_down")):
        t[s + f"mlp.{src}"] = w[p + dst]
    else:
      for src, dst in (("gate_proj", "w_gate"), ("up_proj", "w_up"), ("down_proj", "w_down")):
        t[s + f"mlp.{src}.kernel"] = w[p + dst]
        if p + dst + ".lora_a" in w:
          t[s + f"mlp.{src}.kernel_lora_a"] = w[p + dst + ".lora_a"]
          t[s + f"mlp.{src}.kernel_lora_b"] = w[p + dst + ".lora_b"]
  return t


CASES = {
    "llama3": lambda: config.llama31_8b(num_layers=2, vocab_size=96, embed_dim=64, hidden_dim=128, num_heads=4,
                                        num_kv_heads=2, head_dim=16, lora_rank=4, lora_alpha=4.0),
    "qwen3": lambda: config.tiny_qwen3(num_layers=2, vocab_size=96, embed_dim=64, hidden_dim=128, num_heads=4,
                                       num_kv_heads=2, head_dim=16, lora_rank=4, lora_alpha=4.0),
    "gemma3": lambda: config.gemma3_1b(num_layers=2, vocab_size=96, embed_dim=64, hidden_dim=128, num_heads=4,
                                       num_kv_heads=1, head_dim=16, lora_rank=4, lora_alpha=4.0),
    "qwen3-moe": lambda: config.qwen3_30b_a3b(num_layers=2, vocab_size=96, embed_dim=64, hidden_dim=32, num_heads=4,
                                              num_kv_heads=2, head_dim=16, lora_rank=4, lora_alpha=4.0,
                                              num_experts=4, num_experts_per_tok=2),
}


@pytest.mark.parametrize("name", list(CASES))
def test_round_trip_through_the_reference_layout(name):
  cfg = CASES[name]()
  w = dummy_model.create_dummy_weights(cfg, seed=3)
  if cfg.family == "gemma3":   # k and v share their A in the reference's kv_einsum
    for i in range(cfg.num_layers):
      w[f"l{i}.wv.lora_a"] = w[f"l{i}.wk.lora_a"].clone()
  tree = {k: v.numpy() if v.dtype != torch.bfloat16 else v for k, v in _to_tree(cfg, w).items()}
  back = dummy_model.from_reference_tree(cfg, tree)
  assert set(back) == set(w), (sorted(set(w) - set(back)), sorted(set(back) - set(w)))
  for k in w:
    assert tuple(back[k].shape) == tuple(w[k].shape), k
    assert torch.equal(back[k].float(), w[k].float()), k
  assert any(k.endswith(".lora_a") for k in back)


def test_gemma3_lora_leaves_merge_like_the_reference_saver():
  """safetensors_saver.py:88-107 reshapes a 3-D lora_a to [d0*d1, d2] and a 3-D lora_b to
  [d0, d1*d2] and forms lora_a @ lora_b; gemma3/params.py:301-318 first splits kv_einsum's
  lora_b [r,2,K,dh] into k ([:, 0]) and v ([:, 1]) with the shared lora_a.  The merged delta of
  every attention projection in that layout equals A @ B of the flat leaves."""
  cfg = CASES["gemma3"]()
  w = dummy_model.create_dummy_weights(cfg, seed=4)
  w["l0.wv.lora_a"] = w["l0.wk.lora_a"].clone()
  w["l1.wv.lora_a"] = w["l1.wk.lora_a"].clone()
  tree = _to_tree(cfg, w)
  flat = dummy_model.from_reference_tree(cfg, tree)

  def merged(a, b):
    a, b = a.float(), b.float()
    if a.ndim == 3:
      a = a.reshape(a.shape[0] * a.shape[1], a.shape[2])
    if b.ndim == 3:
      b = b.reshape(b.shape[0], b.shape[1] * b.shape[2])
    return a @ b

  s = "layers.0.attn."
  kv_a, kv_b = tree[s + "kv_einsum.w_lora_a"], tree[s + "kv_einsum.w_lora_b"]
  pairs = {"wq": (tree[s + "q_einsum.w_lora_a"], tree[s + "q_einsum.w_lora_b"]),
           "wk": (kv_a, kv_b[:, 0]), "wv": (kv_a, kv_b[:, 1]),
           "wo": (tree[s + "attn_vec_einsum.w_lora_a"], tree[s + "attn_vec_einsum.w_lora_b"])}
  for name, (a, b) in pairs.items():
    want = merged(a, b)
    got = flat[f"l0.{name}.lora_a"].float() @ flat[f"l0.{name}.lora_b"].float()
    assert want.shape == got.shape == tuple(w[f"l0.{name}"].shape), name
    np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=1e-6, atol=1e-9)
