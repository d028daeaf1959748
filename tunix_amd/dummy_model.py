"""Random-initialised weights of the shapes the sampler runs on
(tunix/models/dummy_model_creator.py:29-92: every kernel ~ scale * N(0, 1), default scale 0.02).

Weights use flat names with 2-D kernels, the layout QLoRAModel consumes:
  embed [V,D], final_norm [D], lm_head [D,V] (absent with tied embeddings)
  l{i}.attn_norm, l{i}.mlp_norm [D]  (+ q_norm/k_norm [dh]; gemma3: post_attn_norm, post_ffw_norm)
  l{i}.wq [D,Hq*dh], wk/wv [D,Hkv*dh], wo [Hq*dh,D], w_gate/w_up [D,F], w_down [F,D]
  MoE: l{i}.router [D,E], l{i}.e_gate/e_up [E,D,F], l{i}.e_down [E,F,D]
  LoRA: <linear>.lora_a [K,r] ~ N(0,0.02), <linear>.lora_b [r,N] ~ N(0,0.01)
Norm weights are ones (llama3 / qwen3: `w * x`) or zeros (gemma3: `(1 + scale) * x`).
`from_reference_tree` converts arrays laid out like the reference's nnx parameter tree.
"""
from __future__ import annotations

import numpy as np
import torch

from .config import ModelConfig


def create_dummy_weights(cfg: ModelConfig, seed: int = 0, device="cpu", scale: float = 0.02,
                         lora_b_scale: float = 0.01) -> dict:
  dev = torch.device(device)
  gen = torch.Generator(device=dev)
  gen.manual_seed(seed)
  bf = torch.bfloat16

  def normal(*shape, s=scale):
    return (torch.randn(*shape, generator=gen, device=dev, dtype=torch.float32) * s).to(bf)

  D, F, V = cfg.embed_dim, cfg.hidden_dim, cfg.vocab_size
  w = {"embed": normal(V, D)}
  norm_fill = 0.0 if cfg.family == "gemma3" else 1.0
  w["final_norm"] = torch.full((D,), norm_fill, dtype=bf, device=dev)
  if not cfg.tied_embedding:
    w["lm_head"] = normal(D, V)
  for i in range(cfg.num_layers):
    p = f"l{i}."
    w[p + "attn_norm"] = torch.full((D,), norm_fill, dtype=bf, device=dev)
    w[p + "mlp_norm"] = torch.full((D,), norm_fill, dtype=bf, device=dev)
    if cfg.family in ("qwen3", "gemma3"):
      w[p + "q_norm"] = torch.full((cfg.head_dim,), norm_fill, dtype=bf, device=dev)
      w[p + "k_norm"] = torch.full((cfg.head_dim,), norm_fill, dtype=bf, device=dev)
    if cfg.family == "gemma3":
      w[p + "post_attn_norm"] = torch.full((D,), norm_fill, dtype=bf, device=dev)
      w[p + "post_ffw_norm"] = torch.full((D,), norm_fill, dtype=bf, device=dev)
    w[p + "wq"] = normal(D, cfg.q_dim)
    w[p + "wk"] = normal(D, cfg.kv_dim)
    w[p + "wv"] = normal(D, cfg.kv_dim)
    w[p + "wo"] = normal(cfg.q_dim, D)
    if cfg.num_experts:
      E = cfg.num_experts
      w[p + "router"] = normal(D, E)
      w[p + "e_gate"] = normal(E, D, F)
      w[p + "e_up"] = normal(E, D, F)
      w[p + "e_down"] = normal(E, F, D)
    else:
      w[p + "w_gate"] = normal(D, F)
      w[p + "w_up"] = normal(D, F)
      w[p + "w_down"] = normal(F, D)
  for name in cfg.lora_names():
    K, N = w[name].shape
    w[name + ".lora_a"] = normal(K, cfg.lora_rank, s=0.02)
    w[name + ".lora_b"] = normal(cfg.lora_rank, N, s=lora_b_scale)
  return w


def from_reference_tree(cfg: ModelConfig, tree: dict) -> dict:
  """Maps arrays shaped like the reference's parameter tree (dot-joined paths) to flat names.

  llama3 / qwen3 (llama3/model.py:311-334, :461-487): attn.{q,k,v}_proj.w [D,H,dh],
  attn.o_proj.w [H,dh,D], mlp.{gate,up,down}_proj.kernel; LoRA w_lora_a/w_lora_b and
  kernel_lora_a/kernel_lora_b (tunix/models/llama3/mapping_sglang_jax.py:64-145).
  gemma3 (gemma3/model.py:527-565): attn.q_einsum.w [H,D,dh], attn.kv_einsum.w [2,K,D,dh],
  attn.attn_vec_einsum.w [H,dh,D]; its LoRA leaves (gemma3/params.py:301-318 and the merge at
  safetensors_saver.py:88-107): q_einsum.w_lora_a [D,r] / w_lora_b [r,H,dh]; kv_einsum.w_lora_a
  [D,r], shared by k and v, / w_lora_b [r,2,K,dh]; attn_vec_einsum.w_lora_a [H,dh,r] / w_lora_b
  [r,D]; mlp.*_proj.kernel_lora_a / kernel_lora_b.  MoE models carry LoRA on the attention
  projections only.
  """
  def arr(x):
    return x if isinstance(x, torch.Tensor) else torch.as_tensor(np.asarray(x))

  out = {"embed": arr(tree["embedder.input_embedding"])}
  fam = cfg.family
  nk = "scale" if fam == "gemma3" else "w"
  out["final_norm"] = arr(tree[f"final_norm.{nk}"])
  if "lm_head.w" in tree:
    out["lm_head"] = arr(tree["lm_head.w"])
  D = cfg.embed_dim
  for i in range(cfg.num_layers):
    s, p = f"layers.{i}.", f"l{i}."
    if fam == "gemma3":
      out[p + "attn_norm"] = arr(tree[s + "pre_attention_norm.scale"])
      out[p + "post_attn_norm"] = arr(tree[s + "post_attention_norm.scale"])
      out[p + "mlp_norm"] = arr(tree[s + "pre_ffw_norm.scale"])
      out[p + "post_ffw_norm"] = arr(tree[s + "post_ffw_norm.scale"])
      out[p + "q_norm"] = arr(tree[s + "attn._query_norm.scale"])
      out[p + "k_norm"] = arr(tree[s + "attn._key_norm.scale"])
      q = arr(tree[s + "attn.q_einsum.w"])                      # [H,D,dh]
      out[p + "wq"] = q.permute(1, 0, 2).reshape(D, -1)
      kv = arr(tree[s + "attn.kv_einsum.w"])                    # [2,K,D,dh]
      out[p + "wk"] = kv[0].permute(1, 0, 2).reshape(D, -1)
      out[p + "wv"] = kv[1].permute(1, 0, 2).reshape(D, -1)
      out[p + "wo"] = arr(tree[s + "attn.attn_vec_einsum.w"]).reshape(-1, D)
      r = cfg.lora_rank
      if s + "attn.q_einsum.w_lora_a" in tree:
        out[p + "wq.lora_a"] = arr(tree[s + "attn.q_einsum.w_lora_a"])
        out[p + "wq.lora_b"] = arr(tree[s + "attn.q_einsum.w_lora_b"]).reshape(r, -1)
      if s + "attn.kv_einsum.w_lora_a" in tree:
        a = arr(tree[s + "attn.kv_einsum.w_lora_a"])               # [D,r]: one A for k and v
        b = arr(tree[s + "attn.kv_einsum.w_lora_b"])               # [r,2,K,dh]
        out[p + "wk.lora_a"], out[p + "wv.lora_a"] = a, a.clone()
        out[p + "wk.lora_b"] = b[:, 0].reshape(r, -1)
        out[p + "wv.lora_b"] = b[:, 1].reshape(r, -1)
      if s + "attn.attn_vec_einsum.w_lora_a" in tree:
        out[p + "wo.lora_a"] = arr(tree[s + "attn.attn_vec_einsum.w_lora_a"]).reshape(-1, r)
        out[p + "wo.lora_b"] = arr(tree[s + "attn.attn_vec_einsum.w_lora_b"])
    else:
      out[p + "attn_norm"] = arr(tree[s + "input_layernorm.w"])
      out[p + "mlp_norm"] = arr(tree[s + "post_attention_layernorm.w"])
      if fam == "qwen3":
        out[p + "q_norm"] = arr(tree[s + "attn.q_norm.w"])
        out[p + "k_norm"] = arr(tree[s + "attn.k_norm.w"])
      for src, dst in (("q_proj", "wq"), ("k_proj", "wk"), ("v_proj", "wv")):
        out[p + dst] = arr(tree[s + f"attn.{src}.w"]).reshape(D, -1)
        if s + f"attn.{src}.w_lora_a" in tree:
          out[p + dst + ".lora_a"] = arr(tree[s + f"attn.{src}.w_lora_a"])
          out[p + dst + ".lora_b"] = arr(tree[s + f"attn.{src}.w_lora_b"]).reshape(cfg.lora_rank, -1)
      out[p + "wo"] = arr(tree[s + "attn.o_proj.w"]).reshape(-1, D)
      if s + "attn.o_proj.w_lora_a" in tree:
        out[p + "wo.lora_a"] = arr(tree[s + "attn.o_proj.w_lora_a"]).reshape(-1, cfg.lora_rank)
        out[p + "wo.lora_b"] = arr(tree[s + "attn.o_proj.w_lora_b"])
    if cfg.num_experts:
      out[p + "router"] = arr(tree[s + "mlp.router.kernel"])
      out[p + "e_gate"] = arr(tree[s + "mlp.gate_proj"])
      out[p + "e_up"] = arr(tree[s + "mlp.up_proj"])
      out[p + "e_down"] = arr(tree[s + "mlp.down_proj"])
    else:
      for src, dst in (("gate_proj", "w_gate"), ("up_proj", "w_up"), ("down_proj", "w_down")):
        out[p + dst] = arr(tree[s + f"mlp.{src}.kernel"])
        if s + f"mlp.{src}.kernel_lora_a" in tree:
          out[p + dst + ".lora_a"] = arr(tree[s + f"mlp.{src}.kernel_lora_a"])
          out[p + dst + ".lora_b"] = arr(tree[s + f"mlp.{src}.kernel_lora_b"])
  return out
