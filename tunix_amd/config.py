"""Model descriptions for the decode path: the three families the sampler runs
(tunix/models/llama3/model.py:85-187, qwen3/model.py ModelConfig, gemma3/model.py:93-300)
plus the qwix-style QLoRA settings (tunix/cli/utils/model.py:31-77).
"""
from __future__ import annotations

import dataclasses

Q_INT4, Q_NF4 = 0, 1
QTYPE_BY_NAME = {"int4": Q_INT4, "nf4": Q_NF4}

# 5 local sliding-window layers, then 1 global (tunix/models/gemma3/model.py:441-448)
GEMMA3_PATTERN_LEN = 6

ATTN_LINEARS = ("wq", "wk", "wv", "wo")
MLP_LINEARS = ("w_gate", "w_up", "w_down")


@dataclasses.dataclass
class ModelConfig:
  family: str                      # 'llama3' | 'qwen3' | 'gemma3'
  num_layers: int
  vocab_size: int
  embed_dim: int
  hidden_dim: int                  # dense MLP width, or per-expert width for MoE
  num_heads: int
  num_kv_heads: int
  head_dim: int
  norm_eps: float = 1e-6
  # RoPE base actually used.  Llama3 and Qwen3 attention call apply_rope without rope_theta
  # (llama3/model.py:356-365, qwen3/model.py:545-554), so the default 1e6 applies whatever the
  # checkpoint config says.
  rope_theta: float = 1_000_000.0
  tied_embedding: bool = False
  # quantisation of the linears (None: dense bf16, not built)
  qtype: int = Q_INT4
  group: int = 64
  int4_bound: float = 7.0          # int4 scale = group absmax / this bound (codes clamp to [-8, 7])
  quantize_head: bool = False      # lm_head stays bf16 unless set (module_path never matches it)
  # LoRA
  lora_rank: int = 0
  lora_alpha: float = 0.0
  lora_targets: tuple = ATTN_LINEARS + MLP_LINEARS
  head_lora: bool = False
  # MoE (qwen3)
  num_experts: int = 0
  num_experts_per_tok: int = 0
  # gemma3
  sliding_window: int = 0
  local_base_frequency: float = 10_000.0
  global_base_frequency: float = 1_000_000.0
  local_scale_factor: float = 1.0
  global_scale_factor: float = 1.0
  query_pre_attn_scalar: float = 0.0

  def __post_init__(self):
    if self.family not in ("llama3", "qwen3", "gemma3"):
      raise ValueError(f"unknown model family {self.family!r}")
    if self.family == "gemma3" and self.query_pre_attn_scalar == 0.0:
      self.query_pre_attn_scalar = self.head_dim ** -0.5
    if self.num_heads % self.num_kv_heads:
      raise ValueError("num_heads must be a multiple of num_kv_heads")

  # ---- helpers shared by the engine and by checkers ----------------------------------------
  def is_local_layer(self, i: int) -> bool:
    return self.family == "gemma3" and (i % GEMMA3_PATTERN_LEN) != GEMMA3_PATTERN_LEN - 1

  def rope_params(self, i: int) -> tuple[float, float]:
    """(base frequency, scale factor) of layer i (gemma3/model.py:838-846)."""
    if self.family != "gemma3":
      return float(self.rope_theta), 1.0
    if self.is_local_layer(i):
      return float(self.local_base_frequency), float(self.local_scale_factor)
    return float(self.global_base_frequency), float(self.global_scale_factor)

  def layer_linear_names(self, i: int) -> list[str]:
    p = f"l{i}."
    names = [p + n for n in ATTN_LINEARS]
    if self.num_experts:
      names += [p + "e_gate", p + "e_up", p + "e_down"]
    else:
      names += [p + n for n in MLP_LINEARS]
    return names

  def quantized_names(self) -> list[str]:
    names = []
    for i in range(self.num_layers):
      names += self.layer_linear_names(i)
    if self.quantize_head and not self.tied_embedding:
      names.append("lm_head")
    return names

  def lora_names(self) -> list[str]:
    if self.lora_rank <= 0:
      return []
    names = [f"l{i}.{n}" for i in range(self.num_layers) for n in self.lora_targets]
    if self.head_lora:
      names.append("lm_head")
    return names

  @property
  def q_dim(self) -> int:
    return self.num_heads * self.head_dim

  @property
  def kv_dim(self) -> int:
    return self.num_kv_heads * self.head_dim


# ---- the shapes the headline metric and the parity cases are quoted on ------------------------
def tiny_qwen3(**kw) -> ModelConfig:
  """2-layer Qwen3-style decoder: D512, 8q/2kv, dh64, MLP 1536, V32000, int4 g64, LoRA r8."""
  d = dict(family="qwen3", num_layers=2, vocab_size=32000, embed_dim=512, hidden_dim=1536,
           num_heads=8, num_kv_heads=2, head_dim=64, norm_eps=1e-6, qtype=Q_INT4, group=64,
           lora_rank=8, lora_alpha=8.0)
  d.update(kw)
  return ModelConfig(**d)


def gemma3_1b(**kw) -> ModelConfig:
  """Gemma3-1B shape (gemma3/model.py:158-174): int4 g128, LoRA r16, tied embeddings."""
  d = dict(family="gemma3", num_layers=26, vocab_size=262144, embed_dim=1152, hidden_dim=6912,
           num_heads=4, num_kv_heads=1, head_dim=256, norm_eps=1e-6, tied_embedding=True,
           qtype=Q_INT4, group=128, lora_rank=16, lora_alpha=16.0, sliding_window=512,
           local_base_frequency=10_000.0, global_base_frequency=1_000_000.0)
  d.update(kw)
  return ModelConfig(**d)


def llama31_8b(**kw) -> ModelConfig:
  """Llama-3.1-8B shape (llama3/model.py:143-155): NF4 g64 with bf16 scales, LoRA r64."""
  d = dict(family="llama3", num_layers=32, vocab_size=128256, embed_dim=4096, hidden_dim=14336,
           num_heads=32, num_kv_heads=8, head_dim=128, norm_eps=1e-5, qtype=Q_NF4, group=64,
           lora_rank=64, lora_alpha=64.0)
  d.update(kw)
  return ModelConfig(**d)


def qwen3_30b_a3b(**kw) -> ModelConfig:
  """Qwen3-30B-A3B shape: 128 experts top-8, expert MLP 768, int4 g128, LoRA r16 on attention."""
  d = dict(family="qwen3", num_layers=48, vocab_size=151936, embed_dim=2048, hidden_dim=768,
           num_heads=32, num_kv_heads=4, head_dim=128, norm_eps=1e-6, qtype=Q_INT4, group=128,
           lora_rank=16, lora_alpha=16.0, lora_targets=ATTN_LINEARS, num_experts=128,
           num_experts_per_tok=8)
  d.update(kw)
  return ModelConfig(**d)
