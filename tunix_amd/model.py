"""Device-resident QLoRA decoder: packed int4/NF4 weights + separate LoRA tensors, and the
kernel sequence of one forward pass over T tokens per row (T = 1: a decode step).

Mirrors the layer structure of tunix/models/llama3/model.py:546-564, qwen3/model.py:1161-1182
(+ MoELayer :787-832) and gemma3/model.py:875-898; every arithmetic step is a libtunix_hip.so
kernel.  LoRA A/B stay separate buffers so that `update_lora` can swap them between rollouts
(tunix/generate/sampler.py:333-352, tunix/rl/rollout/vanilla_rollout.py:92-121).
"""
from __future__ import annotations

import math

import numpy as np
import torch

from . import _lib as L
from . import ops
from .config import ModelConfig

_NORM = {"llama3": L.TNX_NORM_LLAMA, "qwen3": L.TNX_NORM_QWEN3, "gemma3": L.TNX_NORM_GEMMA3}
_MOE_PENDING = -1   # norm_after: the weighted combine of an MoE layer still awaits its sum
_ROPE = {"llama3": L.TNX_ROPE_LLAMA, "qwen3": L.TNX_ROPE_QWEN3, "gemma3": L.TNX_ROPE_GEMMA3}


def _pad32(r: int) -> int:
  return (r + 31) // 32 * 32 if r > 0 else 0


def rope_timescale(head_dim: int, theta: float) -> np.ndarray:
  """theta ** (2i / head_dim) in fp32, as apply_rope computes it (llama3/model.py:256-257)."""
  fraction = (np.float32(2.0) * np.arange(0, head_dim // 2, dtype=np.float32)
              / np.float32(head_dim)).astype(np.float32)
  return np.power(np.float32(theta), fraction).astype(np.float32)


class FusedLinear:
  """One quantised projection (possibly several reference linears sharing an input) with its
  LoRA tensors in kernel layout."""

  def __init__(self, cfg: ModelConfig, weights: dict, names: list[str], device,
               interleave2: bool = False):
    self.names = names
    self.K = weights[names[0]].shape[0]
    self.widths = [weights[n].shape[1] for n in names]
    self.N = sum(self.widths)
    self.interleave2 = interleave2
    self.group, self.qtype, self.int4_bound = cfg.group, cfg.qtype, cfg.int4_bound
    self.device = device
    self.codes = self.scales = None
    self.expanded = None   # optional second copy for calls with many rows (`expand`)
    self.load_base(weights)
    r = cfg.lora_rank
    self.has_lora = any((n + ".lora_a") in weights for n in names)
    self.rp = _pad32(r) if self.has_lora else 0
    self.r = r
    self.lora_scale = float(cfg.lora_alpha) / float(r) if self.has_lora else 0.0
    self.seg_end, self.seg_toff = [], []
    off = 0
    for i, wd in enumerate(self.widths):
      off += wd
      self.seg_end.append(off)
      self.seg_toff.append(i * self.rp)
    if self.has_lora:
      self.a_t = torch.zeros(len(names) * self.rp, self.K, dtype=torch.bfloat16, device=device)
      self.b_t = torch.zeros(self.N, self.rp, dtype=torch.bfloat16, device=device)
      self._row_perm = None
      if interleave2:
        c = torch.arange(self.N, device=device)
        half = self.N // 2
        h, cc = c // half, c % half
        self._row_perm = (cc // 16) * 32 + h * 16 + (cc % 16)
      self.load_lora(weights)

  def check_base(self, weights: dict):
    """Raises ValueError unless `weights` holds every member of this projection in the shape it was
    built with; touches nothing."""
    for n, wd in zip(self.names, self.widths):
      if n not in weights:
        raise ValueError(f"New state must have the same structure as the old state: {n} is missing")
      if tuple(weights[n].shape) != (self.K, wd):
        raise ValueError(f"New state must have the same shape as the old state: {n} {tuple(weights[n].shape)} "
                         f"vs {(self.K, wd)}")

  def check_lora(self, weights: dict):
    """Raises ValueError for an adapter leaf of this projection whose shape differs from the one
    it was built with, or whose partner leaf is missing; touches nothing."""
    if not self.has_lora:
      return
    for n, wd in zip(self.names, self.widths):
      a, b = weights.get(n + ".lora_a"), weights.get(n + ".lora_b")
      if a is None and b is None:
        continue
      if a is None or b is None:
        raise ValueError(f"New state must have the same structure as the old state: {n} has one LoRA leaf only")
      if tuple(a.shape) != (self.K, self.r) or tuple(b.shape) != (self.r, wd):
        raise ValueError(
            f"New state must have the same shape as the old state: {n} lora_a {tuple(a.shape)}"
            f" lora_b {tuple(b.shape)} vs {(self.K, self.r)} / {(self.r, wd)}")

  def load_base(self, weights: dict):
    """(Re-)quantises and packs the base kernels of every member from `weights` (all members of a
    fused projection must be present, with the shapes the linear was built with)."""
    self.check_base(weights)
    ws = []
    for n, wd in zip(self.names, self.widths):
      ws.append(weights[n].to(device=self.device, dtype=torch.bfloat16))
    w = torch.cat(ws, dim=1).contiguous() if len(ws) > 1 else ws[0].contiguous()
    codes, scales = ops.quantize_pack(w, self.group, self.qtype, self.interleave2, self.int4_bound)
    if self.codes is None:
      self.codes, self.scales = codes, scales
    else:   # in place: captured graphs and descriptors keep their pointers
      self.codes.copy_(codes)
      self.scales.copy_(scales)
      if self.expanded is not None:
        self.expanded.copy_(ops.qw_expand(self.codes, self.scales, self.K, self.N, self.group, self.qtype))

  def expanded_bytes(self) -> int:
    return int(L.lib().tnx_qw_expanded_bytes(self.K, self.N))

  def expand(self):
    """Keeps a second copy of the frozen weight, converted to bf16 in the many-row kernel's
    fragment order (2 bytes per weight): prefill and per-token-logps passes then load it instead
    of converting codes in their loop.  Decode steps never read it."""
    if self.expanded is None and self.wants_expansion():
      self.expanded = ops.qw_expand(self.codes, self.scales, self.K, self.N, self.group, self.qtype)

  def wants_expansion(self) -> bool:
    """From the copy the many-row kernel runs two work-groups per compute unit: 8-10 % over
    integer codes converted in the loop, 20-25 % over a table code book (NF4).  (The kernel
    addresses the copy with 32-bit offsets.)"""
    return self.expanded_bytes() < (1 << 31)

  def load_lora(self, weights: dict):
    """Copies lora_a [K,r] / lora_b [r,N_i] of every member into the kernel layout."""
    if not self.has_lora:
      return
    self.check_lora(weights)
    b_full = torch.zeros(self.N, self.rp, dtype=torch.bfloat16, device=self.b_t.device)
    off = 0
    for i, (n, wd) in enumerate(zip(self.names, self.widths)):
      a = weights.get(n + ".lora_a")
      if a is not None:
        b = weights[n + ".lora_b"]
        self.a_t[i * self.rp: i * self.rp + self.r].copy_(a.to(self.a_t.device, torch.bfloat16).t())
        b_full[off: off + wd, : self.r].copy_(b.to(self.b_t.device, torch.bfloat16).t())
      off += wd
    if self._row_perm is not None:
      self.b_t[self._row_perm] = b_full
    else:
      self.b_t.copy_(b_full)

  @property
  def t_cols(self) -> int:
    return len(self.names) * self.rp


class ExpertBank:
  """Per-expert QW weights of one MoE layer: fused gate|up (interleaved) and down."""

  def __init__(self, cfg: ModelConfig, weights: dict, prefix: str, device):
    g = weights[prefix + "e_gate"]
    E = g.shape[0]
    self.cfg, self.prefix, self.device = cfg, prefix, device
    self.E, self.D, self.F = E, g.shape[1], g.shape[2]
    cb, sb = ops.qw_sizes(self.D, 2 * self.F, cfg.group)
    self.gu_codes = torch.empty(E * cb // 4, dtype=torch.int32, device=device)
    self.gu_scales = torch.empty(E * sb // 2, dtype=torch.bfloat16, device=device)
    cb2, sb2 = ops.qw_sizes(self.F, self.D, cfg.group)
    self.dn_codes = torch.empty(E * cb2 // 4, dtype=torch.int32, device=device)
    self.dn_scales = torch.empty(E * sb2 // 2, dtype=torch.bfloat16, device=device)
    self.router_t = torch.empty(E, self.D, dtype=torch.bfloat16, device=device)
    self.load_base(weights)

  def check_base(self, weights: dict):
    """Raises ValueError unless `weights` holds the router and the three expert kernels in the
    shapes the bank was built with; touches nothing."""
    prefix, E = self.prefix, self.E
    for n, shape in ((prefix + "e_gate", (E, self.D, self.F)), (prefix + "e_up", (E, self.D, self.F)),
                     (prefix + "e_down", (E, self.F, self.D)), (prefix + "router", (self.D, E))):
      if n not in weights:
        raise ValueError(f"New state must have the same structure as the old state: {n} is missing")
      if tuple(weights[n].shape) != shape:
        raise ValueError(f"New state must have the same shape as the old state: {n} {tuple(weights[n].shape)} vs {shape}")

  def load_base(self, weights: dict):
    """(Re-)quantises the experts and copies the router from `weights`, in place."""
    self.check_base(weights)
    cfg, prefix, device, E = self.cfg, self.prefix, self.device, self.E
    g, u, d = weights[prefix + "e_gate"], weights[prefix + "e_up"], weights[prefix + "e_down"]
    cb, sb = ops.qw_sizes(self.D, 2 * self.F, cfg.group)
    cb2, sb2 = ops.qw_sizes(self.F, self.D, cfg.group)
    for e in range(E):
      w = torch.cat([g[e], u[e]], dim=1).to(device, torch.bfloat16).contiguous()
      c, s = ops.quantize_pack(w, cfg.group, cfg.qtype, True, cfg.int4_bound)
      self.gu_codes[e * cb // 4:(e + 1) * cb // 4].copy_(c)
      self.gu_scales[e * sb // 2:(e + 1) * sb // 2].copy_(s)
      c, s = ops.quantize_pack(d[e].to(device, torch.bfloat16).contiguous(), cfg.group, cfg.qtype, False,
                               cfg.int4_bound)
      self.dn_codes[e * cb2 // 4:(e + 1) * cb2 // 4].copy_(c)
      self.dn_scales[e * sb2 // 2:(e + 1) * sb2 // 2].copy_(s)
    self.router_t.copy_(weights[prefix + "router"].to(device, torch.bfloat16).t())


class QLoRAModel:
  """Packed weights of one model on one GPU."""

  def __init__(self, cfg: ModelConfig, weights: dict, device="cuda", expand_many_rows: bool | None = None):
    """expand_many_rows: keep the converted second copy of every dense quantised linear
    (`FusedLinear.expand`) for the calls with many rows.  None (default): when the copies take
    less than a quarter of the device memory that is free once the model is built."""
    L.lib()  # fail loudly when the HIP library is missing
    self.cfg = cfg
    self.device = torch.device(device)
    dev = self.device
    bf = torch.bfloat16
    self.embed = weights["embed"].to(dev, bf).contiguous()
    self.final_norm = weights["final_norm"].to(dev, bf).contiguous()
    self.head = None
    self.head_w = None
    if not cfg.tied_embedding:
      if cfg.quantize_head:
        self.head = FusedLinear(cfg, weights, ["lm_head"], dev)
      else:
        self.head_w = weights["lm_head"].to(dev, bf).t().contiguous()  # [V, D]
    self.layers = []
    for i in range(cfg.num_layers):
      p = f"l{i}."
      ly = {}
      ly["attn_norm"] = weights[p + "attn_norm"].to(dev, bf).contiguous()
      ly["mlp_norm"] = weights[p + "mlp_norm"].to(dev, bf).contiguous()
      for extra in ("q_norm", "k_norm", "post_attn_norm", "post_ffw_norm"):
        if p + extra in weights:
          ly[extra] = weights[p + extra].to(dev, bf).contiguous()
      ly["qkv"] = FusedLinear(cfg, weights, [p + "wq", p + "wk", p + "wv"], dev)
      ly["o"] = FusedLinear(cfg, weights, [p + "wo"], dev)
      if cfg.num_experts:
        ly["experts"] = ExpertBank(cfg, weights, p, dev)
      else:
        ly["gu"] = FusedLinear(cfg, weights, [p + "w_gate", p + "w_up"], dev, interleave2=True)
        ly["down"] = FusedLinear(cfg, weights, [p + "w_down"], dev)
      theta, sf = cfg.rope_params(i)
      ly["timescale"] = torch.from_numpy(rope_timescale(cfg.head_dim, theta)).to(dev)
      ly["rope_scale"] = sf
      self.layers.append(ly)
    torch.cuda.synchronize(dev)
    # a dense (unquantised or tied) head in the many-row kernel's fragment order, same purpose
    self.head_expanded = None
    dense_head = self.head_w if self.head_w is not None else (self.embed if self.head is None else None)
    head_need = 0
    if dense_head is not None and cfg.embed_dim % 128 == 0 and cfg.vocab_size % 16 == 0:
      head_need = int(L.lib().tnx_qw_expanded_bytes(cfg.embed_dim, cfg.vocab_size))
      if head_need >= (1 << 31):
        head_need = 0
    if expand_many_rows is None:
      need = head_need + sum(f.expanded_bytes() for f in self._linears() if f.wants_expansion())
      expand_many_rows = need <= torch.cuda.mem_get_info(dev)[0] // 4
    if expand_many_rows:
      for f in self._linears():
        f.expand()
      if head_need:
        self.head_expanded = ops.dense_expand(dense_head)
      torch.cuda.synchronize(dev)

  # weight sync: LoRA-only replacement (tunix/generate/sampler.py:333-352)
  def update_lora(self, new_lora: dict):
    expected = set()
    for n in self.cfg.lora_names():
      expected.add(n + ".lora_a")
      expected.add(n + ".lora_b")
    if set(new_lora) != expected:
      raise ValueError(
          "New state must have the same structure as the old state. "
          f"missing={sorted(expected - set(new_lora))} extra={sorted(set(new_lora) - expected)}")
    linears = self._linears()
    for f in linears:      # every shape is checked before the first copy: a rejected state changes nothing
      f.check_lora(new_lora)
    for f in linears:
      f.load_lora(new_lora)
    torch.cuda.synchronize(self.device)

  def _linears(self) -> list:
    out = [ly[key] for ly in self.layers for key in ("qkv", "o", "gu", "down") if key in ly]
    if self.head is not None:
      out.append(self.head)
    return out

  # full state replacement (tunix/generate/sampler.py:265-332; VanillaRollout.update_params,
  # tunix/rl/rollout/vanilla_rollout.py:92-121, merges a partial state into the old one first)
  def update_params(self, new_state: dict):
    """Replaces parameters by name.  A state holding only LoRA leaves (`*.lora_a` / `*.lora_b`)
    is the LoRA-only swap and must name every adapter (`update_lora`).  A state with base
    parameters replaces those -- embedding, norms, head, and linears, which are re-quantised and
    re-packed in place; the members of a fused projection (q|k|v, gate|up, an expert bank)
    come together -- and may carry LoRA leaves as well.  Shapes must match the old state's."""
    base = {k: v for k, v in new_state.items() if not k.endswith((".lora_a", ".lora_b"))}
    lora = {k: v for k, v in new_state.items() if k.endswith((".lora_a", ".lora_b"))}
    if not base:
      self.update_lora(lora)
      return
    dev, bf = self.device, torch.bfloat16
    known = {"embed", "final_norm"} | ({"lm_head"} if not self.cfg.tied_embedding else set())
    for i in range(self.cfg.num_layers):
      p = f"l{i}."
      known |= {p + n for n in ("attn_norm", "mlp_norm", "q_norm", "k_norm", "post_attn_norm", "post_ffw_norm",
                                "wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down", "router", "e_gate", "e_up",
                                "e_down")}
    extra = sorted(set(base) - known)
    if extra:
      raise ValueError(f"New state must have the same structure as the old state. extra={extra}")

    # First pass: every name, fused-member set and shape is checked and the work is only listed;
    # a state that is rejected leaves the model exactly as it was (the reference validates the
    # structure before it replaces anything, sampler.py:280-284, :322-325).
    copies, reloads = [], []

    def plan_copy(dst: torch.Tensor, name: str, transpose: bool = False):
      shape = tuple(base[name].shape)[::-1] if transpose else tuple(base[name].shape)
      if shape != tuple(dst.shape):
        raise ValueError(f"New state must have the same shape as the old state: {name} {tuple(base[name].shape)}")
      copies.append((dst, name, transpose))

    if "embed" in base:
      plan_copy(self.embed, "embed")
    if "final_norm" in base:
      plan_copy(self.final_norm, "final_norm")
    if "lm_head" in base:
      if self.head is not None:
        self.head.check_base(base)
        reloads.append(self.head)
      elif self.head_w is not None:
        plan_copy(self.head_w, "lm_head", transpose=True)
    for i, ly in enumerate(self.layers):
      p = f"l{i}."
      for n in ("attn_norm", "mlp_norm", "q_norm", "k_norm", "post_attn_norm", "post_ffw_norm"):
        if p + n in base:
          if n not in ly:
            raise ValueError(f"New state must have the same structure as the old state. extra={[p + n]}")
          plan_copy(ly[n], p + n)
      for key in ("qkv", "o", "gu", "down"):
        if key in ly and any(n in base for n in ly[key].names):
          ly[key].check_base(base)
          reloads.append(ly[key])
      if "experts" in ly and any(p + n in base for n in ("router", "e_gate", "e_up", "e_down")):
        ly["experts"].check_base(base)
        reloads.append(ly["experts"])
      elif "experts" not in ly and any(p + n in base for n in ("router", "e_gate", "e_up", "e_down")):
        raise ValueError(f"New state must have the same structure as the old state. extra={[p + 'e_gate']}")
    linears = self._linears()
    if lora:
      known_lora = {n + sfx for n in self.cfg.lora_names() for sfx in (".lora_a", ".lora_b")}
      extra = sorted(set(lora) - known_lora)
      if extra:
        raise ValueError(f"New state must have the same structure as the old state. extra={extra}")
      for f in linears:
        f.check_lora(lora)
    # Second pass: nothing below raises for a reason the first pass could have seen.
    for dst, name, transpose in copies:
      src = base[name].to(dev, bf)
      dst.copy_(src.t() if transpose else src)
    for obj in reloads:
      obj.load_base(base)
    if self.head_expanded is not None and any(n in ("embed", "lm_head") for _, n, _ in copies):
      src = self.head_w if self.head_w is not None else self.embed
      self.head_expanded.copy_(ops.dense_expand(src))
    if lora:
      for f in linears:
        f.load_lora(lora)
    torch.cuda.synchronize(self.device)

  def weight_bytes(self) -> dict:
    """Bytes one decode step reads: codes+scales, LoRA, head (algorithmic traffic)."""
    q = lora = 0
    for ly in self.layers:
      for key in ("qkv", "o", "gu", "down"):
        if key in ly:
          f = ly[key]
          q += f.codes.numel() * 4 + f.scales.numel() * 2
          if f.has_lora:
            lora += (f.K * f.r * len(f.names) + f.N * f.r) * 2
      if "experts" in ly:
        ex = ly["experts"]
        q += (ex.gu_codes.numel() + ex.dn_codes.numel()) * 4
        q += (ex.gu_scales.numel() + ex.dn_scales.numel()) * 2
    if self.head_w is not None:
      head = self.head_w.numel() * 2
    elif self.head is not None:
      head = self.head.codes.numel() * 4 + self.head.scales.numel() * 2
    else:
      head = self.embed.numel() * 2
    return {"quantized": q, "lora": lora, "head": head}


class Runner:
  """Workspaces + the kernel sequence for up to `max_rows` = B*T token rows.

  State tensors (token buffer, positions, KV cache, step counter) are owned by the caller and
  bound with `bind`; all kernels read the step / column from device memory so that a decode step
  can be captured once into a HIP graph and replayed.
  """

  def __init__(self, model: QLoRAModel, B: int, T: int, S: int, pad_id: int, kv_chunk=None,
               want_logits: bool = False, split_k_override: dict | None = None):
    cfg = model.cfg
    self.model, self.cfg, self.B, self.T, self.S = model, cfg, B, T, S
    self.pad_id = int(pad_id)
    dev = model.device
    M = B * T
    self.M = M
    bf = torch.bfloat16
    D, F = cfg.embed_dim, cfg.hidden_dim
    nqkv = cfg.q_dim + 2 * cfg.kv_dim
    rp = _pad32(cfg.lora_rank)
    self.h = torch.empty(M, D, dtype=bf, device=dev)
    self.xn = torch.empty(M, D, dtype=bf, device=dev)
    self.tmp = torch.empty(M, D, dtype=bf, device=dev)
    self.qkv = torch.empty(M, nqkv, dtype=bf, device=dev)
    self.q = torch.empty(M, cfg.q_dim, dtype=bf, device=dev)
    self.attn = torch.empty(M, cfg.q_dim, dtype=bf, device=dev)
    self.t = torch.zeros(M, max(3 * rp, 32), dtype=bf, device=dev)
    if cfg.num_experts:
      k = cfg.num_experts_per_tok
      self.scores = torch.empty(M, cfg.num_experts, dtype=bf, device=dev)
      self.topk_w = torch.empty(M, k, dtype=bf, device=dev)
      self.topk_id = torch.empty(M, k, dtype=torch.int32, device=dev)
      self.counts = torch.empty(cfg.num_experts, dtype=torch.int32, device=dev)
      self.offsets = torch.empty(cfg.num_experts + 1, dtype=torch.int32, device=dev)
      self.sorted_route = torch.empty(M * k, dtype=torch.int32, device=dev)
      self.act = torch.empty(M * k, F, dtype=bf, device=dev)
      self.y_route = torch.empty(M * k, D, dtype=bf, device=dev)
    else:
      self.act = torch.empty(M, F, dtype=bf, device=dev)
    # {"wo": 4} pins the k split of the linears of that name (a sweep's handle; empty in normal use)
    self.split_k_override = dict(split_k_override or {})
    self.fuse_rope = True   # decode: RoPE + cache write inside the attention kernel where it can
    self.rope_sin = torch.empty(B, max(cfg.head_dim // 2, 1), dtype=torch.float32, device=dev)
    self.rope_cos = torch.empty_like(self.rope_sin)
    self.next_tpart = None
    if M <= 1024 and not cfg.num_experts and model.layers and "gu" in model.layers[0]:
      n_planes = math.ceil(M / 128) * math.ceil(model.layers[0]["gu"].N / 128)
      self.next_tpart = torch.empty(n_planes * 8192, dtype=torch.float32, device=dev)
    need = 1
    for ly in model.layers:
      for key in ("qkv", "o", "gu", "down"):
        if key in ly:
          sk = self._split_k(ly[key], M)
          if sk > 1:
            need = max(need, sk * M * ly[key].N)
    self.splitk_ws = torch.empty(need, dtype=torch.float32, device=dev)
    if kv_chunk is None:
      # decode: one wave streams the keys of one (row, kv head); the key range is split only as
      # far as needed to put about a thousand waves (one per SIMD) on the device
      kv_chunk = 0
      waves = B * cfg.num_kv_heads
      if T == 1 and waves < 1024 and S > 64:
        n_chunks = min(math.ceil(1024 / waves), S // 32)
        kv_chunk = max(32, math.ceil(S / n_chunks / 32) * 32)
        if kv_chunk >= S:
          kv_chunk = 0
    self.kv_chunk = kv_chunk
    nb = ops.attn_ws_bytes(B, T, S, cfg.num_heads, cfg.head_dim, kv_chunk)
    self.attn_ws = torch.empty(max(nb // 4, 1), dtype=torch.float32, device=dev)
    self.zero = torch.zeros(1, dtype=torch.int32, device=dev)
    # head
    self.nvb = ops.lmhead_nblocks(cfg.vocab_size)
    self.head_rows = B
    self.xlast = torch.empty(B, D, dtype=bf, device=dev)
    self.part = torch.empty(B * self.nvb * 4, dtype=torch.float32, device=dev)
    self.best_id = torch.empty(B, dtype=torch.int32, device=dev)
    self.best_logp = torch.empty(B, dtype=torch.float32, device=dev)
    self.logits = (torch.empty(B, cfg.vocab_size, dtype=torch.float32, device=dev)
                   if want_logits else None)

  # ---- building blocks -----------------------------------------------------------------------
  def _split_k(self, f: FusedLinear, M: int) -> int:
    if f.names[0] in self.split_k_override:
      return self.split_k_override[f.names[0]]
    key = f.names[0].split(".")[-1]
    if key in self.split_k_override:
      return self.split_k_override[key]
    blocks = math.ceil(f.N / 128) * math.ceil(M / 128)
    ktiles = f.K // 128
    if blocks >= 200 or M > 128:
      return 1
    split = int(max(1, min(8, ktiles, 256 // blocks)))
    # A gate|up linear that runs unsplit applies its activation itself and can leave the next
    # linear's adapter down-projection behind: two launches fewer (finishing pass, LoRA down),
    # ≈ 9 us, against ≈ 1.1 us per k-tile the unsplit work-groups run longer.
    if f.interleave2 and ktiles - math.ceil(ktiles / split) <= 7:
      return 1
    return split

  def linear(self, f: FusedLinear, x, y, M, epilogue=L.TNX_EPI_STORE, residual=None, defer=False,
             next_f: FusedLinear | None = None, t_ready: bool = False):
    """Runs one fused linear.  With defer=True a split-k linear skips its finishing pass and
    returns split_k (> 1): the caller hands the partial planes in self.splitk_ws to the kernel
    that consumes them (`norm_after` for a RESIDUAL linear of model width, the rope / cache
    write for a plain STORE); otherwise returns 1 with y complete."""
    if f.has_lora and not t_ready:
      ops.lora_down(x, f.a_t, self.t, M=M)
    split = self._split_k(f, M)
    # a gate|up linear can leave the down-projection of the next linear's adapter behind
    # (`fuses_next`): then that linear is called with t_ready=True
    kw = {}
    if next_f is not None and self.fuses_next(f, next_f, M, epilogue):
      kw = dict(next_a_t=next_f.a_t, next_rank=next_f.rp, next_tpart=self.next_tpart)
    d = ops.make_qlinear_desc(
        M=M, K=f.K, N=f.N, group=f.group, qtype=f.qtype, x=x, codes=f.codes, scales=f.scales, y=y,
        epilogue=epilogue, residual=residual, lora_rank=f.rp,
        lora_nseg=(-1 if f.interleave2 else len(f.names)), lora_seg_end=f.seg_end,
        lora_seg_toff=f.seg_toff, t=self.t if f.has_lora else None, t_ld=self.t.shape[1],
        lora_b=f.b_t if f.has_lora else None, lora_scale=f.lora_scale, split_k=split,
        ws=self.splitk_ws if split > 1 else None, w_expanded=f.expanded, **kw)
    if kw:
      ops.qlinear(d)
      ops.lora_reduce(self.next_tpart, M, math.ceil(f.N / 128), next_f.rp, self.t)
      return 1
    deferred = defer and split > 1 and (
        epilogue == L.TNX_EPI_STORE
        or (epilogue == L.TNX_EPI_RESIDUAL and f.N == self.cfg.embed_dim and f.N % 8 == 0))
    ops.qlinear(d, finish=not deferred)
    return split if deferred else 1

  def fuses_next(self, f: FusedLinear, next_f: FusedLinear, M: int, epilogue: int) -> bool:
    return (next_f.has_lora and next_f.rp <= 64 and M <= 1024 and self._split_k(f, M) == 1
            and epilogue in (L.TNX_EPI_SILU_MUL, L.TNX_EPI_GELU_MUL) and (f.N // 2) % 8 == 0
            and self.next_tpart is not None)

  def norm_after(self, pending: int, w, M):
    """self.xn = norm(self.h) -- or, with the partial planes of a deferred linear pending,
    self.h += bf16(sum of planes) first (the linear's residual epilogue) in the same kernel."""
    cfg = self.cfg
    flavor = _NORM[cfg.family]
    if pending == _MOE_PENDING:   # h += the weighted combine of the routed rows, in the same kernel
      ops.rmsnorm_moe_combine(self.y_route, self.topk_w, cfg.num_experts_per_tok, w, self.xn, cfg.norm_eps,
                              flavor, M, cfg.embed_dim, res_pre=self.h, h_out=self.h)
    elif pending > 1:
      ops.rmsnorm_splitk(self.splitk_ws, pending, w, self.xn, cfg.norm_eps, flavor, M, cfg.embed_dim,
                         res_pre=self.h, h_out=self.h)
    else:
      ops.rmsnorm(self.h, w, self.xn, cfg.norm_eps, flavor, M=M)

  def norm_pair(self, pending: int, w, w2, M):
    """self.h += norm(self.tmp) . w (self.tmp = a linear's output, or its `pending` partial planes);
    self.xn = norm(self.h) . w2 -- Gemma-3's post-norm + residual + next pre-norm in one launch."""
    cfg = self.cfg
    kw = dict(ws=self.splitk_ws, split_k=pending) if pending > 1 else dict(x=self.tmp)
    ops.rmsnorm_pair(w, self.h, w2, self.xn, cfg.norm_eps, _NORM[cfg.family], M, cfg.embed_dim,
                     res_post=self.h, **kw)

  def forward_hidden(self, tokens, positions, col_ptr, kcache, vcache, B=None, T=None, segment_ids=None):
    """Runs all layers for tokens[b, col .. col+T) of each row; leaves the final-normed hidden
    state in self.xn[:B*T].  kcache/vcache: lists of [B,Hkv,S,dh] tensors.  segment_ids (int32,
    the shape of `tokens`): a packed batch, attention stays inside a token's own segment."""
    if segment_ids is not None and (tuple(segment_ids.shape) != tuple(tokens.shape)
                                    or segment_ids.dtype != torch.int32 or not segment_ids.is_contiguous()):
      raise ValueError("segment_ids must be a contiguous int32 tensor of the token buffer's shape")
    cfg, m = self.cfg, self.model
    B = self.B if B is None else B
    T = self.T if T is None else T
    M = B * T
    flavor = _NORM[cfg.family]
    emb_scale = math.sqrt(cfg.embed_dim) if cfg.family == "gemma3" else 1.0
    ops.embed(m.embed, tokens, col_ptr, B, T, emb_scale, self.h)
    pending = 1  # split count of a down-projection whose partial planes still await their sum
    if (T == 1 and self.fuse_rope and m.layers and "q_norm" not in m.layers[0]
        and _ROPE[cfg.family] == L.TNX_ROPE_LLAMA and cfg.head_dim == 128):
      # one table of this step's sines / cosines for all layers (they share theta)
      ops.rope_table(positions, col_ptr, B, m.layers[0]["timescale"], cfg.head_dim, self.rope_sin, self.rope_cos)
    xn_ready = False   # gemma3: the block before has already normed the residual stream into self.xn
    for i, ly in enumerate(m.layers):
      if not xn_ready:
        self.norm_after(pending, ly["attn_norm"], M)
      pending, xn_ready = 1, False
      qkv_split = self.linear(ly["qkv"], self.xn, self.qkv, M, defer=True)
      # decode step of a model without q/k norm and with the Llama rotation: the attention kernel
      # rotates q / k and writes the cache itself, and the stand-alone launch is dropped
      fuse_rope = (T == 1 and "q_norm" not in ly and _ROPE[cfg.family] == L.TNX_ROPE_LLAMA
                   and cfg.head_dim == 128 and self.fuse_rope)
      if not fuse_rope:
        rd = L.RopeDesc()
        rd.B, rd.T, rd.S = B, T, self.S
        rd.Hq, rd.Hkv, rd.dh = cfg.num_heads, cfg.num_kv_heads, cfg.head_dim
        rd.rope_flavor, rd.rope_scale = _ROPE[cfg.family], ly["rope_scale"]
        rd.timescale = ly["timescale"].data_ptr()
        if "q_norm" in ly:
          rd.qk_norm = flavor
          rd.norm_eps = cfg.norm_eps if cfg.family == "qwen3" else 1e-6
          rd.q_norm_w, rd.k_norm_w = ly["q_norm"].data_ptr(), ly["k_norm"].data_ptr()
        else:
          rd.qk_norm = -1
        rd.q_prescale = cfg.query_pre_attn_scalar if cfg.family == "gemma3" else 0.0
        rd.qkv, rd.positions, rd.pos_ld = self.qkv.data_ptr(), positions.data_ptr(), positions.shape[1]
        if qkv_split > 1:  # the rope kernel sums the partial planes itself
          rd.qkv_ws, rd.split_k = self.splitk_ws.data_ptr(), qkv_split
        rd.col_ptr = col_ptr.data_ptr()
        rd.q_out, rd.kcache, rd.vcache = self.q.data_ptr(), kcache[i].data_ptr(), vcache[i].data_ptr()
        ops.rope_kvwrite(rd)
      ad = L.AttnDesc()
      ad.B, ad.T, ad.S = B, T, self.S
      ad.Hq, ad.Hkv, ad.dh = cfg.num_heads, cfg.num_kv_heads, cfg.head_dim
      ad.scale = 0.0 if cfg.family == "gemma3" else cfg.head_dim ** -0.5
      ad.window = cfg.sliding_window if cfg.is_local_layer(i) else 0
      ad.pad_id = self.pad_id
      ad.q, ad.kcache, ad.vcache = self.q.data_ptr(), kcache[i].data_ptr(), vcache[i].data_ptr()
      ad.tokens, ad.tok_ld, ad.col_ptr = tokens.data_ptr(), tokens.shape[1], col_ptr.data_ptr()
      ad.kv_chunk = self.kv_chunk if T == 1 else 0
      if segment_ids is not None:
        ad.segment_ids = segment_ids.data_ptr()
      ad.ws, ad.out = self.attn_ws.data_ptr(), self.attn.data_ptr()
      if fuse_rope:
        if qkv_split > 1:
          ad.qkv_ws, ad.qkv_split = self.splitk_ws.data_ptr(), qkv_split
        else:
          ad.qkv = self.qkv.data_ptr()
        ad.rope_sin, ad.rope_cos = self.rope_sin.data_ptr(), self.rope_cos.data_ptr()
      ops.gqa_attn(ad)
      if cfg.family == "gemma3":
        # h += post_attn_norm(o_proj); xn = mlp_norm(h): one launch, which also sums the
        # projection's partial planes when it ran split
        po = self.linear(ly["o"], self.attn, self.tmp, M, defer=True)
        self.norm_pair(po, ly["post_attn_norm"], ly["mlp_norm"], M)
      else:
        po = self.linear(ly["o"], self.attn, self.h, M, epilogue=L.TNX_EPI_RESIDUAL, residual=self.h,
                         defer=True)
        self.norm_after(po, ly["mlp_norm"], M)
      if cfg.num_experts:
        pending = self._moe(ly["experts"], M)
      elif cfg.family == "gemma3":
        fused = self.fuses_next(ly["gu"], ly["down"], M, L.TNX_EPI_GELU_MUL)
        self.linear(ly["gu"], self.xn, self.act, M, epilogue=L.TNX_EPI_GELU_MUL, next_f=ly["down"])
        pd = self.linear(ly["down"], self.act, self.tmp, M, t_ready=fused, defer=True)
        # h += post_ffw_norm(down_proj); xn = the next block's attn_norm (or the final norm) of h
        nxt = m.layers[i + 1]["attn_norm"] if i + 1 < len(m.layers) else m.final_norm
        self.norm_pair(pd, ly["post_ffw_norm"], nxt, M)
        xn_ready = True
      else:
        fused = self.fuses_next(ly["gu"], ly["down"], M, L.TNX_EPI_SILU_MUL)
        self.linear(ly["gu"], self.xn, self.act, M, epilogue=L.TNX_EPI_SILU_MUL, next_f=ly["down"])
        pending = self.linear(ly["down"], self.act, self.h, M, epilogue=L.TNX_EPI_RESIDUAL,
                              residual=self.h, defer=True, t_ready=fused)
    if not xn_ready:
      self.norm_after(pending, m.final_norm, M)
    return self.xn

  def _moe(self, ex: ExpertBank, M: int) -> int:
    cfg = self.cfg
    k, E = cfg.num_experts_per_tok, cfg.num_experts
    ops.lora_down(self.xn, ex.router_t, self.scores, M=M)          # dense bf16 router
    ops.moe_route_topk(self.scores[:M], k, self.topk_w, self.topk_id)
    ops.moe_sort_routes(self.topk_id[:M], E, self.counts, self.offsets, self.sorted_route)
    d = L.MoeGmmDesc()
    d.n_routes, d.E, d.k, d.K, d.N = M * k, E, k, ex.D, 2 * ex.F
    d.group, d.qtype = cfg.group, cfg.qtype
    d.x, d.x_div = self.xn.data_ptr(), k
    d.codes, d.scales = ex.gu_codes.data_ptr(), ex.gu_scales.data_ptr()
    d.offsets, d.sorted_route = self.offsets.data_ptr(), self.sorted_route.data_ptr()
    d.epilogue, d.y = L.TNX_EPI_SILU_MUL, self.act.data_ptr()
    ops.moe_gmm(d)
    d2 = L.MoeGmmDesc()
    d2.n_routes, d2.E, d2.k, d2.K, d2.N = M * k, E, k, ex.F, ex.D
    d2.group, d2.qtype = cfg.group, cfg.qtype
    d2.x, d2.x_div = self.act.data_ptr(), 1
    d2.codes, d2.scales = ex.dn_codes.data_ptr(), ex.dn_scales.data_ptr()
    d2.offsets, d2.sorted_route = self.offsets.data_ptr(), self.sorted_route.data_ptr()
    d2.epilogue, d2.y = L.TNX_EPI_STORE, self.y_route.data_ptr()
    ops.moe_gmm(d2)
    if cfg.embed_dim % 8 == 0:   # the next norm adds the weighted combine to the residual stream
      return _MOE_PENDING
    ops.moe_combine(self.y_route, self.topk_w, M, k, cfg.embed_dim, self.h, self.h)
    return 1

  def head_desc(self, x, rows, part, temperature=1.0, targets=None, best_id=None, best_logp=None,
                target_logp=None, lse=None, logits_out=None, forbidden=None, entropy=None,
                part_entropy=None, draw=None, logits_fp32=False) -> L.LmHeadDesc:
    cfg, m = self.cfg, self.model
    d = L.LmHeadDesc()
    d.M, d.D, d.V = rows, cfg.embed_dim, cfg.vocab_size
    d.x = x.data_ptr()
    if m.head is not None:
      f = m.head
      d.codes, d.scales, d.group, d.qtype = f.codes.data_ptr(), f.scales.data_ptr(), f.group, f.qtype
      if f.expanded is not None:
        d.w_expanded = f.expanded.data_ptr()
      if f.has_lora:
        d.lora_rank, d.t, d.t_ld = f.rp, self.t.data_ptr(), self.t.shape[1]
        d.lora_b, d.lora_scale = f.b_t.data_ptr(), f.lora_scale
    else:
      d.w_bf16 = (m.head_w if m.head_w is not None else m.embed).data_ptr()
      if m.head_expanded is not None:
        d.w_expanded = m.head_expanded.data_ptr()
    d.temperature = float(temperature)
    d.logits_fp32 = 1 if logits_fp32 else 0
    if forbidden is not None:
      d.forbidden, d.n_forbidden = forbidden.data_ptr(), forbidden.numel()
    for name, tns in (("targets", targets), ("best_id", best_id), ("best_logp", best_logp),
                      ("target_logp", target_logp), ("lse", lse), ("logits_out", logits_out),
                      ("entropy", entropy), ("part_entropy", part_entropy)):
      if tns is not None:
        setattr(d, name, tns.data_ptr())
    d.part = part.data_ptr()
    if draw is not None:  # whole-vocabulary categorical draw inside the head
      d.part_draw = draw["part"].data_ptr()
      d.draw_key0, d.draw_key1 = int(draw["key"][0]), int(draw["key"][1])
      d.draw_rng_variant, d.draw_step_ptr = int(draw["variant"]), draw["step"].data_ptr()
      d.draw_id = draw["ids"].data_ptr()
      if draw.get("logp") is not None:
        d.draw_logp = draw["logp"].data_ptr()
    return d

  def run_head(self, x, rows, **kw):
    m = self.model
    if m.head is not None and m.head.has_lora:
      ops.lora_down(x, m.head.a_t, self.t, M=rows)
    ops.lmhead(self.head_desc(x, rows, self.part, **kw))
