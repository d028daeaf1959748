"""Pins WHERE the oracle's bf16 flow rounds.

oracle/model_ref.py keeps fp32 tensors and calls r() wherever the reference's dtype flow produces
a bf16 value.  A misplaced r() would go unnoticed by the fp32-mode checks against transformers, so
every rounding site is checked here by a second mechanism: the reference's formula is written
out again with REAL torch.bfloat16 / float32 tensors, one torch op per jnp op of the cited
source lines, applying jax's promotion rules (bf16 op bf16 -> bf16, bf16 op f32 -> f32, a python
scalar takes the array's dtype, jnp.mean / jnp.sum of a 16-bit float accumulate in fp32 and cast
back).  There the rounding is done by the dtype of each result, not by a call someone placed.
The two must agree bit for bit.  Each case also shows that it has teeth: a variant with one
rounding moved or dropped gives a different result on the same inputs.
"""
import numpy as np
import pytest
import torch

from oracle import model_ref as MR
from oracle import quant_ref as Q

BF, F32 = torch.bfloat16, torch.float32


def _model(family, eps=1e-6):
  from tunix_amd import config
  m = MR.RefModel.__new__(MR.RefModel)
  m.cfg = {"llama3": config.llama31_8b, "qwen3": config.tiny_qwen3, "gemma3": config.gemma3_1b}[family](num_layers=1)
  m.cfg.norm_eps = eps
  m.bf16, m.acc, m.gemma_score_softmax = True, torch.float64, True
  return m


def _rand_bf(shape, seed, scale=1.0, shift=0.0):
  g = torch.Generator().manual_seed(seed)
  return (torch.randn(*shape, generator=g) * scale + shift).to(BF)


def test_llama_rmsnorm_rounds_the_product_then_divides_in_fp32():
  """llama3/model.py:290-297: rms from fp32 squares; `self.w * x` is bf16 * bf16 (one rounding),
  `/ rms` promotes to fp32, astype rounds once more."""
  x, w = _rand_bf((6, 256), 1, 3.0), _rand_bf((256,), 2, 0.3, 1.0)
  rms = torch.sqrt(torch.mean(x.to(F32) ** 2, dim=-1, keepdim=True) + 1e-5)
  typed = ((w * x).to(F32) / rms).to(BF)
  m = _model("llama3", 1e-5)
  got = m.rmsnorm(x.float(), w.float(), flavor="llama3")
  assert torch.equal(got, typed.float())
  unrounded_product = Q.rb(w.float() * x.float() / rms)                  # the all-fp32 norm
  assert not torch.equal(got, unrounded_product)
  assert (got != unrounded_product).float().mean() > 0.02               # a known share of last-bit flips


def test_qwen3_rmsnorm_is_fp32_until_the_final_cast():
  """qwen3/model.py:450-456: x and w are cast to fp32 first; one rounding at the end."""
  x, w = _rand_bf((6, 256), 3, 3.0), _rand_bf((256,), 4, 0.3, 1.0)
  x32 = x.to(F32)
  rms = torch.sqrt(torch.mean(x32 ** 2, dim=-1, keepdim=True) + 1e-6)
  typed = (w.to(F32) * (x32 / rms)).to(BF)
  got = _model("qwen3").rmsnorm(x.float(), w.float(), flavor="qwen3")
  assert torch.equal(got, typed.float())
  llama_style = _model("llama3", 1e-6).rmsnorm(x.float(), w.float(), flavor="llama3")
  assert not torch.equal(got, llama_style)


def test_gemma3_rmsnorm_rounds_every_step():
  """gemma3/model.py:940-950 on a bf16 x: square (bf16), mean (fp32 accumulation, bf16 result),
  + 1e-6 (bf16), rsqrt (bf16), x * . (bf16), 1 + scale (bf16), product (bf16)."""
  x, sc = _rand_bf((6, 256), 5, 3.0), _rand_bf((256,), 6, 0.2)
  var = torch.mean(torch.square(x).to(F32), dim=-1, keepdim=True).to(BF)
  normed = x * torch.rsqrt((var + 1e-6).to(F32)).to(BF)
  typed = normed * (1 + sc)
  assert typed.dtype == BF and var.dtype == BF
  got = _model("gemma3").rmsnorm(x.float(), sc.float(), flavor="gemma3")
  assert torch.equal(got, typed.float())
  x32 = x.float()
  fp32_norm = Q.rb(x32 * torch.rsqrt((x32 * x32).mean(-1, keepdim=True) + 1e-6) * (1 + sc.float()))
  assert (got != fp32_norm).float().mean() > 0.05


@pytest.mark.parametrize("family", ["llama3", "qwen3", "gemma3"])
def test_rope_rounding_sites(family):
  """llama3/model.py:249-270 and gemma3/model.py:402-430: sin / cos stay fp32, bf16 * f32 -> f32,
  one rounding in astype.  qwen3/model.py:404-425: sin / cos are cast to bf16 first, so every
  product and the difference / sum are bf16 operations."""
  B, T, H, dh, theta = 2, 5, 3, 64, 1_000_000.0
  x = _rand_bf((B, T, H, dh), 7, 2.0)
  pos = torch.tensor([[0, 1, 2, 3, 4], [7, 30, 500, 1023, 4095]])
  ts = torch.from_numpy(MR.RefModel.timescale(dh, theta))
  ang = pos.to(F32)[..., None] / ts[None, None, :]
  sf = 1.0
  if family == "gemma3":
    sf = 8.0
    ang = ang / sf
  ang = ang[..., None, :]
  sin, cos = torch.sin(ang), torch.cos(ang)
  x1, x2 = x[..., : dh // 2], x[..., dh // 2:]
  if family == "qwen3":
    sin, cos = sin.to(BF), cos.to(BF)
    first, second = x1 * cos - x2 * sin, x2 * cos + x1 * sin            # all bf16
    assert first.dtype == BF
  else:
    first = (x1.to(F32) * cos - x2.to(F32) * sin).to(BF)                # bf16 * f32 promotes to f32
    second = (x2.to(F32) * cos + x1.to(F32) * sin).to(BF)
  typed = torch.cat([first, second], dim=-1).float()
  m = _model(family)
  got = m.rope(x.float(), pos, theta, flavor=family, scale_factor=sf)
  assert torch.equal(got, typed)
  other = m.rope(x.float(), pos, theta, flavor="llama3" if family == "qwen3" else "qwen3", scale_factor=sf)
  assert (got != other).float().mean() > 0.02      # the two flows differ in a visible share of elements


def _typed_attention(q, k, v, mask, scale, gemma):
  """One query position per row; q [B,Hq,dh], k / v [B,S,Hkv,dh] bf16; mask [B,S]."""
  B, Hq, dh = q.shape
  Hkv = k.shape[2]
  G = Hq // Hkv
  out = torch.empty(B, Hq, dh, dtype=BF)
  for b in range(B):
    for h in range(Hq):
      kk, vv = k[b, :, h // G], v[b, :, h // G]
      s = (kk.to(torch.float64) @ q[b, h].to(torch.float64)).to(F32).to(BF)   # bf16 einsum result
      if not gemma:
        s = s * scale                                   # bf16 * python float -> bf16
        s = torch.where(mask[b], s, torch.tensor(MR.K_MASK, dtype=BF))
        p = torch.softmax(s.to(F32), dim=-1).to(BF)     # llama3/model.py:390-392
      else:
        s = torch.where(mask[b], s, torch.tensor(MR.K_MASK, dtype=BF))
        e = torch.exp((s - s.max()).to(F32)).to(BF)     # jnp.exp of a bf16 array: bf16 result
        den = e.to(F32).sum().to(BF)                    # jnp.sum: fp32 accumulation, bf16 result
        p = e / den                                     # bf16 / bf16
        assert p.dtype == BF
      out[b, h] = (p.to(torch.float64) @ vv.to(torch.float64)).to(F32).to(BF)
  return out


@pytest.mark.parametrize("gemma", [False, True])
def test_attention_rounding_sites(gemma):
  """Scores rounded to bf16 (and scaled in bf16: llama3/model.py:383-388), softmax in fp32 cast to
  bf16 for Llama / Qwen3, and in the scores' own dtype for Gemma-3 (gemma3/model.py:647)."""
  B, S, Hq, Hkv, dh = 3, 40, 4, 2, 64
  q = _rand_bf((B, 1, Hq, dh), 11, 1.5)
  k, v = _rand_bf((B, S, Hkv, dh), 12, 1.5), _rand_bf((B, S, Hkv, dh), 13)
  mask = torch.ones(B, 1, S, dtype=torch.bool)
  mask[1, 0, 25:] = False
  mask[2, 0, :3] = False
  scale = dh ** -0.5
  m = _model("gemma3" if gemma else "llama3")
  got = m.attention(q.float(), k.float(), v.float(), mask, None if gemma else scale, score_dtype_softmax=gemma)
  typed = _typed_attention(q[:, 0], k, v, mask[:, 0], scale, gemma)
  assert torch.equal(got[:, 0], typed.float())
  other = m.attention(q.float(), k.float(), v.float(), mask, None if gemma else scale, score_dtype_softmax=not gemma)
  assert not torch.equal(got, other)                    # the softmax dtype is visible in the output


def test_activation_residual_embedding_and_logit_rounding_sites():
  """silu = x * sigmoid(x) as two bf16 ops and a bf16 product with `up` (llama3/model.py:493);
  gelu(tanh) as one bf16 op (gemma3/model.py:785-797); residual adds in bf16
  (llama3/model.py:560-563); Gemma-3's embedding scale sqrt(D) cast to the embedding dtype before
  the product (gemma3/model.py:353-358: 34.0 for D = 1152, not 33.94); logits = bf16 matmul cast
  to fp32 (llama3/model.py:688-697)."""
  g, u = _rand_bf((4, 96), 21, 2.0), _rand_bf((4, 96), 22)
  m = _model("llama3")
  typed = (g * torch.sigmoid(g.to(F32)).to(BF)) * u
  got = m.r(m.act(g.float()) * u.float())
  assert torch.equal(got, typed.float())
  one_rounding = Q.rb(g.float() * torch.sigmoid(g.float()) * u.float())
  assert (got != one_rounding).float().mean() > 0.02
  mg = _model("gemma3")
  typed_gelu = torch.nn.functional.gelu(g.to(F32), approximate="tanh").to(BF) * u
  assert torch.equal(mg.r(mg.act(g.float()) * u.float()), typed_gelu.float())
  a, b = _rand_bf((4, 96), 23, 4.0), _rand_bf((4, 96), 24, 0.01)
  assert torch.equal(m.r(a.float() + b.float()), (a + b).float())
  # embedding scale
  mg.w = {"embed": _rand_bf((50, 1152), 25, 0.02)}
  mg.cfg.embed_dim, mg.cfg.vocab_size = 1152, 50
  ids = torch.tensor([[1, 7, 49]])
  typed_emb = mg.w["embed"][ids] * torch.tensor(np.sqrt(1152.0), dtype=F32).to(BF)
  assert float(torch.tensor(np.sqrt(1152.0), dtype=F32).to(BF)) == 34.0
  assert torch.equal(mg.embed(ids), typed_emb.float())
  assert not torch.equal(mg.embed(ids), Q.rb(mg.w["embed"][ids].float() * float(np.sqrt(1152.0))))
  # logits of a tied head
  h = _rand_bf((2, 3, 1152), 26)
  mg.cfg.tied_embedding = True
  typed_lg = (h.to(torch.float64) @ mg.w["embed"].to(torch.float64).t()).to(F32).to(BF).to(F32)
  assert torch.equal(mg.logits(h.float()), typed_lg)


def test_lora_delta_rounds_t_and_adds_in_the_accumulator():
  """y = x W^ + (alpha / r) * bf16(x A) B: the down-projection is a bf16 einsum result (one
  rounding), the delta joins the base product before the output's single rounding."""
  from tunix_amd import config
  cfg = config.tiny_qwen3(num_layers=1, lora_rank=8, lora_alpha=16.0)
  K, N, r = 128, 64, 8
  w = {"l0.wq": _rand_bf((K, N), 31, 0.05), "l0.wq.lora_a": _rand_bf((K, r), 32, 0.05),
       "l0.wq.lora_b": _rand_bf((r, N), 33, 0.05)}
  m = MR.RefModel.__new__(MR.RefModel)
  m.cfg, m.bf16, m.acc, m.gemma_score_softmax = cfg, True, torch.float64, True
  m.w, m.q, m.lora = w, {}, {"l0.wq": (w["l0.wq.lora_a"].float(), w["l0.wq.lora_b"].float())}
  x = _rand_bf((5, K), 34)
  t = (x.to(torch.float64) @ w["l0.wq.lora_a"].to(torch.float64)).to(F32).to(BF)
  want = (x.to(torch.float64) @ w["l0.wq"].to(torch.float64)
          + 2.0 * (t.to(torch.float64) @ w["l0.wq.lora_b"].to(torch.float64))).to(F32)
  got = m.linear(x.float(), "l0.wq")
  np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=1e-6, atol=1e-7)
  t_unrounded = x.to(torch.float64) @ w["l0.wq.lora_a"].to(torch.float64)
  other = (x.to(torch.float64) @ w["l0.wq"].to(torch.float64)
           + 2.0 * (t_unrounded @ w["l0.wq.lora_b"].to(torch.float64))).to(F32)
  assert (Q.rb(got) != Q.rb(other)).float().mean() > 0.005


def test_gemma3_score_dtype_softmax_stays_within_the_logp_tolerance():
  """How far Gemma-3's bf16 softmax (the reference's flow, the oracle's default) is from an fp32
  softmax (what the HIP attention kernel computes, see its header): measured on a 3-layer Gemma-3
  shaped model with sliding-window layers, the log-probabilities of the two flows differ by far
  less than the 2e-2 the bf16 path is held to."""
  from tunix_amd import config, dummy_model
  from oracle import utils_ref as U
  cfg = config.gemma3_1b(num_layers=3, vocab_size=2048, embed_dim=256, hidden_dim=512, num_heads=4,
                         num_kv_heads=1, head_dim=64, sliding_window=8)
  w = dummy_model.create_dummy_weights(cfg, seed=5)
  rng = np.random.default_rng(5)
  tb = rng.integers(1, cfg.vocab_size, size=(3, 24))
  tb[1, :5] = 0
  mask = tb != 0
  args = (torch.from_numpy(tb.astype(np.int64)), torch.from_numpy(U.build_positions_from_mask(mask).astype(np.int64)))
  lps = []
  for score_dtype in (True, False):
    ref = MR.RefModel(cfg, w)
    ref.gemma_score_softmax = score_dtype
    lg = ref(*args, ref.init_cache(3, 24), torch.from_numpy(U.make_causal_attn_mask(mask)), 0)
    lps.append(torch.log_softmax(lg.float(), -1))
  diff = (lps[0] - lps[1]).abs().max().item()
  assert 0 < diff <= 2e-2, diff
