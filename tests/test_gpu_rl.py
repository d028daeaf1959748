"""GPU parity of the per-token log-probability path and the rollout engine against the oracle
(tolerances of the path: log-probabilities <= 2e-2 absolute against the bf16-flow oracle)."""
import numpy as np
import pytest
import torch

from oracle import model_ref as MR
from oracle import quant_ref as Q
from oracle import rl_ref as R

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tiny(gpu):
  from tunix_amd import config, dummy_model
  from tunix_amd.model import QLoRAModel
  cfg = config.tiny_qwen3(vocab_size=4096)
  # N(0, 0.02) weights as in the parity configurations: logits stay below 1 in magnitude, where
  # one bf16 ulp of a logit is far below the 2e-2 tolerance of the path
  w = dummy_model.create_dummy_weights(cfg, seed=77)
  return cfg, w, QLoRAModel(cfg, w, gpu)


def _tokens(cfg, B, P, T, seed):
  rng = np.random.default_rng(seed)
  prompt = rng.integers(2, cfg.vocab_size, size=(B, P)).astype(np.int32)
  comp = rng.integers(2, cfg.vocab_size, size=(B, T)).astype(np.int32)
  prompt[0, :5] = 0          # left padding
  prompt[2, :P - 1] = 0      # a one-token prompt
  comp[1, T - 4:] = 0        # right padding
  comp[3, 1:] = 0
  return prompt, comp


def test_per_token_logps_match_oracle(tiny, gpu):
  from tunix_amd.rl import common
  cfg, w, model = tiny
  B, P, T = 4, 24, 16
  prompt, comp = _tokens(cfg, B, P, T, 1)
  got = common.compute_per_token_logps(model, prompt, comp, pad_id=0, eos_id=1).cpu().numpy()
  ref = MR.RefModel(cfg, w)
  want = R.compute_per_token_logps(ref, prompt, comp, 0).numpy()
  valid = comp != 0
  err = np.abs(got - want)[valid].max()
  assert err <= 2e-2, err
  assert np.isfinite(got).all() and (got <= 1e-6).all()
  # temperature
  got_t = common.compute_per_token_logps(model, prompt, comp, pad_id=0, temperature=0.7).cpu().numpy()
  want_t = R.compute_per_token_logps(ref, prompt, comp, 0, temperature=0.7).numpy()
  assert np.abs(got_t - want_t)[valid].max() <= 2e-2
  assert np.abs(got_t - got)[valid].max() > 1e-3


def test_per_token_entropy_matches_oracle(tiny, gpu):
  """return_entropy: -sum p log p of the (temperature-scaled) next-token distribution at every
  completion position (tunix/rl/common.py:479-481, :1136-1148), from the fused head kernel."""
  from tunix_amd.rl import common
  cfg, w, model = tiny
  prompt, comp = _tokens(cfg, 4, 24, 16, 3)
  ref = MR.RefModel(cfg, w)
  for temp in (1.0, 0.6):
    lp, ent = common.compute_per_token_logps(model, prompt, comp, pad_id=0, temperature=temp, return_entropy=True)
    want_lp, want_ent = R.compute_per_token_logps(ref, prompt, comp, 0, temperature=temp, return_entropy=True)
    valid = comp != 0
    tol = 2e-2 / temp   # the bf16 resolution of a logit, divided by the temperature with it
    assert np.abs(lp.cpu().numpy() - want_lp.numpy())[valid].max() <= tol
    got = ent.cpu().numpy()
    assert np.isfinite(got).all() and (got >= 0).all() and (got <= np.log(cfg.vocab_size) + 1e-4).all()
    assert np.abs(got - want_ent.numpy())[valid].max() <= tol
    # the plain call returns the same log-probabilities bit for bit
    assert torch.equal(lp, common.compute_per_token_logps(model, prompt, comp, pad_id=0, temperature=temp))


def test_per_token_logps_chunking_and_batching_are_invariant(tiny, gpu):
  """tests/rl/common_test.py:340-399: the chunked computation returns the same values; here
  bit for bit, also when the batch is split over several forward passes."""
  from tunix_amd.rl import common
  cfg, w, model = tiny
  prompt, comp = _tokens(cfg, 4, 24, 16, 2)
  full = common.compute_per_token_logps(model, prompt, comp, pad_id=0)
  for chunk in (1, 5, 16):
    c = common.compute_per_token_logps(model, prompt, comp, pad_id=0, chunk_size=chunk)
    assert torch.equal(c, full), chunk
  # one sequence per forward pass selects other GEMM tilings (fewer rows): same values up to
  # the fp32 summation order, far inside the tolerance of the path
  one_by_one = common.compute_per_token_logps(model, prompt, comp, pad_id=0, max_rows=40)
  assert (one_by_one - full).abs().max().item() <= 1e-2


def test_packed_per_token_logps(tiny, gpu):
  """Packed batches (segment_ids / segment_positions: tunix/rl/common.py:260-271, :408-418): the
  HIP path against the oracle's packed branch (itself pinned by packed == unpacked), against the
  same sequences scored alone, and the shape / front padding of the result."""
  from tunix_amd.rl import common
  from packed_cases import packed_case
  cfg, w, model = tiny
  (A, Bq, Cq), ids, seg, pos = packed_case(cfg.vocab_size)
  empty = np.zeros((2, 0), np.int32)
  got = common.compute_per_token_logps(model, empty, ids, pad_id=0, segment_ids=seg, segment_positions=pos)
  assert tuple(got.shape) == (2, 24) and (got[:, 0] == 0).all()
  got = got.cpu().numpy()
  ref = MR.RefModel(cfg, w)
  want = R.compute_per_token_logps(ref, empty, ids, 0, segment_ids=seg, segment_positions=pos).numpy()
  real = seg != 0
  real[:, 0] = False
  assert np.abs(got - want)[real].max() <= 2e-2
  for row, off, q in ((0, 0, A), (0, 10, Bq), (1, 0, Cq)):
    alone = common.compute_per_token_logps(model, q[None, :1], q[None, 1:], pad_id=0).cpu().numpy()[0]
    # other key-block boundaries and GEMM row tiles than the packed pass: equal up to the bf16
    # resolution of the logits
    assert np.abs(got[row, off + 1: off + len(q)] - alone).max() <= 2e-2
  # entropy comes padded the same way; a missing segment_positions raises as in the reference
  lp, ent = common.compute_per_token_logps(model, empty, ids, pad_id=0, segment_ids=seg, segment_positions=pos,
                                           return_entropy=True)
  assert tuple(ent.shape) == (2, 24) and (ent[:, 0] == 0).all() and np.array_equal(lp.cpu().numpy(), got)
  with pytest.raises(ValueError, match="segment_positions"):
    common.compute_per_token_logps(model, empty, ids, pad_id=0, segment_ids=seg)
  # without the segment ids the second sequence sees the first: its scores move
  plain = common.compute_per_token_logps(model, ids[:, :1], ids[:, 1:], pad_id=0).cpu().numpy()
  assert np.abs(plain[0, 10:] - got[0, 11:]).max() > 1e-3


def test_per_token_logps_argument_errors(tiny, gpu):
  from tunix_amd.rl import common
  cfg, w, model = tiny
  with pytest.raises(ValueError):
    common.compute_per_token_logps(model, np.zeros((2, 4), np.int32), np.zeros((3, 4), np.int32), pad_id=0)
  empty = common.compute_per_token_logps(model, np.ones((2, 4), np.int32), np.ones((2, 0), np.int32), pad_id=0)
  assert tuple(empty.shape) == (2, 0)


def test_rollout_engine_contract_and_logprob_consistency(tiny, gpu):
  """generate() -> RolloutOutput; the log-probabilities the sampler reports for its own greedy
  tokens agree with get_per_token_logps over the same tokens (decode kernels vs the
  whole-sequence pass), and update_params changes them."""
  from tunix_amd.generate.utils import IdTokenizer
  from tunix_amd.rl import HipRollout, RolloutConfig
  cfg, w, model = tiny
  tok = IdTokenizer(cfg.vocab_size, pad_id=0, eos_id=1)
  ro = HipRollout(model, tok, 64)
  assert ro.pad_id() == 0 and ro.eos_id() == 1 and ro.model() is model
  rng = np.random.default_rng(3)
  prompts = [" ".join(str(int(t)) for t in rng.integers(2, cfg.vocab_size, size=n)) for n in (7, 16, 12)]
  rc = RolloutConfig(max_tokens_to_generate=12, temperature=0.0, top_p=None, max_prompt_length=16,
                     eos_tokens=[-1], return_logprobs=True)
  out = ro.generate(prompts, rc)
  assert len(out.text) == 3 and out.left_padded_prompt_tokens.shape == (3, 16)
  assert all(len(t) == 12 for t in out.tokens) and all(len(lp) == 12 for lp in out.logprobs)
  comp = np.stack(out.tokens).astype(np.int32)
  lps = ro.get_per_token_logps(out.left_padded_prompt_tokens, comp).cpu().numpy()
  assert np.abs(lps - np.asarray(out.logprobs, dtype=np.float32)).max() <= 2e-2
  # same tokens through the oracle
  ref = MR.RefModel(cfg, w)
  want = R.compute_per_token_logps(ref, out.left_padded_prompt_tokens, comp, 0).numpy()
  assert np.abs(lps - want).max() <= 2e-2
  # new adapter weights move the result; restoring them restores it bit for bit
  new = {k: (v.float() * 3).to(torch.bfloat16) for k, v in w.items() if ".lora_" in k}
  ro.update_params(new)
  moved = ro.get_per_token_logps(out.left_padded_prompt_tokens, comp).cpu().numpy()
  assert np.abs(moved - lps).max() > 1e-3
  ro.update_params({k: v for k, v in w.items() if ".lora_" in k})
  back = ro.get_per_token_logps(out.left_padded_prompt_tokens, comp).cpu().numpy()
  np.testing.assert_array_equal(back, lps)
  with pytest.raises(ValueError, match="same structure"):
    ro.update_params({"l0.wq.lora_a": new["l0.wq.lora_a"]})


def test_grpo_clipped_ratio(gpu):
  from tunix_amd.rl import common
  rng = np.random.default_rng(4)
  B, T = 8, 33
  lp = rng.normal(size=(B, T)).astype(np.float32) - 2
  old = lp + rng.normal(size=(B, T)).astype(np.float32) * 0.3
  adv = rng.normal(size=(B,)).astype(np.float32)
  ratio, loss, clipped = common.grpo_clipped_ratio(torch.from_numpy(lp).to(gpu), torch.from_numpy(old).to(gpu),
                                                   torch.from_numpy(adv).to(gpu), 0.2, 0.28)
  r_ref, l_ref, c_ref = R.grpo_ratio(lp, old, adv, 0.2, 0.28)
  np.testing.assert_allclose(ratio.cpu().numpy(), r_ref, rtol=2e-6)
  np.testing.assert_allclose(loss.cpu().numpy(), l_ref, rtol=2e-6, atol=1e-7)
  np.testing.assert_array_equal(clipped.cpu().numpy(), c_ref)
  ratio1, loss1, _ = common.grpo_clipped_ratio(torch.from_numpy(lp).to(gpu), None, torch.from_numpy(adv).to(gpu))
  np.testing.assert_array_equal(ratio1.cpu().numpy(), 1.0)
  np.testing.assert_allclose(loss1.cpu().numpy(), -adv[:, None] * np.ones((B, T), np.float32))


def test_fused_head_logps_training_scale_shapes(gpu):
  """The standalone fused per-token-logps case: hidden N(0,1) rows x a quantized lm_head
  (int4 g128 + LoRA r64) -> log-softmax -> gather -> GRPO ratio, logits never materialised.
  The oracle checks it at a vocabulary the CPU handles in seconds; at the full 128256-wide
  vocabulary the checks are properties: the fused statistics agree with the logits of a few
  rows materialised by the same kernel, and log-probabilities are a normalised distribution."""
  from tunix_amd import _lib as L
  from tunix_amd import ops
  D, r, group = 4096, 64, 128

  def run(V, rows, seed, want_logits_rows=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, D, generator=g).to(torch.bfloat16)
    w = (torch.randn(D, V, generator=g) * 0.02).to(torch.bfloat16)
    a = (torch.randn(D, r, generator=g) * 0.02).to(torch.bfloat16)
    b = (torch.randn(r, V, generator=g) * 0.01).to(torch.bfloat16)
    targets = torch.randint(0, V, (rows,), generator=g, dtype=torch.int32)
    gx, gt = x.to(gpu), targets.to(gpu)
    c, s = ops.quantize_pack(w.to(gpu), group, Q.INT4)
    t = torch.zeros(rows, r, dtype=torch.bfloat16, device=gpu)
    ops.lora_down(gx, a.t().contiguous().to(gpu), t)
    gb = b.t().contiguous().to(gpu)
    d = L.LmHeadDesc()
    d.M, d.D, d.V = rows, D, V
    d.x, d.codes, d.scales, d.group, d.qtype = gx.data_ptr(), c.data_ptr(), s.data_ptr(), group, Q.INT4
    d.lora_rank, d.t, d.t_ld, d.lora_b, d.lora_scale = r, t.data_ptr(), r, gb.data_ptr(), 1.0
    d.temperature = 1.0
    part = torch.empty(rows * ops.lmhead_nblocks(V) * 4, dtype=torch.float32, device=gpu)
    tlp = torch.empty(rows, dtype=torch.float32, device=gpu)
    lse = torch.empty(rows, dtype=torch.float32, device=gpu)
    d.targets, d.part, d.target_logp, d.lse = gt.data_ptr(), part.data_ptr(), tlp.data_ptr(), lse.data_ptr()
    ops.lmhead(d)
    lg = None
    if want_logits_rows:
      n = want_logits_rows
      lg = torch.empty(n, V, dtype=torch.float32, device=gpu)
      d2 = L.LmHeadDesc.from_buffer_copy(d)
      d2.M, d2.logits_out = n, lg.data_ptr()
      tlp2 = torch.empty(n, dtype=torch.float32, device=gpu)
      lse2 = torch.empty(n, dtype=torch.float32, device=gpu)
      d2.target_logp, d2.lse = tlp2.data_ptr(), lse2.data_ptr()
      ops.lmhead(d2)
      # from 512 rows on the many-rows kernel computes the statistics, the launch that materialises
      # the logits of a few rows does not: same logits up to the fp32 accumulation order
      torch.testing.assert_close(tlp2, tlp[:n], rtol=0, atol=2e-5 if rows < 512 else 1e-2)
      torch.testing.assert_close(lse2, lse[:n], rtol=0, atol=2e-5)
    torch.cuda.synchronize()
    return x, w, a, b, targets, tlp.cpu(), lse.cpu(), (None if lg is None else lg.cpu())

  # (1) against the oracle at a reduced vocabulary
  V = 2048
  x, w, a, b, targets, tlp, lse, _ = run(V, 192, 11)
  codes, scale = Q.quantize(w.float().numpy(), group, Q.INT4)
  logits = Q.rb(Q.qlinear_lora(x.float(), codes, scale, group, Q.INT4, a.float(), b.float(), 1.0))
  want = R.selective_log_softmax(logits, targets)
  assert (tlp - want).abs().max().item() <= 2e-2
  # (2) the full vocabulary: properties
  V = 128256
  rows = 1024
  x, w, a, b, targets, tlp, lse, lg = run(V, rows, 12, want_logits_rows=8)
  assert torch.isfinite(tlp).all() and (tlp <= 0).all()
  ref_lse = torch.logsumexp(lg, -1)
  np.testing.assert_allclose(lse[:8].numpy(), ref_lse.numpy(), atol=2e-5)
  sel = lg[torch.arange(8), targets[:8].long()] - ref_lse
  # one bf16 ulp of a logit of magnitude <= 2 (2^-7) where the two kernels round a target logit apart
  np.testing.assert_allclose(tlp[:8].numpy(), sel.numpy(), atol=1e-2)
  np.testing.assert_allclose(torch.exp(lg - ref_lse[:, None]).sum(-1).numpy(), 1.0, atol=1e-4)
  # (3) GRPO ratio against noisy reference log-probabilities (eps 0.2)
  from tunix_amd.rl import common
  g = torch.Generator().manual_seed(13)
  old = tlp + torch.randn(rows, generator=g) * 0.05
  adv = torch.randn(rows // 64, generator=g)
  ratio, loss, _ = common.grpo_clipped_ratio(tlp.view(-1, 64).to(gpu), old.view(-1, 64).to(gpu), adv.to(gpu), 0.2)
  r_ref, l_ref, _ = R.grpo_ratio(tlp.view(-1, 64).numpy(), old.view(-1, 64).numpy(), adv.numpy(), 0.2, 0.2)
  np.testing.assert_allclose(ratio.cpu().numpy(), r_ref, rtol=2e-6)
  np.testing.assert_allclose(loss.cpu().numpy(), l_ref, rtol=2e-6, atol=1e-7)


@pytest.mark.parametrize("method", ["kl", "mse_kl", "low_var_kl"])
@pytest.mark.parametrize("clamp", [None, 0.05])
def test_kl_divergence_matches_oracle(gpu, method, clamp):
  """tnx_kl_divergence against the oracle (itself pinned to the reference's KL tables): fp32
  arithmetic, so 1e-6 absolute (expf against numpy's exp in exp(d) - d - 1) plus 1e-6 relative;
  closed forms at equal inputs; the training-scale size of 128 x 1024 tokens."""
  from tunix_amd.rl import common as C
  rng = np.random.default_rng(5)
  for shape in ((3, 7), (128, 1024)):
    lp = (-rng.gamma(2.0, 1.5, size=shape)).astype(np.float32)
    ref = (lp + rng.normal(0, 0.3, size=shape)).astype(np.float32)
    ref[0, 0] = lp[0, 0] - 30.0 if method != "low_var_kl" else lp[0, 0] + 30.0   # an outlier for the clamp
    got = C.compute_kl_divergence(torch.from_numpy(lp).to(gpu), torch.from_numpy(ref).to(gpu), method, clamp)
    want = R.compute_kl_divergence(lp, ref, method, clamp)
    assert got.shape == shape and got.dtype == torch.float32
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=2e-6, atol=1e-6)
    if clamp is not None:
      assert got.abs().max().item() <= float(np.float32(clamp))
    same = C.compute_kl_divergence(torch.from_numpy(lp).to(gpu), torch.from_numpy(lp).to(gpu), method)
    assert (same == 0).all()
  with pytest.raises(ValueError, match="must be one of"):
    C.compute_kl_divergence(torch.zeros(2, device=gpu), torch.zeros(2, device=gpu), "reverse")


def _agg_cases():
  import json
  import os
  with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "aggregate_loss_cases.json")) as f:
    return [(c["mode"], c["loss"], c["mask"], c["kwargs"], c["expected"]) for c in json.load(f)]


@pytest.mark.parametrize("mode,loss,mask,kwargs,expected", _agg_cases())
def test_aggregate_loss_literal_cases(gpu, mode, loss, mask, kwargs, expected):
  """The cases of tests/rl/common_test.py:457-576 through tnx_aggregate_loss, same tolerance."""
  from tunix_amd.rl import common as C
  m = C.aggregate_loss(torch.tensor(loss, device=gpu), torch.tensor(mask, device=gpu), mode, **kwargs)
  np.testing.assert_allclose(m.compute().item(), expected, rtol=1e-6, atol=1e-6)


AGG_MODES = ["token-mean", "sequence-mean-token-mean", "sequence-mean-token-scale", "seq-mean-token-sum",
             "sequence-mean-token-sum-norm"]


@pytest.mark.parametrize("mode", AGG_MODES)
def test_aggregate_loss_training_scale(gpu, mode):
  """128 x 1024 tokens with ragged masks and two empty rows against the float64 oracle (fp32 sums
  of 1e5 terms: 1e-5 relative), and what holds at any size: the result is linear in the loss,
  the same on every launch, and zero under an all-zero mask."""
  from tunix_amd.rl import common as C
  rng = np.random.default_rng(11)
  B, T = 128, 1024
  loss = rng.normal(0.3, 1.0, size=(B, T)).astype(np.float32)
  lens = rng.integers(1, T + 1, size=B)
  lens[[5, 77]] = 0
  mask = (np.arange(T)[None, :] < lens[:, None])
  kwargs = {"norm": 37.5} if "norm" in mode or "scale" in mode else {}
  gl, gm = torch.from_numpy(loss).to(gpu), torch.from_numpy(mask).to(gpu)
  m = C.aggregate_loss(gl, gm, mode, **kwargs)
  num, den, min_denom = R.aggregate_loss(loss, mask, mode, **kwargs)
  assert m.min_denom == min_denom
  np.testing.assert_allclose(m.unreduced_sum.item(), num, rtol=1e-5, atol=1e-4)
  np.testing.assert_allclose(m.denominator.item(), den, rtol=1e-7)
  np.testing.assert_allclose(m.compute().item(), R.weighted_metric_compute(num, den, min_denom), rtol=1e-5,
                             atol=1e-6)
  again = C.aggregate_loss(gl, gm, mode, **kwargs)
  assert again.unreduced_sum.item() == m.unreduced_sum.item()
  scaled = C.aggregate_loss(gl * 4.0, gm, mode, **kwargs)          # a power of two: exact
  assert scaled.unreduced_sum.item() == 4.0 * m.unreduced_sum.item()
  zero = C.aggregate_loss(gl, torch.zeros_like(gm), mode, **kwargs)
  assert zero.compute().item() == 0.0
  # an integer or bf16 mask and a bf16 loss are converted, as the reference's astype does
  m16 = C.aggregate_loss(gl.to(torch.bfloat16), gm.to(torch.int32), mode, **kwargs)
  num16, _, _ = R.aggregate_loss(gl.to(torch.bfloat16).float().cpu().numpy(), mask, mode, **kwargs)
  np.testing.assert_allclose(m16.unreduced_sum.item(), num16, rtol=1e-5, atol=1e-4)


def test_aggregate_loss_argument_errors(gpu):
  from tunix_amd.rl import common as C
  x, k = torch.ones(2, 3, device=gpu), torch.ones(2, 3, device=gpu)
  with pytest.raises(ValueError, match="Unsupported loss aggregation mode"):
    C.aggregate_loss(x, k, "mean")
  for bad in (0, -2.0, "x"):
    with pytest.raises(ValueError, match="Invalid 'norm' value"):
      C.aggregate_loss(x, k, "sequence-mean-token-sum-norm", norm=bad)
  seg = torch.ones(2, 3, dtype=torch.int32, device=gpu)
  with pytest.raises(ValueError, match="num_segments must be provided"):
    C.aggregate_loss(x, k, "token-mean", segment_ids=seg)
  with pytest.raises(ValueError, match="explicit 'norm'"):
    C.aggregate_loss(x, k, "sequence-mean-token-scale", segment_ids=seg, num_segments=2)
  with pytest.raises(ValueError):
    C.aggregate_loss(x, k[:, :2], "token-mean")


def test_sampler_trainer_agreement_matches_oracle(gpu):
  """tnx_logp_drift against the oracle (fp32 two-pass moments there, double raw moments here:
  1e-5 relative, 1e-4 on the correlation), at the training-scale size, on the closed forms, and
  with an empty mask."""
  from tunix_amd.rl import common as C
  rng = np.random.default_rng(9)
  for shape in ((3, 7), (128, 512)):
    a = -rng.gamma(2.0, 1.0, size=shape).astype(np.float32)
    b = (a + rng.normal(0, 0.05, size=shape)).astype(np.float32)
    lens = rng.integers(0, shape[1] + 1, size=shape[0])
    mask = np.arange(shape[1])[None, :] < lens[:, None]
    b[~mask] -= 3.0
    ga, gb, gm = (torch.from_numpy(v).to(gpu) for v in (a, b, mask))
    got = C.sampler_trainer_agreement(ga, gb, gm)
    want = R.sampler_trainer_agreement(a, b, mask)
    assert list(got) == list(want)
    for k in want:
      np.testing.assert_allclose(got[k], want[k], rtol=1e-4 if k.endswith("corr") else 1e-5, atol=1e-7, err_msg=k)
    same = C.sampler_trainer_agreement(ga, ga, gm)
    assert same["sampler_trainer/logp_diff_max"] == 0 and same["sampler_trainer/prob_diff_max"] == 0
    np.testing.assert_allclose(same["sampler_trainer/probs_pearson_corr"], 1.0, rtol=1e-5)
    empty = C.sampler_trainer_agreement(ga, gb, torch.zeros_like(gm))
    assert all(v == 0 for v in empty.values())
  anti = C.sampler_trainer_agreement(torch.tensor([[0.2, 0.8]], device=gpu).log(),
                                     torch.tensor([[0.8, 0.2]], device=gpu).log(),
                                     torch.ones(1, 2, device=gpu))
  np.testing.assert_allclose(anti["sampler_trainer/probs_pearson_corr"], -1.0, rtol=1e-5)
  with pytest.raises(ValueError):
    C.sampler_trainer_agreement(torch.zeros(2, 3, device=gpu), torch.zeros(2, 4, device=gpu),
                                torch.ones(2, 3, device=gpu))


def test_rollout_and_logps_paths_agree_by_the_drift_monitor(tiny, gpu):
  """The monitor on the two paths of this package: the log-probabilities the decode loop records
  and compute_per_token_logps over the same tokens differ by bf16 rounding only."""
  from tunix_amd.generate import CacheConfig, Sampler
  from tunix_amd.generate.utils import IdTokenizer
  from tunix_amd.rl import common as C
  cfg, w, model = tiny
  tok = IdTokenizer(cfg.vocab_size, pad_id=0, eos_id=1)
  sampler = Sampler(model, tok, CacheConfig(64, cfg.num_layers, cfg.num_kv_heads, cfg.head_dim))
  T = 12
  out = sampler(["5 6 7 8", "9 10 11", "40 41 42 43 44 45"], max_generation_steps=T, return_logprobs=True,
                eos_tokens=[-1], pad_output=True)
  comp = torch.from_numpy(np.stack(out.tokens).astype(np.int32)).to(gpu)
  prompt = torch.from_numpy(out.padded_prompt_tokens.astype(np.int32)).to(gpu)
  rollout_lp = torch.from_numpy(np.stack(out.logprobs).astype(np.float32)).to(gpu)
  trainer_lp = C.compute_per_token_logps(model, prompt, comp, pad_id=0)
  m = C.sampler_trainer_agreement(rollout_lp, trainer_lp, torch.ones_like(comp))
  assert m["sampler_trainer/logp_diff_max"] <= 2e-2, m
  assert m["sampler_trainer/prob_diff_max"] <= 1e-3, m
  # (with these N(0, 0.02) weights every probability is close to 1 / V, the variances lie below
  # the 1e-12 floor of the formula and the correlation figure carries no information)
  want = R.sampler_trainer_agreement(rollout_lp.cpu().numpy(), trainer_lp.cpu().numpy(), np.ones((3, T)))
  for k in want:
    np.testing.assert_allclose(m[k], want[k], rtol=1e-4, atol=1e-6, err_msg=k)


MODES = ["token-mean", "sequence-mean-token-mean", "sequence-mean-token-scale", "seq-mean-token-sum",
         "sequence-mean-token-sum-norm"]


@pytest.mark.parametrize("mode", MODES)
def test_segmented_aggregate_loss_matches_oracle(gpu, mode):
  """tnx_aggregate_loss_segmented against the oracle on packed rows (random segment layouts with
  padding, empty segments, unscored segments, ids beyond num_segments), on the reference's own
  packed gate case (-2.25), and packed == unpacked; two launches give identical bits."""
  from tunix_amd.rl import common as C
  rng = np.random.default_rng(21)
  for (B, T, S) in ((1, 4, 3), (5, 37, 6), (16, 2500, 300), (3, 1024, 9)):
    loss = rng.normal(0, 1, size=(B, T)).astype(np.float32)
    seg = np.zeros((B, T), dtype=np.int32)
    for b in range(B):   # runs of ascending segment ids, then padding; some ids skipped
      cuts = np.sort(rng.choice(np.arange(1, T), size=min(S + 1, T - 1), replace=False))
      ids = np.concatenate([np.arange(1, len(cuts) + 1), [0]])
      ids[rng.random(len(ids)) < 0.15] = 0
      seg[b] = np.repeat(ids, np.diff(np.concatenate([[0], cuts, [T]])))[:T]
    mask = (rng.random((B, T)) < 0.7).astype(np.float32)
    mask[seg == 2] = 0.0                      # a segment with no scored token is not active
    kw = {"norm": 17.0} if mode == "sequence-mean-token-scale" else {}
    want = R.aggregate_loss_segmented(loss, mask, mode, seg, S, **kw)
    gl, gm, gs = (torch.from_numpy(v).to(gpu) for v in (loss, mask, seg))
    got = C.aggregate_loss(gl, gm, mode, segment_ids=gs, num_segments=S, **kw)
    again = C.aggregate_loss(gl, gm, mode, segment_ids=gs, num_segments=S, **kw)
    np.testing.assert_allclose(got.unreduced_sum.item(), want[0], rtol=2e-5, atol=2e-4)
    np.testing.assert_allclose(got.denominator.item(), want[1], rtol=1e-6)
    assert got.min_denom == want[2]
    assert got.unreduced_sum.item() == again.unreduced_sum.item()
    if mode == "sequence-mean-token-sum-norm":
      named = C.aggregate_loss(gl, gm, mode, segment_ids=gs, num_segments=S, norm=5.0)
      assert named.denominator.item() == 5.0
  # the reference's packed gate (tests/rl/algo_core_test.py:51-143)
  loss = -torch.tensor([[1.5, 1.5, 1.5, 3.0]], device=gpu)
  ones = torch.ones(1, 4, device=gpu)
  seg = torch.tensor([[1, 1, 1, 2]], dtype=torch.int32, device=gpu)
  if mode == "sequence-mean-token-mean":
    packed = C.aggregate_loss(loss, ones, mode, segment_ids=seg, num_segments=3).compute().item()
    np.testing.assert_allclose(packed, -2.25, rtol=1e-6)
    unpacked = C.aggregate_loss(-torch.tensor([[1.5, 1.5, 1.5], [3.0, 0.0, 0.0]], device=gpu),
                                torch.tensor([[1.0, 1, 1], [1, 0, 0]], device=gpu), mode).compute().item()
    np.testing.assert_allclose(packed, unpacked, rtol=1e-6)
