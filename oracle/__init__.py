"""CPU oracle: a restatement of the reference's algorithm for the quantized rollout-decode path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this directory; only
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it, as the checker.

Every function cites the google/tunix file:line it follows (paths relative to the reference
tree).  Pinning status of each part:

  utils_ref      masks / positions / index helpers: pinned by the literal vectors of
                 tests/generate/utils_test.py:91-168 and tests/sft/sft_utils_test.py:22-68.
  rl_ref         KL estimators: pinned by the three tables of tests/rl/common_test.py:35-77
                 (mutually consistent closed forms); selective_log_softmax: pinned against
                 scipy.special.logsumexp / torch.log_softmax and the chunk-invariance property of
                 tests/rl/common_test.py:340-399; GRPO ratio: closed form + the old=None case of
                 tests/rl/algo_core_test.py:51-143 (ratio == 1).
                 aggregate_loss (five modes, no packing segments) and WeightedMetric.compute:
                 pinned by the thirteen literal cases of tests/rl/common_test.py:457-576.
                 aggregate_loss_segmented (packed batches, :857-940): pinned by the packed gate of
                 tests/rl/algo_core_test.py:51-143 (-2.25, and -1.875 for the per-row form) and by
                 the property that gate asserts -- packed equals unpacked -- run on the same
                 thirteen literal cases.
                 sampler_trainer_agreement (grpo_learner.py:405-440; the reference holds no
                 vector for it): pinned by numpy.corrcoef / masked means and maxima over the
                 masked subset, and by the closed forms (equal inputs, a constant log offset,
                 an anti-correlated pair, an empty mask).
  model_ref      RMSNorm / RoPE / GQA attention / SwiGLU / full decoder: pinned against
                 transformers' Qwen3 / Llama / Gemma3 / Qwen3Moe random-init models in fp32
                 (tol 1e-3, the equivalence tests/model_alignment/qwen_align_test.py:113-200
                 asserts for the reference itself) and by brute-force fp64 attention.  Where the
                 bf16 mode rounds (the r() calls): pinned by tests/test_oracle_rounding.py, which
                 writes each cited formula out again with real bf16 / fp32 tensors and jax's
                 promotion rules, so that the dtypes do the rounding, and shows for every site
                 that a moved or dropped rounding changes the result.  What stays unpinned
                 there: the precision XLA keeps INSIDE one bf16 op (the accumulation order and
                 width of a bf16 einsum or reduction), i.e. bit-exact agreement with XLA-CPU.
  quant_ref      int4 / NF4 group quantisation and the QArray arithmetic live in the third-party
                 package qwix (pyproject.toml:43 `qwix>=0.1.6`, not vendored, not installed):
                 PARITY UNPINNED against qwix.  The format is defined by include/tunix_hip.h;
                 pinned here only by closed forms (fp64 x @ dequant, zero codes, scale linearity,
                 group boundaries, brute force at tiny sizes).  The LoRA delta is pinned by the
                 merge formula tunix/models/safetensors_saver.py:107 and the B = 0 invariant.
  threefry       jax.random bit stream (threefry2x32, fold_in, uniform, categorical): pinned by
                 the golden arrays of tests/rl/common_test.py:35-108, which were produced from
                 jax.random.PRNGKey(0) inputs.
  sampler_ref    sample_best / sample_top_p / the prefill+decode loop of
                 tunix/generate/sampler.py: greedy pinned by numpy.argmax first-index rule;
                 top-p ids for a seed depend on the threefry pin above plus XLA's log/exp
                 rounding: PARITY UNPINNED for exact sampled ids.
"""
