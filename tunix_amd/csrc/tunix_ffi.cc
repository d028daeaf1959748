// XLA FFI handlers over libtunix_hip.so: one jax.ffi custom-call target per kernel family, so that
// the reference's JAX code (tunix/generate/sampler.py, tunix/rl/common.py) can call the HIP
// kernels from jitted functions.  Built only where jaxlib's headers exist:
//     make -C tunix_amd/csrc ffi XLA_FFI_INCLUDE=$(python -c "import jaxlib, os; print(os.path.join(os.path.dirname(jaxlib.__file__), 'include'))")
// Every handler fills the C descriptor from the call frame and forwards XLA's stream; XLA owns all
// buffers (outputs and workspaces are Ret buffers), optional operands arrive as zero-element
// buffers, scalars that live on the device (the step counter) are one-element int32 buffers.
#include <hip/hip_runtime.h>

#include "tunix_hip.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;
using Buf = ffi::AnyBuffer;
using Out = ffi::Result<ffi::AnyBuffer>;

namespace {
template <class T> T* ptr(Buf b) { return b.element_count() ? reinterpret_cast<T*>(b.untyped_data()) : nullptr; }
template <class T> T* ptr(Out& b) { return b->element_count() ? reinterpret_cast<T*>(b->untyped_data()) : nullptr; }
ffi::Error done(int rc) {
  return rc ? ffi::Error(ffi::ErrorCode::kInvalidArgument, tnx_last_error()) : ffi::Error::Success();
}
int64_t rows(Buf b) {   // product of all but the last dimension
  int64_t n = 1;
  for (size_t i = 0; i + 1 < b.dimensions().size(); ++i) n *= b.dimensions()[i];
  return n;
}
int64_t last(Buf b) { return b.dimensions().back(); }
}  // namespace

static ffi::Error LoraDown(hipStream_t s, Buf x, Buf a_t, Out t) {
  return done(tnx_lora_down(s, ptr<const uint16_t>(x), rows(x), last(x), ptr<const uint16_t>(a_t),
                            (int)a_t.dimensions()[0], ptr<uint16_t>(t), t->dimensions().back()));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(tnx_lora_down_ffi, LoraDown,
    ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>().Arg<Buf>().Arg<Buf>().Ret<Buf>());

static ffi::Error QLinear(hipStream_t s, Buf x, Buf codes, Buf scales, Buf t, Buf lora_b, Buf residual, Out y, Out ws,
                          int32_t group, int32_t qtype, int32_t lora_rank, int32_t lora_nseg,
                          ffi::Span<const int64_t> seg_end, ffi::Span<const int32_t> seg_toff, float lora_scale,
                          int32_t epilogue, int32_t split_k) {
  tnx_qlinear_desc d = {};
  d.M = rows(x); d.K = last(x);
  d.N = (epilogue == TNX_EPI_SILU_MUL || epilogue == TNX_EPI_GELU_MUL) ? 2 * y->dimensions().back() : y->dimensions().back();
  d.group = group; d.qtype = qtype; d.epilogue = epilogue; d.split_k = split_k;
  d.x = ptr<const uint16_t>(x); d.codes = ptr<const uint32_t>(codes); d.scales = ptr<const uint16_t>(scales);
  d.residual = ptr<const uint16_t>(residual); d.y = y->untyped_data(); d.ws = ptr<float>(ws);
  d.lora_rank = lora_rank; d.lora_nseg = lora_nseg; d.lora_scale = lora_scale;
  for (size_t i = 0; i < seg_end.size() && i < 4; ++i) d.lora_seg_end[i] = seg_end[i];
  for (size_t i = 0; i < seg_toff.size() && i < 4; ++i) d.lora_seg_toff[i] = seg_toff[i];
  d.t = ptr<const uint16_t>(t); d.t_ld = t.element_count() ? last(t) : 0; d.lora_b = ptr<const uint16_t>(lora_b);
  int rc = tnx_qlinear_lora(s, &d);
  if (!rc && split_k > 1) rc = tnx_splitk_finish(s, &d);
  return done(rc);
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(tnx_qlinear_lora_ffi, QLinear,
    ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
        .Arg<Buf>().Ret<Buf>().Ret<Buf>().Attr<int32_t>("group").Attr<int32_t>("qtype").Attr<int32_t>("lora_rank")
        .Attr<int32_t>("lora_nseg").Attr<ffi::Span<const int64_t>>("lora_seg_end")
        .Attr<ffi::Span<const int32_t>>("lora_seg_toff").Attr<float>("lora_scale").Attr<int32_t>("epilogue")
        .Attr<int32_t>("split_k"));

// y = norm(h), h = x (+ res_pre); x may be the split_k partial planes of a linear (ws, fp32)
static ffi::Error RmsNorm(hipStream_t s, Buf x, Buf ws, Buf res_pre, Buf w, Out h_out, Out y, float eps, int32_t flavor,
                          int32_t split_k) {
  const int64_t D = last(w), M = y->element_count() / D;
  if (split_k > 1)
    return done(tnx_rmsnorm_splitk(s, ptr<const float>(ws), split_k, ptr<const uint16_t>(res_pre), ptr<uint16_t>(h_out),
                                   ptr<const uint16_t>(w), nullptr, ptr<uint16_t>(y), M, D, eps, flavor));
  return done(tnx_rmsnorm(s, ptr<const uint16_t>(x), ptr<const uint16_t>(res_pre), ptr<uint16_t>(h_out),
                          ptr<const uint16_t>(w), nullptr, ptr<uint16_t>(y), M, D, eps, flavor));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(tnx_rmsnorm_ffi, RmsNorm,
    ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>()
        .Ret<Buf>().Attr<float>("eps").Attr<int32_t>("flavor").Attr<int32_t>("split_k"));

// in place on the caches: bind them with input_output_aliases (operands 6, 7 -> results 1, 2)
static ffi::Error RopeKv(hipStream_t s, Buf qkv, Buf timescale, Buf q_norm_w, Buf k_norm_w, Buf positions, Buf col,
                         Buf kcache, Buf vcache, Out q_out, Out kc_out, Out vc_out, int32_t Hq, int32_t Hkv,
                         int32_t rope_flavor, float rope_scale, int32_t qk_norm, float norm_eps, float q_prescale) {
  tnx_rope_desc d = {};
  d.B = positions.dimensions()[0]; d.T = rows(qkv) / d.B; d.S = kcache.dimensions()[2];
  d.Hq = Hq; d.Hkv = Hkv; d.dh = (int)kcache.dimensions()[3];
  d.rope_flavor = rope_flavor; d.rope_scale = rope_scale; d.timescale = ptr<const float>(timescale);
  d.qk_norm = qk_norm; d.norm_eps = norm_eps; d.q_prescale = q_prescale;
  d.q_norm_w = ptr<const uint16_t>(q_norm_w); d.k_norm_w = ptr<const uint16_t>(k_norm_w);
  d.qkv = ptr<const uint16_t>(qkv); d.positions = ptr<const int32_t>(positions); d.pos_ld = last(positions);
  d.col_ptr = ptr<const int32_t>(col); d.q_out = ptr<uint16_t>(q_out);
  d.kcache = ptr<uint16_t>(kc_out); d.vcache = ptr<uint16_t>(vc_out);   // aliased to kcache / vcache
  return done(tnx_qknorm_rope_kvwrite(s, &d));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(tnx_qknorm_rope_kvwrite_ffi, RopeKv,
    ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
        .Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Attr<int32_t>("Hq").Attr<int32_t>("Hkv")
        .Attr<int32_t>("rope_flavor").Attr<float>("rope_scale").Attr<int32_t>("qk_norm").Attr<float>("norm_eps")
        .Attr<float>("q_prescale"));

static ffi::Error Attn(hipStream_t s, Buf q, Buf kcache, Buf vcache, Buf tokens, Buf segment_ids, Buf col, Out out, Out ws,
                       int32_t Hq, float scale, int32_t window, int32_t pad_id, int32_t kv_chunk) {
  tnx_attn_desc d = {};
  d.B = kcache.dimensions()[0]; d.Hkv = (int)kcache.dimensions()[1]; d.S = kcache.dimensions()[2];
  d.dh = (int)kcache.dimensions()[3]; d.Hq = Hq; d.T = q.element_count() / (d.B * Hq * d.dh);
  d.scale = scale; d.window = window; d.pad_id = pad_id; d.kv_chunk = kv_chunk;
  d.q = ptr<const uint16_t>(q); d.kcache = ptr<const uint16_t>(kcache); d.vcache = ptr<const uint16_t>(vcache);
  d.tokens = ptr<const int32_t>(tokens); d.tok_ld = last(tokens.element_count() ? tokens : segment_ids);
  d.segment_ids = ptr<const int32_t>(segment_ids); d.col_ptr = ptr<const int32_t>(col);
  d.ws = ptr<float>(ws); d.out = ptr<uint16_t>(out);
  return done(tnx_gqa_attn(s, &d));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(tnx_gqa_attn_ffi, Attn,
    ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
        .Arg<Buf>().Ret<Buf>().Ret<Buf>().Attr<int32_t>("Hq").Attr<float>("scale").Attr<int32_t>("window")
        .Attr<int32_t>("pad_id").Attr<int32_t>("kv_chunk"));

static ffi::Error LmHead(hipStream_t s, Buf x, Buf w_bf16, Buf codes, Buf scales, Buf t, Buf lora_b, Buf targets,
                         Buf forbidden, Out part, Out best_id, Out best_logp, Out target_logp, Out lse, int32_t V,
                         int32_t group, int32_t qtype, int32_t lora_rank, float lora_scale, float temperature,
                         int32_t logits_fp32) {
  tnx_lmhead_desc d = {};
  d.M = rows(x); d.D = last(x); d.V = V;
  d.x = ptr<const uint16_t>(x); d.w_bf16 = ptr<const uint16_t>(w_bf16);
  d.codes = ptr<const uint32_t>(codes); d.scales = ptr<const uint16_t>(scales); d.group = group; d.qtype = qtype;
  d.lora_rank = lora_rank; d.t = ptr<const uint16_t>(t); d.t_ld = t.element_count() ? last(t) : 0;
  d.lora_b = ptr<const uint16_t>(lora_b); d.lora_scale = lora_scale; d.temperature = temperature;
  d.forbidden = ptr<const int32_t>(forbidden); d.n_forbidden = (int)forbidden.element_count();
  d.targets = ptr<const int32_t>(targets); d.part = ptr<float>(part);
  d.best_id = ptr<int32_t>(best_id); d.best_logp = ptr<float>(best_logp);
  d.target_logp = ptr<float>(target_logp); d.lse = ptr<float>(lse); d.logits_fp32 = logits_fp32;
  return done(tnx_lmhead_logp(s, &d));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(tnx_lmhead_logp_ffi, LmHead,
    ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
        .Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Attr<int32_t>("V")
        .Attr<int32_t>("group").Attr<int32_t>("qtype").Attr<int32_t>("lora_rank").Attr<float>("lora_scale")
        .Attr<float>("temperature").Attr<int32_t>("logits_fp32"));

// the grouped GEMM over routes already sorted by expert (megablox.gmm's operator shape)
static ffi::Error MoeGmm(hipStream_t s, Buf x, Buf codes, Buf scales, Buf offsets, Buf sorted_route, Out y, int32_t E,
                         int32_t k, int32_t x_div, int32_t N, int32_t group, int32_t qtype, int32_t epilogue) {
  tnx_moe_gmm_desc d = {};
  d.n_routes = sorted_route.element_count(); d.E = E; d.k = k; d.K = last(x); d.N = N; d.group = group; d.qtype = qtype;
  d.x = ptr<const uint16_t>(x); d.x_div = x_div; d.codes = ptr<const uint32_t>(codes);
  d.scales = ptr<const uint16_t>(scales); d.offsets = ptr<const int32_t>(offsets);
  d.sorted_route = ptr<const int32_t>(sorted_route); d.epilogue = epilogue; d.y = ptr<uint16_t>(y);
  return done(tnx_moe_int4_gmm(s, &d));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(tnx_moe_int4_gmm_ffi, MoeGmm,
    ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
        .Ret<Buf>().Attr<int32_t>("E").Attr<int32_t>("k").Attr<int32_t>("x_div").Attr<int32_t>("N")
        .Attr<int32_t>("group").Attr<int32_t>("qtype").Attr<int32_t>("epilogue"));

static ffi::Error SampleTopK(hipStream_t s, Buf logits, Buf forbidden, Buf step, Out ids, Out logp, Out ws, int32_t k,
                             float top_p, float temperature, int64_t key, int32_t rng_variant) {
  return done(tnx_sample_topk(s, ptr<const float>(logits), rows(logits), last(logits), k, top_p, temperature,
                              (uint32_t)(key >> 32), (uint32_t)key, rng_variant, ptr<const int32_t>(forbidden),
                              (int)forbidden.element_count(), ptr<const int32_t>(step), ptr<float>(ws),
                              ptr<int32_t>(ids), ptr<float>(logp)));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(tnx_sample_topk_ffi, SampleTopK,
    ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>()
        .Ret<Buf>().Attr<int32_t>("k").Attr<float>("top_p").Attr<float>("temperature").Attr<int64_t>("key")
        .Attr<int32_t>("rng_variant"));

static ffi::Error GrpoRatio(hipStream_t s, Buf logp, Buf old_logp, Buf adv, Out ratio, Out loss, Out clipped,
                            float eps_lo, float eps_hi) {
  return done(tnx_grpo_ratio(s, ptr<const float>(logp), ptr<const float>(old_logp), ptr<const float>(adv),
                             logp.element_count(), last(logp), eps_lo, eps_hi, ptr<float>(ratio), ptr<float>(loss),
                             ptr<int32_t>(clipped)));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(tnx_grpo_ratio_ffi, GrpoRatio,
    ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>()
        .Ret<Buf>().Attr<float>("eps_lo").Attr<float>("eps_hi"));

static ffi::Error Kl(hipStream_t s, Buf logp, Buf ref_logp, Out kl, int32_t method, float clamp) {
  return done(tnx_kl_divergence(s, ptr<const float>(logp), ptr<const float>(ref_logp), logp.element_count(), method,
                                clamp, ptr<float>(kl)));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(tnx_kl_divergence_ffi, Kl,
    ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Attr<int32_t>("method")
        .Attr<float>("clamp"));

// out = (unreduced sum, denominator); segment_ids with elements selects the packed-batch form
static ffi::Error AggLoss(hipStream_t s, Buf loss, Buf mask, Buf segment_ids, Out out, Out ws, int32_t mode, float norm,
                          int32_t num_segments) {
  const int64_t B = loss.dimensions()[0], T = last(loss);
  if (segment_ids.element_count())
    return done(tnx_aggregate_loss_segmented(s, ptr<const float>(loss), ptr<const float>(mask),
                                             ptr<const int32_t>(segment_ids), B, T, num_segments, mode, norm,
                                             ptr<float>(ws), ptr<float>(out)));
  return done(tnx_aggregate_loss(s, ptr<const float>(loss), ptr<const float>(mask), B, T, mode, norm, ptr<float>(ws),
                                 ptr<float>(out)));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(tnx_aggregate_loss_ffi, AggLoss,
    ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>()
        .Attr<int32_t>("mode").Attr<float>("norm").Attr<int32_t>("num_segments"));

static ffi::Error Drift(hipStream_t s, Buf rollout_logp, Buf trainer_logp, Buf mask, Out out5, Out ws) {
  return done(tnx_logp_drift(s, ptr<const float>(rollout_logp), ptr<const float>(trainer_logp), ptr<const float>(mask),
                             rollout_logp.dimensions()[0], last(rollout_logp), ws->untyped_data(), ptr<float>(out5)));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(tnx_logp_drift_ffi, Drift,
    ffi::Ffi::Bind().Ctx<ffi::PlatformStream<hipStream_t>>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>());
