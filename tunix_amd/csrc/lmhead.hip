// Fused lm_head -> log-softmax statistics.  Every work-group computes a [16*MT x 128] tile of
// bf16-rounded logits with the shared skinny-GEMM main loop and reduces it on the spot to
// (max, first arg-max, sum of exponentials, logit of the row's target id); a second small
// kernel merges the per-block statistics of a row.  Full-vocabulary logits reach HBM only when
// the caller asks for them (logits_out).
#include <string.h>

#include <mutex>

#include "gemm_tile.h"
#include "rng.h"

// defined beside the 128 x 256 GEMM kernel: 0 = launched, 1 = not a shape it takes, < 0 = error
int tnx_internal_wide_head(hipStream_t st, const tnx_lmhead_desc* d, float temperature, int64_t nvb,
                           float* part_ent);

namespace {

struct LHArgs {
  int64_t M, D, V;
  const uint16_t* x;
  const uint16_t* w_bf16;
  const uint32_t* codes;
  const uint16_t* scales;
  int group, qtype;
  int lora_rank;
  const uint16_t* t;
  int64_t t_ld;
  const uint16_t* lora_b;
  float lora_scale;
  float temperature;
  const int32_t* forbidden;
  int n_forbidden;
  const int32_t* targets;
  float* part;
  int64_t nvb;
  float* logits_out;
  float* part_ent;   // optional [M, nvb]: sum of exp(l - max) * l per block, for the entropy
  // optional whole-vocabulary categorical draw (Gumbel-max with jax's threefry stream)
  float* part_draw;  // [M, nvb, 3]: best (logit + noise), its id, its logit
  uint32_t key0, key1;
  int variant;
  const int32_t* step_ptr;
  int logits_fp32;   // keep the fp32 accumulator as the logit (reference mode)
};

constexpr float kNegInf = -__builtin_inff();

struct Stat {
  float mx;
  int idx;
  float sum;
  float tgt;
  float wsum;  // sum of exp(l - mx) * l  (entropy = logsumexp - wsum / sum)
  float gv;    // best logit + gumbel noise, its column and its logit (the categorical draw)
  int gi;
  float gl;
};
// Merge two statistics; `a` covers lower column indices than `b`.
__device__ __forceinline__ Stat merge(const Stat& a, const Stat& b) {
  Stat r;
  r.mx = fmaxf(a.mx, b.mx);
  r.idx = (b.mx > a.mx) ? b.idx : a.idx;  // equal maxima: keep the lower index
  const float wa = a.mx == kNegInf ? 0.f : __expf(a.mx - r.mx);
  const float wb = b.mx == kNegInf ? 0.f : __expf(b.mx - r.mx);
  r.sum = a.sum * wa + b.sum * wb;
  r.wsum = a.wsum * wa + b.wsum * wb;
  r.tgt = fmaxf(a.tgt, b.tgt);
  const bool tb = b.gv > a.gv || (b.gv == a.gv && b.gi < a.gi);  // larger value, then lower index
  r.gv = tb ? b.gv : a.gv;
  r.gi = tb ? b.gi : a.gi;
  r.gl = tb ? b.gl : a.gl;
  return r;
}

// A work-group covers 16 * MT rows x 64 * NT columns = NT / 2 statistics blocks of 128 columns.
// NT = 2 everywhere today.  The dense (bf16 weight) flavour is bound by what a compute unit can
// fetch; it needs no code-book table, so its LDS footprint lets two work-groups share a compute
// unit, and the launch bound (a register budget, the work-group size is always 256) keeps it
// within half the register file.  NT = 4 for the dense flavour (256 columns: half the activation
// re-reads per weight byte, one work-group of four waves per unit with its accumulators in AGPRs)
// was measured at 376 us against 312 us for the Llama-3.1-8B head at 128 rows: two independent
// four-wave groups hide each other's barrier and load waits, one group waits together.
template <int MT, int NT, bool DENSE>
__global__ __launch_bounds__(DENSE && NT == 2 ? 512 : 256) void lmhead_kernel(const LHArgs a) {
  static_assert(NT == 2 || NT == 4, "one or two 128-column statistics blocks per work-group");
  extern __shared__ __align__(16) unsigned char smem[];
  uint16_t* sA = reinterpret_cast<uint16_t*>(smem);
  uint32_t* sLut = tile_lut(smem, MT);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lm = lane & 15, lq = lane >> 4;
  const int64_t vb = blockIdx.x;
  const int64_t m0 = (int64_t)blockIdx.y * (MT * 16);
  const int64_t ntile0 = (vb * 4 + wave) * NT;

  const uint32_t* lut_lane = nullptr;
  if constexpr (!DENSE) {
    build_lut(sLut, a.qtype, tid, 256);
    lut_lane = sLut + (lane & (TNX_LUT_COPIES - 1));
  }
  TileSrc s;
  s.M = a.M; s.K = a.D; s.x = a.x; s.row_index = nullptr; s.row_div = 1; s.x_rows = a.M;
  s.w_bf16 = a.w_bf16;
  s.codes = a.codes; s.scales = a.scales; s.group = a.group; s.qtype = a.qtype;
  s.ntiles = a.V / 16; s.lora_rank = a.lora_rank; s.t = a.t; s.t_ld = a.t_ld;
  s.lora_b = a.lora_b; s.lora_scale = a.lora_scale;

  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) zero_acc(acc[mt][nt]);
  tile_mainloop<MT, NT, DENSE>(s, m0, ntile0, 0, (int)(a.D / KTILE), sA, lut_lane, acc);
  if (a.lora_rank > 0) {
    int toff[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) toff[nt] = 0;
    tile_lora<MT, NT>(s, m0, ntile0, toff, acc);
  }

  __syncthreads();  // sA is reused for the cross-wave reduction
  Stat* sRed = reinterpret_cast<Stat*>(smem);  // [4 waves][16*MT rows]
  int64_t col[NT];
  bool ok[NT], in_v[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    col[nt] = (ntile0 + nt) * 16 + lm;
    in_v[nt] = (ntile0 + nt) < s.ntiles;
    ok[nt] = in_v[nt];
  }
  for (int f = 0; f < a.n_forbidden; ++f) {
    const int64_t fid = a.forbidden[f];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      if (fid == col[nt]) ok[nt] = false;
  }
  // fold_in(key, step) for the draw: threefry of the key over the counter pair (0, step)
  uint32_t ks0 = 0u, ks1 = 0u;
  if (a.part_draw) {
    ks1 = (uint32_t)(*a.step_ptr);
    threefry2x32(a.key0, a.key1, ks0, ks1);
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int rl = mt * 16 + lq * 4 + i;
      const int64_t row = m0 + rl;
      const bool rok = row < a.M;
      // logits are the bf16 einsum output cast to fp32, then divided by the temperature
      float raw[NT], l[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        raw[nt] = a.logits_fp32 ? acc[mt][nt][i] : rbf(acc[mt][nt][i]);
        l[nt] = ok[nt] ? __fdiv_rn(raw[nt], a.temperature) : kNegInf;
      }
      if (a.logits_out && rok) {  // raw model logits: no temperature, no forbidden mask
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          if (in_v[nt]) a.logits_out[row * a.V + col[nt]] = raw[nt];
      }
      const int tg = (a.targets && rok) ? a.targets[row] : -1;
      // this lane's columns grow with nt: the first maximum wins
      float mx = l[0], tgt = tg == (int)col[0] ? l[0] : kNegInf;
      int idx = (int)col[0];
#pragma unroll
      for (int nt = 1; nt < NT; ++nt) {
        if (l[nt] > mx) {
          mx = l[nt];
          idx = (int)col[nt];
        }
        if (tg == (int)col[nt]) tgt = l[nt];
      }
      // arg-max over the 16 lanes of the row (columns grow with lm)
#pragma unroll
      for (int o = 1; o < 16; o <<= 1) {
        const float omx = __shfl_xor(mx, o, 64);
        const int oidx = __shfl_xor(idx, o, 64);
        if (omx > mx || (omx == mx && oidx < idx)) {
          mx = omx;
          idx = oidx;
        }
        tgt = fmaxf(tgt, __shfl_xor(tgt, o, 64));
      }
      float se = 0.f, we = 0.f;
      if (mx != kNegInf) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const float e = l[nt] == kNegInf ? 0.f : __expf(l[nt] - mx);
          se += e;
          we += l[nt] == kNegInf ? 0.f : e * l[nt];
        }
      }
#pragma unroll
      for (int o = 1; o < 16; o <<= 1) {
        se += __shfl_xor(se, o, 64);
        we += __shfl_xor(we, o, 64);
      }
      // the draw: arg-max of logit + gumbel noise over this row's columns in the wave
      // (noise of element (row, v): counter row * V + v of M * V, one draw over [M, V])
      float gv = kNegInf, gl = kNegInf;
      int gi = 0x7fffffff;
      if (a.part_draw && rok) {
        const uint64_t tot = (uint64_t)a.M * (uint64_t)a.V;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const float n = l[nt] == kNegInf ? kNegInf
              : l[nt] + gumbel_from_bits(random_bits(ks0, ks1, (uint64_t)row * a.V + col[nt], tot, a.variant));
          if (n > gv) {   // columns grow with nt: ties keep the lower column
            gv = n;
            gi = (int)col[nt];
            gl = l[nt];
          }
        }
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) {
          const float ov = __shfl_xor(gv, o, 64), ol = __shfl_xor(gl, o, 64);
          const int oi = __shfl_xor(gi, o, 64);
          if (ov > gv || (ov == gv && oi < gi)) {
            gv = ov;
            gi = oi;
            gl = ol;
          }
        }
      }
      if (lm == 0) {
        Stat r;
        r.mx = mx; r.idx = idx; r.sum = se; r.tgt = tgt; r.wsum = we;
        r.gv = gv; r.gi = gi; r.gl = gl;
        sRed[wave * (MT * 16) + rl] = r;
      }
    }
  __syncthreads();
  if (tid < MT * 16 && m0 + tid < a.M) {
    Stat r = sRed[tid];
#pragma unroll
    for (int w = 1; w < 4; ++w) r = merge(r, sRed[w * (MT * 16) + tid]);
    // the work-group's statistics go to its first 128-column block; its other blocks (NT = 4)
    // get the neutral element, so the merging pass and the workspace layout do not change
    constexpr int BPW = NT / 2;
#pragma unroll
    for (int k = 0; k < BPW; ++k) {
      const int64_t pb = vb * BPW + k;
      if (pb >= a.nvb) break;
      if (k == 1) {
        r.mx = kNegInf; r.idx = 0x7fffffff; r.sum = 0.f; r.tgt = kNegInf; r.wsum = 0.f;
        r.gv = kNegInf; r.gi = 0x7fffffff; r.gl = kNegInf;
      }
      float* p = a.part + ((m0 + tid) * a.nvb + pb) * 4;
      p[0] = r.mx;
      p[1] = __int_as_float(r.idx);
      p[2] = r.sum;
      p[3] = r.tgt;
      if (a.part_ent) a.part_ent[(m0 + tid) * a.nvb + pb] = r.wsum;
      if (a.part_draw) {
        float* q = a.part_draw + ((m0 + tid) * a.nvb + pb) * 3;
        q[0] = r.gv;
        q[1] = __int_as_float(r.gi);
        q[2] = r.gl;
      }
    }
  }
}

// One wave per row merges the per-block statistics in column order.
__global__ __launch_bounds__(64) void lmhead_finish_kernel(const float* part, int64_t nvb,
                                                           int32_t* best_id, float* best_logp,
                                                           float* target_logp, float* lse_out,
                                                           const float* part_ent, float* entropy_out,
                                                           const float* part_draw, int32_t* draw_id,
                                                           float* draw_logp) {
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x;
  const float* p = part + row * nvb * 4;
  // lane l owns the contiguous block range [l*per, (l+1)*per): merges stay in column order
  const int64_t per = (nvb + 63) / 64;
  Stat r;
  r.mx = kNegInf; r.idx = 0x7fffffff; r.sum = 0.f; r.tgt = kNegInf; r.wsum = 0.f;
  r.gv = kNegInf; r.gi = 0x7fffffff; r.gl = kNegInf;
  for (int64_t c = lane * per; c < min(nvb, (lane + 1) * per); ++c) {
    Stat b;
    b.mx = p[c * 4]; b.idx = __float_as_int(p[c * 4 + 1]); b.sum = p[c * 4 + 2]; b.tgt = p[c * 4 + 3];
    b.wsum = part_ent ? part_ent[row * nvb + c] : 0.f;
    b.gv = kNegInf; b.gi = 0x7fffffff; b.gl = kNegInf;
    if (part_draw) {
      const float* q = part_draw + (row * nvb + c) * 3;
      b.gv = q[0]; b.gi = __float_as_int(q[1]); b.gl = q[2];
    }
    r = merge(r, b);
  }
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    Stat b;
    b.mx = __shfl_xor(r.mx, o, 64);
    b.idx = __shfl_xor(r.idx, o, 64);
    b.sum = __shfl_xor(r.sum, o, 64);
    b.tgt = __shfl_xor(r.tgt, o, 64);
    b.wsum = __shfl_xor(r.wsum, o, 64);
    b.gv = __shfl_xor(r.gv, o, 64);
    b.gi = __shfl_xor(r.gi, o, 64);
    b.gl = __shfl_xor(r.gl, o, 64);
    r = (lane & o) ? merge(b, r) : merge(r, b);  // the lower lane holds the lower columns
  }
  if (lane == 0) {
    const float lse = r.mx + logf(r.sum);
    if (best_id) best_id[row] = r.idx;
    if (best_logp) best_logp[row] = r.mx - lse;
    if (target_logp) target_logp[row] = r.tgt - lse;
    if (lse_out) lse_out[row] = lse;
    if (entropy_out) entropy_out[row] = lse - r.wsum / r.sum;  // -sum p log p
    if (draw_id) draw_id[row] = r.gi;
    if (draw_logp) draw_logp[row] = r.gl - lse;
  }
}

template <class Kern>
int raise_lds_limit(Kern kern, size_t bytes) {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) {
    tnx_set_error("cannot raise dynamic LDS limit: %s", hipGetErrorString(e));
    return TNX_ELAUNCH;
  }
  return TNX_OK;
}

template <int MT, bool DENSE>
int launch_lmhead(hipStream_t st, const LHArgs& a) {
  constexpr int NT = 2;
  static std::once_flag once;
  static int attr_rc = TNX_OK;
  constexpr size_t kLds = DENSE ? 2 * (size_t)MT * 16 * A_LD * sizeof(uint16_t) : tile_smem_bytes(MT);
  static_assert(kLds >= 4 * (size_t)MT * 16 * sizeof(Stat), "the statistics exchange reuses the activation buffers");
  std::call_once(once, [] { attr_rc = raise_lds_limit(&lmhead_kernel<MT, NT, DENSE>, kLds); });
  if (attr_rc) return attr_rc;
  dim3 grid((unsigned)cdiv(a.nvb, NT / 2), (unsigned)cdiv(a.M, MT * 16));
  hipLaunchKernelGGL((lmhead_kernel<MT, NT, DENSE>), grid, dim3(256), kLds, st, a);
  TNX_CHECK_LAUNCH("lmhead");
  return TNX_OK;
}

}  // namespace

extern "C" int64_t tnx_lmhead_nblocks(int64_t V) { return cdiv(V, 128); }

extern "C" int tnx_lmhead_logp(void* stream, const tnx_lmhead_desc* d) {
  TNX_REQUIRE(d, "lmhead: null descriptor");
  TNX_REQUIRE(d->M > 0 && d->D > 0 && d->V > 0, "lmhead: bad shape");
  TNX_REQUIRE(d->D % KTILE == 0 && d->V % 16 == 0, "lmhead: D %% 128 and V %% 16 must be 0 (D=%lld V=%lld)",
              (long long)d->D, (long long)d->V);
  TNX_REQUIRE(d->M <= 65535LL * 128, "lmhead: too many rows in one call");
  TNX_REQUIRE(d->x && d->part, "lmhead: null pointer");
  TNX_REQUIRE((uint64_t)(d->M + 128) * (uint64_t)d->D * 2 < (1ull << 32) &&
                  (uint64_t)d->V * (uint64_t)d->D * 2 < (1ull << 32),
              "lmhead: x and the head weights must stay below 4 GiB each (32-bit buffer offsets)");
  TNX_REQUIRE(d->w_bf16 || (d->codes && d->scales), "lmhead: no head weights");
  if (!d->w_bf16) {
    int rc = tnx_qw_sizes(d->D, d->V, d->group, nullptr, nullptr);
    if (rc) return rc;
    TNX_REQUIRE(d->qtype == TNX_Q_INT4 || d->qtype == TNX_Q_NF4, "lmhead: bad qtype");
  }
  if (d->lora_rank > 0)
    TNX_REQUIRE(d->lora_rank % 32 == 0 && d->t && d->lora_b && d->t_ld % 8 == 0, "lmhead: bad LoRA arguments");
  LHArgs a;
  a.M = d->M; a.D = d->D; a.V = d->V; a.x = d->x; a.w_bf16 = d->w_bf16; a.codes = d->codes;
  a.scales = d->scales; a.group = d->group; a.qtype = d->qtype; a.lora_rank = d->lora_rank;
  a.t = d->t; a.t_ld = d->t_ld; a.lora_b = d->lora_b; a.lora_scale = d->lora_scale;
  a.temperature = d->temperature == 0.f ? 1.0f : d->temperature;
  a.forbidden = d->forbidden; a.n_forbidden = d->forbidden ? d->n_forbidden : 0;
  a.targets = d->targets; a.part = d->part; a.nvb = tnx_lmhead_nblocks(d->V);
  a.logits_out = d->logits_out;
  TNX_REQUIRE(!d->entropy || d->part_entropy, "lmhead: entropy needs the part_entropy workspace [M, n_vblocks]");
  a.part_ent = d->entropy ? d->part_entropy : nullptr;
  a.part_draw = nullptr; a.key0 = a.key1 = 0; a.variant = 0; a.step_ptr = nullptr;
  a.logits_fp32 = d->logits_fp32 != 0;
  if (d->draw_id) {
    TNX_REQUIRE(d->part_draw && d->draw_step_ptr, "lmhead: the draw needs the part_draw workspace [M, n_vblocks, 3] and a step pointer");
    TNX_REQUIRE(d->draw_rng_variant == 0 || d->draw_rng_variant == 1, "lmhead: rng_variant must be 0 or 1");
    TNX_REQUIRE(d->temperature > 0.f, "lmhead: the draw needs a positive temperature");
    a.part_draw = d->part_draw; a.key0 = d->draw_key0; a.key1 = d->draw_key1; a.variant = d->draw_rng_variant;
    a.step_ptr = d->draw_step_ptr;
  }
  hipStream_t st = as_stream(stream);
  int rc;
  const bool dense = d->w_bf16 != nullptr;
  // many rows on a quantised head (per-token log-probabilities at training scale): the
  // 128 x 256 GEMM kernel with a statistics epilogue, when the request is one it covers
  rc = tnx_internal_wide_head(st, d, a.temperature, a.nvb, a.part_ent);
  if (rc == 1) {
    if (d->M <= 16) rc = dense ? launch_lmhead<1, true>(st, a) : launch_lmhead<1, false>(st, a);
    else if (d->M <= 32) rc = dense ? launch_lmhead<2, true>(st, a) : launch_lmhead<2, false>(st, a);
    else if (d->M <= 64) rc = dense ? launch_lmhead<4, true>(st, a) : launch_lmhead<4, false>(st, a);
    else rc = dense ? launch_lmhead<8, true>(st, a) : launch_lmhead<8, false>(st, a);
  }
  if (rc) return rc;
  hipLaunchKernelGGL(lmhead_finish_kernel, dim3((unsigned)d->M), dim3(64), 0, st, a.part, a.nvb,
                     d->best_id, d->best_logp, d->target_logp, d->lse, a.part_ent, d->entropy, a.part_draw,
                     d->draw_id, d->draw_logp);
  TNX_CHECK_LAUNCH("lmhead_finish");
  return TNX_OK;
}
