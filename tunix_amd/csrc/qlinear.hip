// Quantized (int4 / NF4, group scales) skinny GEMM fused with the rank-r LoRA delta, the MoE
// grouped variant, the LoRA down-projection, the QW packer and its inverse.  The main loop is
// in gemm_tile.h.
#include <string.h>

#include <mutex>

#include "gemm_tile.h"
#include "rng.h"

namespace {

struct QLArgs {
  int64_t M, K, N;
  int group, qtype;
  const uint16_t* x;
  const uint32_t* codes;
  const uint16_t* scales;
  int lora_rank, lora_nseg;
  int64_t lora_seg_end[4];
  int lora_seg_toff[4];
  int64_t t_ld;
  const uint16_t* t;
  const uint16_t* lora_b;
  float lora_scale;
  int epilogue;
  const uint16_t* residual;
  void* y;
  int split_k;
  float* ws;
  int ktiles_per_split;
  // grouped (MoE) mode: blockIdx.x = expert; rows are routes sorted by expert
  const int32_t* offsets;
  const int32_t* sorted_route;
  int x_div;
  int n_experts;
  int64_t codes_stride, scales_stride;  // per-expert strides in elements
  // fused down-projection of the next linear's adapter (*_MUL epilogue of qgemm128)
  const uint16_t* next_a_t;
  int next_rank;
  float* next_tpart;
  // optional: the weights converted once into the many-row kernel's fragments (tnx_qw_expand)
  const uint16_t* w_pre;
};
// Second argument of the 128 x 256 kernel: with `part` set it reduces its tile to lm_head
// statistics instead of storing it.
struct WideHead {
  float* part;               // [M, nvb, 4]: max, first arg-max, sum of exp, target logit
  float* part_ent;           // optional [M, nvb]: sum of exp(l - max) * l
  const int32_t* targets;    // optional [M]
  int64_t nvb;               // 128-column blocks of the vocabulary
  float temperature;
  float* logits_out;         // optional fp32 [M, N]: the raw logits (the staged bf16 values), or null
  // optional whole-vocabulary categorical draw (Gumbel-max with jax.random's bit stream): per
  // (row, block) the best logit + noise, its id and its logit, as lmhead_kernel leaves them
  float* part_draw;          // [M, nvb, 3], or null
  uint32_t key0, key1;
  int variant;
  const int32_t* step_ptr;
  int64_t rows_total;        // M of the whole call: the noise of element (row, v) is number row * V + v of M * V
};

__device__ __forceinline__ float silu_bf16(float g) {
  // jax.nn.silu = x * sigmoid(x) as two bf16 HLO ops.
  float s = rbf(1.0f / (1.0f + __expf(-g)));
  return rbf(g * s);
}
__device__ __forceinline__ float gelu_tanh_bf16(float g) {
  const float k0 = 0.7978845608028654f, k1 = 0.044715f;
  float inner = k0 * (g + k1 * g * g * g);
  return rbf(0.5f * g * (1.0f + tanhf(inner)));
}

// Epilogue shared by the plain and the grouped kernel.  `out_row(r)` maps a tile row to the
// output row (identity, or the route id in grouped mode).
template <int MT, int NT, class RowMap>
__device__ __forceinline__ void store_tile(const QLArgs& a, int64_t m0, int64_t m_end,
                                           int64_t ntile0, int64_t ntiles, f32x4 (&acc)[MT][NT],
                                           RowMap out_row) {
  const int lane = threadIdx.x & 63, lm = lane & 15, lq = lane >> 4;
  if (a.split_k > 1) {  // partial tile of this k split; tnx_splitk_finish sums the splits and applies the epilogue
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      if (ntile0 + nt >= ntiles) continue;
      const int64_t col = (ntile0 + nt) * 16 + lm;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int64_t row = m0 + mt * 16 + lq * 4 + i;
          if (row < m_end)
            a.ws[((int64_t)blockIdx.z * a.M + out_row(row)) * a.N + col] = acc[mt][nt][i];
        }
    }
    return;
  }
  if (a.epilogue == TNX_EPI_SILU_MUL || a.epilogue == TNX_EPI_GELU_MUL) {
    if constexpr (NT % 2 == 0) {
      uint16_t* y = reinterpret_cast<uint16_t*>(a.y);
      const int64_t ldy = a.N / 2;
#pragma unroll
      for (int p = 0; p < NT / 2; ++p) {
        if (ntile0 + 2 * p >= ntiles) continue;
        const int64_t col = ((ntile0 + 2 * p) / 2) * 16 + lm;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int64_t row = m0 + mt * 16 + lq * 4 + i;
            if (row >= m_end) continue;
            const float g = rbf(acc[mt][2 * p][i]);
            const float u = rbf(acc[mt][2 * p + 1][i]);
            const float act = a.epilogue == TNX_EPI_SILU_MUL ? silu_bf16(g) : gelu_tanh_bf16(g);
            y[out_row(row) * ldy + col] = f2bf(rbf(act) * u);
          }
      }
    }
    return;
  }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    if (ntile0 + nt >= ntiles) continue;
    const int64_t col = (ntile0 + nt) * 16 + lm;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t row = m0 + mt * 16 + lq * 4 + i;
        if (row >= m_end) continue;
        const float v = acc[mt][nt][i];
        const int64_t o = out_row(row) * a.N + col;
        if (a.epilogue == TNX_EPI_F32) {
          reinterpret_cast<float*>(a.y)[o] = v;
        } else if (a.epilogue == TNX_EPI_RESIDUAL) {
          reinterpret_cast<uint16_t*>(a.y)[o] = f2bf(rbf(v) + bf2f(a.residual[o]));
        } else {
          reinterpret_cast<uint16_t*>(a.y)[o] = f2bf(v);
        }
      }
  }
}

// Grouped GEMM over routed tokens: blockIdx.x = expert, blockIdx.z = 16*MT-row block inside
// the expert's route list.  Rows are gathered through sorted_route; outputs are indexed by
// route.
template <int MT, int NT>
__global__ __launch_bounds__(256) void moe_gmm_kernel(const QLArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  uint16_t* sA = reinterpret_cast<uint16_t*>(smem);
  uint32_t* sLut = tile_lut(smem, MT);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int e = blockIdx.x;
  const int r_begin = a.offsets[e], r_end = a.offsets[e + 1];
  const int64_t m0 = (int64_t)blockIdx.z * (MT * 16);
  if (m0 >= r_end - r_begin) return;
  const int64_t ntile0 = ((int64_t)blockIdx.y * 4 + wave) * NT;

  build_lut(sLut, a.qtype, tid, 256);
  const uint32_t* lut_lane = sLut + (lane & (TNX_LUT_COPIES - 1));

  TileSrc s;
  s.M = r_end - r_begin; s.K = a.K; s.x = a.x; s.row_index = a.sorted_route + r_begin;
  s.row_div = a.x_div; s.x_rows = a.M / a.x_div; s.w_bf16 = nullptr;
  s.codes = a.codes + (int64_t)e * a.codes_stride; s.scales = a.scales + (int64_t)e * a.scales_stride;
  s.group = a.group; s.qtype = a.qtype; s.ntiles = a.N / 16; s.lora_rank = 0; s.t = nullptr;
  s.t_ld = 0; s.lora_b = nullptr; s.lora_scale = 0.f;

  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) zero_acc(acc[mt][nt]);
  tile_mainloop<MT, NT, false>(s, m0, ntile0, 0, (int)(a.K / KTILE), sA, lut_lane, acc);
  const int32_t* routes = s.row_index;
  store_tile<MT, NT>(a, m0, s.M, ntile0, s.ntiles, acc,
                     [routes](int64_t r) { return (int64_t)routes[r]; });
}

}  // namespace
#include "qgemm128.h"
#include "qgemm_wide.h"
#include "moe_gmm16.h"
namespace {

// y = epi(sum of the split_k partial tiles, added in split order).  One thread per output
// element; the fixed summation order makes split-k results reproducible run to run.
__global__ void splitk_finish_kernel(const QLArgs a) {
  const bool mul = a.epilogue == TNX_EPI_SILU_MUL || a.epilogue == TNX_EPI_GELU_MUL;
  const int64_t ncol = mul ? a.N / 2 : a.N;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= a.M * ncol) return;
  const int64_t row = idx / ncol, c = idx % ncol;
  const int64_t plane = a.M * a.N;
  if (mul) {
    const int64_t cg = (c / 16) * 32 + (c % 16);
    const float* pg = a.ws + row * a.N + cg;
    float g = 0.f, u = 0.f;
    for (int z = 0; z < a.split_k; ++z) {
      g += pg[z * plane];
      u += pg[z * plane + 16];
    }
    g = rbf(g);
    u = rbf(u);
    const float act = a.epilogue == TNX_EPI_SILU_MUL ? silu_bf16(g) : gelu_tanh_bf16(g);
    reinterpret_cast<uint16_t*>(a.y)[idx] = f2bf(act * u);
    return;
  }
  float v = 0.f;
  for (int z = 0; z < a.split_k; ++z) v += a.ws[z * plane + idx];
  if (a.epilogue == TNX_EPI_F32)
    reinterpret_cast<float*>(a.y)[idx] = v;
  else if (a.epilogue == TNX_EPI_RESIDUAL)
    reinterpret_cast<uint16_t*>(a.y)[idx] = f2bf(rbf(v) + bf2f(a.residual[idx]));
  else
    reinterpret_cast<uint16_t*>(a.y)[idx] = f2bf(v);
}

// t[M,R] = bf16(x . A): one tm x tn output tile (tm, tn <= 16) per work-group, K split over
// 8 waves.  The operands are loaded straight into the MFMA layout (every lane of a quarter-wave
// its own row), which a compute unit serves one lane at a time, a few tens of GB/s: the op is
// bound by the bytes one work-group must read, (tm + tn) rows of K elements, and for decode-sized
// M the host picks tiles smaller than the 16 x 16 MFMA shape (unused rows and columns are zero
// operands) to spread the reads over every compute unit.  (The kernel for K not a multiple of
// 64; otherwise lora_down_lds_kernel below.)
// The contraction may visit k in any order as long as both operands agree, so each lane takes
// 16 consecutive elements per 64-wide step (two MFMAs): the four lanes of a row cover one whole
// 128-byte line.
__global__ __launch_bounds__(512) void lora_down_kernel(const uint16_t* x, int64_t M, int64_t K,
                                                        const uint16_t* a_t, int R, uint16_t* t,
                                                        int64_t t_ld, int tm, int tn) {
  __shared__ float red[8][64][4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lm = lane & 15, lq = lane >> 4;
  const int64_t m0 = (int64_t)blockIdx.x * tm;
  const int n0 = blockIdx.y * tn;
  const int64_t row = m0 + lm;
  const bool a_on = lm < tm && row < M, b_on = lm < tn && n0 + lm < R;
  const uint16_t* xr = x + (a_on ? row : 0) * K + lq * 16;
  const uint16_t* ar = a_t + (int64_t)(b_on ? n0 + lm : 0) * K + lq * 16;
  f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
  const int ksteps = (int)((K + 63) / 64);
#pragma unroll 8
  for (int ks = wave; ks < ksteps; ks += 8) {
    u32x4 a0 = u32x4{0, 0, 0, 0}, a1 = a0, b0 = a0, b1 = a0;
    const bool k_on = (int64_t)ks * 64 + lq * 16 < K;
    if (a_on && k_on) {
      a0 = *reinterpret_cast<const u32x4*>(xr + (int64_t)ks * 64);
      a1 = *reinterpret_cast<const u32x4*>(xr + (int64_t)ks * 64 + 8);
    }
    if (b_on && k_on) {
      b0 = *reinterpret_cast<const u32x4*>(ar + (int64_t)ks * 64);
      b1 = *reinterpret_cast<const u32x4*>(ar + (int64_t)ks * 64 + 8);
    }
    acc = mfma16(a0, b0, acc);
    acc = mfma16(a1, b1, acc);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) red[wave][lane][i] = acc[i];
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float s = 0.f;
#pragma unroll
      for (int w = 0; w < 8; ++w) s += red[w][lane][i];
      const int mi = lq * 4 + i;
      if (mi < tm && m0 + mi < M && b_on) t[(m0 + mi) * t_ld + n0 + lm] = f2bf(s);
    }
  }
}

// The same product with the operand rows taken through LDS.  A load that hands every lane of a
// quarter-wave a different row (the MFMA operand layout: lane l holds row l % 16) is served one
// lane at a time, ≈ 37 GB/s per compute unit however the data is cached; rows fetched as whole
// kilobytes (a wave's 64 lanes on 1 KB of one row, straight into LDS) come at three times that.
// The tm + tn rows of the tile are laid out one after the other (row stride `row_bytes`, K * 2
// rounded up to 1 KB; 16-byte chunks XOR-swizzled by the row so that the fragment reads of 16
// rows hit 16 bank groups), then every wave multiplies its eighth of the k-steps out of LDS.
// Rows longer than LDS holds are taken in pieces of `kc` elements (a multiple of 512), one after
// the other.  Launched when K is a multiple of 64; the wave sums reuse the tile's LDS.
__global__ __launch_bounds__(512) void lora_down_lds_kernel(const uint16_t* x, int64_t M, int64_t K,
                                                            const uint16_t* a_t, int R, uint16_t* t,
                                                            int64_t t_ld, int tm, int tn, uint32_t row_bytes, int kc) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int lm = lane & 15, lq = lane >> 4;
  const int64_t m0 = (int64_t)blockIdx.x * tm;
  const int n0 = blockIdx.y * tn;
  const uint32_t lds0 = lds_addr(smem);
  // rows past M / R lie beyond the resource and arrive as zeros
  const int64_t xrows = min((int64_t)tm, M - m0);
  const int arows = min(tn, R - n0);
  const u32x4 rx = raw_rsrc(x + m0 * K, (uint64_t)xrows * K * 2);
  const u32x4 ra = raw_rsrc(a_t + (int64_t)n0 * K, (uint64_t)arows * K * 2);
  const int per_row = (int)(row_bytes / 1024u);
  // operand rows of this lane: tile rows the output does not have are clamped (their products
  // are never stored)
  const unsigned char* ra_lds = smem + (uint32_t)min(lm, tm - 1) * row_bytes;
  const unsigned char* rb_lds = smem + (uint32_t)(tm + min(lm, tn - 1)) * row_bytes;
  auto ld = [](const unsigned char* p, uint32_t chunk) { return *reinterpret_cast<const u32x4*>(p + chunk * 16u); };
  const uint32_t sa = (uint32_t)(min(lm, tm - 1) & 15), sb = (uint32_t)((tm + min(lm, tn - 1)) & 15);
  f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int64_t k0 = 0; k0 < K; k0 += kc) {
    if (k0 > 0) __syncthreads();   // every wave is done with the piece before
    // this wave's kilobytes: q = wave, wave + 8, ... of the (row, kilobyte) pairs, walked without a
    // division (per_row is a run-time value: an integer division per request, some forty scalar
    // instructions, stretched the issue of the 20 requests over longer than they take to arrive)
    int lrow = 0, blk = wave;                                   // row of the LDS tile, kilobyte of the row
    while (blk >= per_row) { blk -= per_row; ++lrow; }
    while (lrow < tm + tn) {
      const bool is_x = lrow < tm;
      const int row = is_x ? lrow : lrow - tm;
      // lane j fills chunk 64 blk + j and fetches for it chunk 64 blk + (j ^ (row % 16))
      const uint32_t voff = ((uint32_t)row * (uint32_t)K + (uint32_t)k0) * 2u + (uint32_t)blk * 1024u +
                            (uint32_t)(lane ^ (lrow & 15)) * 16u;
      // chunks past the row's K elements: beyond the resource for the last row, otherwise the next
      // row's first bytes; no fragment read touches them
      dma16(lds0 + (uint32_t)lrow * row_bytes + (uint32_t)blk * 1024u, is_x ? rx : ra, voff, 0);
      blk += 8;
      while (blk >= per_row) { blk -= per_row; ++lrow; }
    }
    tnx_wait_vm(0);
    __syncthreads();
    const int ksteps = (int)(min((int64_t)kc, K - k0) / 64);
#pragma unroll 4
    for (int ks = wave; ks < ksteps; ks += 8) {
      const uint32_t c0 = (uint32_t)(ks * 8 + lq * 2);            // this lane's two 16-byte chunks of the step
      const u32x4 a0 = ld(ra_lds, c0 ^ sa), a1 = ld(ra_lds, (c0 + 1) ^ sa);
      const u32x4 b0 = ld(rb_lds, c0 ^ sb), b1 = ld(rb_lds, (c0 + 1) ^ sb);
      acc = mfma16(a0, b0, acc);
      acc = mfma16(a1, b1, acc);
    }
  }
  __syncthreads();   // every wave is done with the tile: its first 8 KB take the wave sums
  float* red = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int i = 0; i < 4; ++i) red[(wave * 64 + lane) * 4 + i] = acc[i];
  __syncthreads();
  if (wave == 0) {
    const bool b_on = lm < tn && n0 + lm < R;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < 8; ++w) sum += red[(w * 64 + lane) * 4 + i];
      const int mi = lq * 4 + i;
      if (mi < tm && m0 + mi < M && b_on) t[(m0 + mi) * t_ld + n0 + lm] = f2bf(sum);
    }
  }
}

// t[M, :R] = bf16(sum of fragment planes).  A plane holds, per (row tile, column tile, lane), the
// four rows 4*(lane/16)+i of column lane%16 of a 16 x 16 tile, exactly as the MFMA that produced
// it laid them out.  One work-group sums 8 consecutive lanes' values (128 bytes of every plane):
// 32 thread groups take every 32nd plane each, then the 32 partial sums are added in order.
__global__ __launch_bounds__(256) void lora_reduce_kernel(const float* tpart, int64_t M, int64_t ncb, int R,
                                                          uint16_t* t, int64_t t_ld) {
  __shared__ f32x4 red[32][8];
  const int g = threadIdx.x & 7, sl = threadIdx.x >> 3;
  const int q = blockIdx.x * 8 + g;           // (row tile * 4 + column tile) * 64 + lane
  const int lane = q & 63, n = (q >> 6) & 3, mt = q >> 8;
  const int64_t mb = blockIdx.y;
  if (n * 16 >= R) return;                     // same for the whole work-group
  const float* p = tpart + mb * ncb * 8192 + (int64_t)q * 4;
  // A thread's planes (every 32nd) are requested eight at a time before the first is added: one
  // memory round trip per eight instead of one per plane (a loop of load-then-add waits for each
  // plane in turn, and the planes come from memory).  Planes past the last are clamped loads
  // whose values are not added; the order of the additions is the planes' order.
  f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int64_t cb0 = sl; cb0 < ncb; cb0 += 256) {
    f32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const f32x4*>(p + min(cb0 + 32 * u, ncb - 1) * 8192);
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (cb0 + 32 * u < ncb) s += v[u];
  }
  red[sl][g] = s;
  __syncthreads();
  if (sl != 0) return;
#pragma unroll 8
  for (int k = 1; k < 32; ++k) s += red[k][g];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t row = mb * 128 + mt * 16 + (lane >> 4) * 4 + i;
    if (row < M) t[row * t_ld + n * 16 + (lane & 15)] = f2bf(s[i]);
  }
}

// ---- QW packer ---------------------------------------------------------------------------
__device__ __forceinline__ int64_t packed_col(int64_t c, int64_t N, int interleave2) {
  if (!interleave2) return c;
  const int64_t half = N / 2;
  const int64_t h = c / half, cc = c % half;
  return (cc / 16) * 32 + h * 16 + (cc % 16);
}

// One thread per (group of `group` consecutive k, source column).
__global__ void quantize_pack_kernel(const void* w, int w_is_f32, int64_t K, int64_t N, int group,
                                     int qtype, int interleave2, float int4_bound, uint32_t* codes,
                                     uint16_t* scales) {
  const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t g = blockIdx.y;
  if (c >= N) return;
  const int64_t k0 = g * group;
  auto ld = [&](int64_t k) -> float {
    return w_is_f32 ? reinterpret_cast<const float*>(w)[k * N + c]
                    : bf2f(reinterpret_cast<const uint16_t*>(w)[k * N + c]);
  };
  float amax = 0.f;
  for (int i = 0; i < group; ++i) amax = fmaxf(amax, fabsf(ld(k0 + i)));
  const uint16_t sbits = f2bf(qtype == TNX_Q_NF4 ? amax : amax / int4_bound);
  const float s = bf2f(sbits);
  const int64_t pc = packed_col(c, N, interleave2);
  const int64_t nt = pc / 16, lm = pc % 16;
  const int64_t ktiles = K / KTILE;
  const int spt = scales_per_tile(group), slot_w = KTILE / spt;
  // scales: [nt][kt][16][spt]; a group wider than a slot repeats its scale in every slot.
  for (int64_t k = k0; k < k0 + group; k += slot_w) {
    const int64_t kt = k / KTILE;
    const int si = (int)((k % KTILE) / slot_w);
    scales[((nt * ktiles + kt) * 16 + lm) * spt + si] = sbits;
  }
  for (int i0 = 0; i0 < group; i0 += 8) {
    uint32_t word = 0;
    for (int i = 0; i < 8; ++i) {
      const float v = ld(k0 + i0 + i);
      int code;
      if (qtype == TNX_Q_NF4) {
        code = 7;
        if (s != 0.f) {
          const float xn = v / s;
          code = 0;
          for (int e = 0; e < 15; ++e)
            code += xn > 0.5f * (kNf4Levels[e] + kNf4Levels[e + 1]) ? 1 : 0;
        }
      } else {
        code = 8;
        if (s != 0.f) {
          float q = rintf(v / s);
          q = fminf(fmaxf(q, -8.f), 7.f);
          code = (int)q + 8;
        }
      }
      word |= (uint32_t)code << (4 * i);
    }
    const int64_t k = k0 + i0;
    const int64_t kt = k / KTILE;
    const int j = (int)((k % KTILE) / 32), lq = (int)((k % 32) / 8);
    codes[((nt * ktiles + kt) * 64 + lq * 16 + lm) * 4 + j] = word;
  }
}

__global__ void qw_dequant_kernel(const uint32_t* codes, const uint16_t* scales, int64_t K,
                                  int64_t N, int group, int qtype, int interleave2, float* out) {
  const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t k = blockIdx.y;
  if (c >= N) return;
  const int64_t pc = packed_col(c, N, interleave2);
  const int64_t nt = pc / 16, lm = pc % 16, ktiles = K / KTILE, kt = k / KTILE;
  const int spt = scales_per_tile(group);
  const int si = (int)((k % KTILE) / (KTILE / spt));
  const int j = (int)((k % KTILE) / 32), lq = (int)((k % 32) / 8), i = (int)(k % 8);
  const uint32_t word = codes[((nt * ktiles + kt) * 64 + lq * 16 + lm) * 4 + j];
  const float s = bf2f(scales[((nt * ktiles + kt) * 16 + lm) * spt + si]);
  out[k * N + c] = rbf(rbf(code_level(qtype, (word >> (4 * i)) & 15)) * s);
}

// The converted copy for the many-row kernel: block (column tile of 256, k-tile) = 64 KB =
// [wave 4][column group 2][slab 8][lane 64] x 16 bytes, a lane's eight bf16 being the weights
// bf16(bf16(level) * scale) of packed column 64 wave + 32 group + lane % 32 of the tile at
// k = 128 kt + 16 slab + 8 (lane / 32) .. + 7: the A fragment of one 32x32x16 MFMA.  Columns past N
// are zeros.  One thread per 16 bytes.
__global__ __launch_bounds__(256) void qw_expand_kernel(const uint32_t* codes, const uint16_t* scales, int64_t K,
                                                         int64_t N, int group, int qtype, u32x4* out) {
  const int ntile = blockIdx.x, kt = blockIdx.y, ktiles = (int)(K / KTILE);
  const int wn = threadIdx.x >> 6, lane = threadIdx.x & 63, l32 = lane & 31, lh = lane >> 5;
  const int spt = scales_per_tile(group);
  for (int cg = 0; cg < 2; ++cg) {
    const int64_t nt16 = (int64_t)ntile * 16 + wn * 4 + 2 * cg + (l32 >> 4);
    const int c16 = l32 & 15;
    const bool live = nt16 < N / 16;
    const int64_t tile = (live ? nt16 : 0) * ktiles + kt;
    for (int u = 0; u < 8; ++u) {
      const int g8 = 2 * u + lh;                       // the 8-deep k group: k = 8 g8 = 8 q + 32 j
      const uint32_t w = codes[(tile * 64 + (g8 & 3) * 16 + c16) * 4 + (g8 >> 2)];
      const float sv = bf2f(scales[(tile * 16 + c16) * spt + (16 * u) / (KTILE / spt)]);
      u32x4 r;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const uint32_t byte = (w >> (8 * b)) & 255u;
        r[b] = pack2bf(rbf(code_level(qtype, byte & 15)) * sv, rbf(code_level(qtype, byte >> 4)) * sv);
      }
      if (!live) r = u32x4{0, 0, 0, 0};
      out[((((int64_t)ntile * ktiles + kt) * 4 + wn) * 2 + cg) * 512 + u * 64 + lane] = r;
    }
  }
}

// The same layout from a dense bf16 matrix w[N][K] (an unquantised or tied lm_head): a permutation.
__global__ __launch_bounds__(256) void dense_expand_kernel(const uint16_t* w, int64_t K, int64_t N, u32x4* out) {
  const int ntile = blockIdx.x, kt = blockIdx.y, ktiles = (int)(K / KTILE);
  const int wn = threadIdx.x >> 6, lane = threadIdx.x & 63, l32 = lane & 31, lh = lane >> 5;
  for (int cg = 0; cg < 2; ++cg) {
    const int64_t col = (int64_t)ntile * 256 + wn * 64 + cg * 32 + l32;
    for (int u = 0; u < 8; ++u) {
      u32x4 r = u32x4{0, 0, 0, 0};
      if (col < N) r = *reinterpret_cast<const u32x4*>(w + col * K + (int64_t)kt * KTILE + u * 16 + lh * 8);
      out[((((int64_t)ntile * ktiles + kt) * 4 + wn) * 2 + cg) * 512 + u * 64 + lane] = r;
    }
  }
}

QLArgs to_args(const tnx_qlinear_desc* d) {
  QLArgs a;
  a.M = d->M; a.K = d->K; a.N = d->N; a.group = d->group; a.qtype = d->qtype;
  a.x = d->x; a.codes = d->codes; a.scales = d->scales;
  a.lora_rank = d->lora_rank; a.lora_nseg = d->lora_nseg;
  for (int i = 0; i < 4; ++i) { a.lora_seg_end[i] = d->lora_seg_end[i]; a.lora_seg_toff[i] = d->lora_seg_toff[i]; }
  a.t_ld = d->t_ld; a.t = d->t; a.lora_b = d->lora_b; a.lora_scale = d->lora_scale;
  a.epilogue = d->epilogue; a.residual = d->residual; a.y = d->y;
  a.split_k = d->split_k < 1 ? 1 : d->split_k; a.ws = d->ws;
  const int ktiles = (int)(d->K / KTILE);
  a.ktiles_per_split = (ktiles + a.split_k - 1) / a.split_k;
  a.offsets = nullptr; a.sorted_route = nullptr; a.x_div = 1; a.codes_stride = 0; a.scales_stride = 0;
  a.next_a_t = d->next_a_t; a.next_rank = d->next_rank; a.next_tpart = d->next_tpart;
  a.w_pre = d->w_expanded;
  return a;
}

int check_desc(const tnx_qlinear_desc* d) {
  TNX_REQUIRE(d != nullptr, "qlinear: null descriptor");
  TNX_REQUIRE(d->M > 0 && d->K > 0 && d->N > 0, "qlinear: M,K,N must be positive");
  TNX_REQUIRE(d->K % KTILE == 0, "qlinear: K=%lld must be a multiple of 128", (long long)d->K);
  TNX_REQUIRE(d->N % 16 == 0, "qlinear: N=%lld must be a multiple of 16", (long long)d->N);
  TNX_REQUIRE(d->group >= 32 && d->group % 32 == 0 &&
                  (d->group <= KTILE ? KTILE % d->group == 0 : d->group % KTILE == 0) &&
                  d->K % d->group == 0,
              "qlinear: unsupported group size %d for K=%lld", d->group, (long long)d->K);
  TNX_REQUIRE(d->qtype == TNX_Q_INT4 || d->qtype == TNX_Q_NF4, "qlinear: bad qtype %d", d->qtype);
  TNX_REQUIRE(d->x && d->codes && d->scales && d->y, "qlinear: null pointer");
  TNX_REQUIRE((uint64_t)(d->M + 128) * (uint64_t)d->K * 2 < (1ull << 32) &&
                  (uint64_t)d->K * (uint64_t)d->N / 2 < (1ull << 32),
              "qlinear: x and the codes must stay below 4 GiB each (32-bit buffer offsets)");
  TNX_REQUIRE(d->epilogue >= TNX_EPI_STORE && d->epilogue <= TNX_EPI_F32, "qlinear: bad epilogue");
  if (d->epilogue == TNX_EPI_RESIDUAL) TNX_REQUIRE(d->residual, "qlinear: residual is null");
  if (d->epilogue == TNX_EPI_SILU_MUL || d->epilogue == TNX_EPI_GELU_MUL)
    TNX_REQUIRE(d->N % 32 == 0, "qlinear: *_MUL epilogue needs N %% 32 == 0");
  if (d->lora_rank > 0) {
    TNX_REQUIRE(d->lora_rank % 32 == 0, "qlinear: lora_rank %d must be a multiple of 32 (zero-pad)",
                d->lora_rank);
    TNX_REQUIRE(d->t && d->lora_b, "qlinear: LoRA pointers are null");
    TNX_REQUIRE(d->lora_nseg == -1 || (d->lora_nseg >= 1 && d->lora_nseg <= 4),
                "qlinear: lora_nseg must be -1 (interleaved pair) or 1..4");
    TNX_REQUIRE(d->t_ld % 8 == 0, "qlinear: t_ld must be a multiple of 8");
    for (int s = 0; s < d->lora_nseg; ++s)
      TNX_REQUIRE(d->lora_seg_end[s] % 16 == 0 && d->lora_seg_toff[s] % 8 == 0,
                  "qlinear: LoRA segment %d misaligned", s);
  }
  if (d->split_k > 1) TNX_REQUIRE(d->ws, "qlinear: split_k > 1 needs a workspace");
  if (d->next_tpart) {
    TNX_REQUIRE(d->epilogue == TNX_EPI_SILU_MUL || d->epilogue == TNX_EPI_GELU_MUL,
                "qlinear: next_tpart needs a *_MUL epilogue");
    TNX_REQUIRE(d->split_k <= 1, "qlinear: next_tpart needs split_k == 1");
    TNX_REQUIRE(d->next_a_t && d->next_rank > 0 && d->next_rank % 16 == 0 && d->next_rank <= 64,
                "qlinear: next_rank must be a multiple of 16 and <= 64 (got %d)", d->next_rank);
    TNX_REQUIRE((d->N / 2) % 8 == 0, "qlinear: next_tpart needs N/2 %% 8 == 0");
  }
  return TNX_OK;
}

// The same product for many rows (prefill, per-token logps): 16 * MT rows x 64 adapter columns
// per work-group through the dense main loop (x staged in LDS, A^T fragments straight from
// global memory, MFMA), instead of tiles sized for a decode batch that re-read K-long rows per
// tile.
template <int MT>
__global__ __launch_bounds__(256) void lora_down_rows_kernel(const uint16_t* x, int64_t M, int64_t K,
                                                             const uint16_t* a_t, int R, uint16_t* t,
                                                             int64_t t_ld) {
  extern __shared__ __align__(16) unsigned char smem[];
  uint16_t* sA = reinterpret_cast<uint16_t*>(smem);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, lm = lane & 15, lq = lane >> 4;
  TileSrc s;
  s.M = M; s.K = K; s.x = x; s.row_index = nullptr; s.row_div = 1; s.x_rows = M;
  s.w_bf16 = a_t; s.codes = nullptr; s.scales = nullptr; s.group = 0; s.qtype = 0;
  s.ntiles = R / 16; s.lora_rank = 0; s.t = nullptr; s.t_ld = 0; s.lora_b = nullptr; s.lora_scale = 0.f;
  const int64_t m0 = (int64_t)blockIdx.x * (16 * MT);
  const int64_t ntile0 = (int64_t)blockIdx.y * 4 + wave;
  f32x4 acc[MT][1];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) zero_acc(acc[mt][0]);
  tile_mainloop<MT, 1, true>(s, m0, ntile0, 0, (int)(K / KTILE), sA, nullptr, acc);
  if (ntile0 >= s.ntiles) return;
  const int64_t col = ntile0 * 16 + lm;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t row = m0 + mt * 16 + lq * 4 + i;
      if (row < M) t[row * t_ld + col] = f2bf(acc[mt][0][i]);
    }
}

// The same product with both operands requested straight into LDS (`buffer_load ... lds`, whole
// 256-byte rows of a k-tile, chunks XOR-swizzled by the row as in the GEMM's activation tiles).
// A work-group of four waves takes 16 MT rows x 64 NG adapter columns -- all of the adapter's
// columns, so that x is read once -- a wave the 16-column tile `wave` of every 64-column group;
// NS k-tiles in LDS, one computed and the others in flight.  The kernel above reads the adapter's
// fragments from global memory in the MFMA operand layout, which the memory path serves a few
// lanes at a time, and re-reads x once per 64 columns; here every byte arrives as part of a whole
// kilobyte.
template <int MT, int NG, int NS>
__global__ __launch_bounds__(256) void lora_down_rows_lds_kernel(const uint16_t* x, int64_t M, int64_t K,
                                                                 const uint16_t* a_t, int R, uint16_t* t,
                                                                 int64_t t_ld) {
  constexpr uint32_t kXBytes = MT * 16 * 256, kStage = kXBytes + NG * 64 * 256;
  constexpr int kReq = MT + 4 * NG;   // requests per thread and k-tile
  extern __shared__ __align__(16) unsigned char smem[];
  const uint32_t lds0 = lds_addr(smem);
  const int tid = threadIdx.x, lane = tid & 63, lm = lane & 15, lq = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t m0 = (int64_t)blockIdx.x * (16 * MT);
  // rows past M / R lie beyond the resource and arrive as zeros
  const u32x4 rx = raw_rsrc(x + m0 * K, (uint64_t)min((int64_t)(16 * MT), M - m0) * K * 2);
  const u32x4 ra = raw_rsrc(a_t, (uint64_t)R * K * 2);
  // thread t requests, per 16-row group of a tile, the 16 bytes that land at byte 16 t of the group:
  // row t / 16, and of that row's 256 bytes the chunk (t % 16) ^ (row % 16)
  const uint32_t rrow = (uint32_t)(tid >> 4);
  const uint32_t req = rrow * (uint32_t)K * 2u + (((uint32_t)(tid & 15) ^ rrow) * 16u);
  const uint32_t grp = 16u * (uint32_t)K * 2u;   // 16 rows further
  const int ktiles = (int)(K / KTILE);
  auto request = [&](int kt) {
    const uint32_t base = lds0 + (uint32_t)(kt % NS) * kStage + (uint32_t)wave * 1024u;
    const int ko = kt * (KTILE * 2);
#pragma unroll
    for (int c = 0; c < MT; ++c) dma16(base + (uint32_t)c * 4096u, rx, req + (uint32_t)c * grp, ko);
#pragma unroll
    for (int c = 0; c < 4 * NG; ++c) dma16(base + kXBytes + (uint32_t)c * 4096u, ra, req + (uint32_t)c * grp, ko);
  };
  f32x4 acc[NG][MT];
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[g][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int u = 0; u < NS - 1; ++u)
    if (u < ktiles) request(u);
  for (int kt = 0; kt < ktiles; ++kt) {
    // this thread's share of k-tile kt has landed (behind it: the requests of the tiles after it) ...
    if (kt + NS - 2 < ktiles) tnx_wait_vm(kReq * (NS - 2));
    else tnx_wait_vm(0);
    __syncthreads();   // ... and everyone's; every wave is done with k-tile kt - 1, whose stage is refilled
    if (kt + NS - 1 < ktiles) request(kt + NS - 1);
    const uint32_t base = lds0 + (uint32_t)(kt % NS) * kStage;
#pragma unroll
    for (int j = 0; j < 4; ++j) {   // 32 k per step: this lane's chunk 4 j + l / 16 of row l % 16
      const uint32_t ch = ((uint32_t)(4 * j + lq) ^ (uint32_t)lm) * 16u;
      u32x4 a[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) a[mt] = lds_ld128(base + (uint32_t)((mt * 16 + lm) * 256) + ch);
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const u32x4 b = lds_ld128(base + kXBytes + (uint32_t)((g * 64 + wave * 16 + lm) * 256) + ch);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[g][mt] = mfma16(a[mt], b, acc[g][mt]);
      }
    }
  }
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const int col = g * 64 + wave * 16 + lm;
    if (col >= R) continue;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t row = m0 + mt * 16 + lq * 4 + i;
        if (row < M) t[row * t_ld + col] = f2bf(acc[g][mt][i]);
      }
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

// qgemm128_kernel and qgemm_wide_kernel address LDS absolutely (their table sits at LDS address 0),
// which holds as long as they have no static LDS: checked here, once per instantiation, before the
// first launch.
template <class Kern>
int prepare_qgemm128(Kern kern, size_t bytes) {
  hipFuncAttributes attr;
  hipError_t e = hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(kern));
  if (e != hipSuccess) {
    tnx_set_error("quantised GEMM: cannot read the kernel's attributes: %s", hipGetErrorString(e));
    return TNX_ELAUNCH;
  }
  if (attr.sharedSizeBytes != 0) {
    tnx_set_error("quantised GEMM: built with %zu bytes of static LDS; its absolute LDS addressing needs none",
                  (size_t)attr.sharedSizeBytes);
    return TNX_ENOSYS;
  }
  return raise_lds_limit(kern, bytes);
}

template <int NT, int SPT, int MT, bool INT4>
int launch_qgemm128_as(hipStream_t st, const QLArgs& a) {
  static std::once_flag once;
  static int attr_rc = TNX_OK;
  constexpr size_t kSmem = big_smem_bytes(NT, MT);
  std::call_once(once, [] { attr_rc = prepare_qgemm128(&qgemm128_kernel<NT, SPT, MT, INT4>, kSmem); });
  if (attr_rc) return attr_rc;
  dim3 grid((unsigned)cdiv(a.M, 16 * MT), (unsigned)cdiv(a.N, 64 * NT), (unsigned)a.split_k);
  hipLaunchKernelGGL((qgemm128_kernel<NT, SPT, MT, INT4>), grid, dim3(512), kSmem, st, a);
  TNX_CHECK_LAUNCH("qgemm128");
  return TNX_OK;
}

// integer codes take the instantiation that converts them without the table
template <int NT, int SPT, int MT>
int launch_qgemm128(hipStream_t st, const QLArgs& a) {
  return a.qtype == TNX_Q_INT4 ? launch_qgemm128_as<NT, SPT, MT, true>(st, a) : launch_qgemm128_as<NT, SPT, MT, false>(st, a);
}

template <int SPT, int MODE>
int launch_qgemm_wide_as(hipStream_t st, const QLArgs& a, const WideHead& h) {
  static std::once_flag once;
  static int attr_rc = TNX_OK;
  constexpr size_t kSmem = MODE == kWidePre ? kWidePreSmemBytes : kWideSmemBytes;
  std::call_once(once, [] { attr_rc = prepare_qgemm128(&qgemm_wide_kernel<SPT, false, MODE>, kSmem); });
  if (attr_rc) return attr_rc;
  const unsigned wgs = (unsigned)(cdiv(a.M, kWideRows) * cdiv(a.N, kWideCols));
  hipLaunchKernelGGL((qgemm_wide_kernel<SPT, false, MODE>), dim3(wgs), dim3(256), kSmem, st, a, h);
  TNX_CHECK_LAUNCH("qgemm_wide");
  return TNX_OK;
}

template <int SPT>
int launch_qgemm_wide(hipStream_t st, const QLArgs& a, const WideHead& h = WideHead{nullptr, nullptr, nullptr, 0, 1.0f, nullptr}) {
  // the converted copy when the caller keeps one (its block offsets are 32-bit); else integer
  // codes take the instantiation that converts them without the table
  if (a.w_pre && cdiv(a.N, kWideCols) * (a.K / KTILE) * 65536 < (int64_t)1 << 31)
    return launch_qgemm_wide_as<2, kWidePre>(st, a, h);
  TNX_REQUIRE(a.codes && a.scales, "quantised GEMM: no packed weights and no usable expanded copy");
  return a.qtype == TNX_Q_INT4 ? launch_qgemm_wide_as<SPT, kWideInt4>(st, a, h)
                               : launch_qgemm_wide_as<SPT, kWideTable>(st, a, h);
}

// The grouped form: the grid covers an upper bound of the 128-row blocks, sum over the experts
// of ceil(rows / 128) <= n_routes / 128 + E (work-groups past the last block exit at once).
template <int SPT, bool INT4>
int launch_qgemm_wide_grouped_as(hipStream_t st, const QLArgs& a) {
  static std::once_flag once;
  static int attr_rc = TNX_OK;
  std::call_once(once, [] { attr_rc = prepare_qgemm128(&qgemm_wide_kernel<SPT, true, INT4 ? kWideInt4 : kWideTable>, kWideSmemBytes); });
  if (attr_rc) return attr_rc;
  const int64_t blocks = a.M / kWideRows + a.n_experts;
  const unsigned wgs = (unsigned)(blocks * cdiv(a.N, kWideCols));
  hipLaunchKernelGGL((qgemm_wide_kernel<SPT, true, INT4 ? kWideInt4 : kWideTable>), dim3(wgs), dim3(256), kWideSmemBytes, st, a,
                     WideHead{nullptr, nullptr, nullptr, 0, 1.0f, nullptr});
  TNX_CHECK_LAUNCH("qgemm_wide_grouped");
  return TNX_OK;
}

template <int SPT>
int launch_qgemm_wide_grouped(hipStream_t st, const QLArgs& a) {
  return a.qtype == TNX_Q_INT4 ? launch_qgemm_wide_grouped_as<SPT, true>(st, a) : launch_qgemm_wide_grouped_as<SPT, false>(st, a);
}

// Shapes the 128 x 256 kernel takes: enough rows to fill the device with its tiles, no k split,
// a bf16 output whose rows can be written in 16-byte chunks, and an adapter (if any) of rank
// <= 64 none of whose 256-column windows touches more than two segments.
bool wide_shape(const QLArgs& a, int64_t min_rows = 512) {
  if (a.split_k > 1 || a.next_tpart || a.M < min_rows) return false;
  if (cdiv(a.M, kWideRows) * cdiv(a.N, kWideCols) < 256) return false;
  const bool mul = a.epilogue == TNX_EPI_SILU_MUL || a.epilogue == TNX_EPI_GELU_MUL;
  if (!mul && a.epilogue != TNX_EPI_STORE && a.epilogue != TNX_EPI_RESIDUAL) return false;
  if ((mul ? a.N / 2 : a.N) % 8 != 0 || ((uintptr_t)a.y & 15) != 0) return false;
  if (a.epilogue == TNX_EPI_RESIDUAL && ((uintptr_t)a.residual & 15) != 0) return false;
  if (a.lora_rank > 0) {
    if (a.lora_rank > 64 || a.lora_rank % 8 != 0) return false;
    if (a.lora_nseg > 2) {
      for (int64_t c0 = 0; c0 < a.N; c0 += kWideCols) {
        const int64_t c1 = std::min<int64_t>(c0 + kWideCols, a.N) - 1;
        int first = 0, last = 0;
        for (int i = 0; i < a.lora_nseg - 1; ++i) {
          first += c0 >= a.lora_seg_end[i];
          last += c1 >= a.lora_seg_end[i];
        }
        if (last - first > 1) return false;
      }
    }
  }
  return true;
}

template <int MT, int NT>
int launch_moe(hipStream_t st, const QLArgs& a, int E, int64_t max_rows) {
  static std::once_flag once;
  static int attr_rc = TNX_OK;
  std::call_once(once, [] { attr_rc = raise_lds_limit(&moe_gmm_kernel<MT, NT>, tile_smem_bytes(MT)); });
  if (attr_rc) return attr_rc;
  dim3 grid((unsigned)E, (unsigned)cdiv(a.N, 64 * NT), (unsigned)cdiv(max_rows, MT * 16));
  hipLaunchKernelGGL((moe_gmm_kernel<MT, NT>), grid, dim3(256), tile_smem_bytes(MT), st, a);
  TNX_CHECK_LAUNCH("moe_gmm");
  return TNX_OK;
}

// The streaming kernel for expert batches of at most 16 rows per block: one persistent
// work-group per compute unit.  It addresses an expert bank and the output with 32-bit offsets,
// pairs adjacent column tiles, needs at most as many (expert, row block) pairs as it has waves
// and parks at most kMoeMaxRun finished tile pairs per wave in LDS.
bool moe16_shape(const QLArgs& a, int E, size_t codes_bytes, size_t scales_bytes, int cus) {
  if (a.N % 32 != 0 || cus <= 0) return false;
  if ((uint64_t)E * codes_bytes >= (1ull << 32) || (uint64_t)E * scales_bytes >= (1ull << 32)) return false;
  const int64_t max_blocks = (int64_t)E + a.M / 16;
  const int64_t waves = (int64_t)cus * kMoeWaves;
  if (max_blocks > waves || max_blocks * (a.N / 32) > waves * kMoeMaxRun) return false;
  const bool mul = a.epilogue == TNX_EPI_SILU_MUL;
  if ((uint64_t)a.M * (uint64_t)(mul ? a.N / 2 : a.N) * 2 >= (1ull << 32) || ((uintptr_t)a.y & 15) != 0) return false;
  return moe16_smem_bytes(E, a.M) <= 160 * 1024;
}

template <bool MUL, int SPT, bool INT4>
int launch_moe16_t(hipStream_t st, const QLArgs& a, int E, int cus) {
  static std::once_flag once;
  static int attr_rc = TNX_OK;
  std::call_once(once, [] { attr_rc = prepare_qgemm128(&moe_gmm16_kernel<MUL, SPT, INT4>, 160 * 1024); });
  if (attr_rc) return attr_rc;
  hipLaunchKernelGGL((moe_gmm16_kernel<MUL, SPT, INT4>), dim3((unsigned)cus), dim3(kMoeWaves * 64), moe16_smem_bytes(E, a.M), st, a, E);
  TNX_CHECK_LAUNCH("moe_gmm16");
  return TNX_OK;
}

template <bool MUL, int SPT>
int launch_moe16_q(hipStream_t st, const QLArgs& a, int E, int cus) {
  return a.qtype == TNX_Q_INT4 ? launch_moe16_t<MUL, SPT, true>(st, a, E, cus) : launch_moe16_t<MUL, SPT, false>(st, a, E, cus);
}

int launch_moe16(hipStream_t st, const QLArgs& a, int E, int cus) {
  const bool mul = a.epilogue == TNX_EPI_SILU_MUL;
  if (scales_per_tile(a.group) == 2)
    return mul ? launch_moe16_q<true, 2>(st, a, E, cus) : launch_moe16_q<false, 2>(st, a, E, cus);
  return mul ? launch_moe16_q<true, 4>(st, a, E, cus) : launch_moe16_q<false, 4>(st, a, E, cus);
}

int device_cus() {
  static int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    return n;
  }();
  return cus;
}

}  // namespace

extern "C" int tnx_qw_sizes(int64_t K, int64_t N, int group, size_t* codes_bytes,
                            size_t* scales_bytes) {
  TNX_REQUIRE(K > 0 && N > 0 && K % KTILE == 0 && N % 16 == 0,
              "qw_sizes: K %% 128 and N %% 16 must be 0 (K=%lld N=%lld)", (long long)K, (long long)N);
  TNX_REQUIRE(group >= 32 && group % 32 == 0 && K % group == 0 &&
                  (group <= KTILE ? KTILE % group == 0 : group % KTILE == 0),
              "qw_sizes: unsupported group %d", group);
  const int spt = scales_per_tile(group);
  if (codes_bytes) *codes_bytes = (size_t)(K * N / 2);
  // 16 bytes of tail padding: kernels read a lane's scales as one 8-byte word
  if (scales_bytes) *scales_bytes = (size_t)((N / 16) * (K / KTILE) * spt * 16 * 2) + 16;
  return TNX_OK;
}

extern "C" int tnx_quantize_pack(void* stream, const void* w, int w_is_f32, int64_t K, int64_t N,
                                 int group, int qtype, int interleave2, float int4_bound, uint32_t* codes,
                                 uint16_t* scales) {
  int rc = tnx_qw_sizes(K, N, group, nullptr, nullptr);
  if (rc) return rc;
  TNX_REQUIRE(w && codes && scales, "quantize_pack: null pointer");
  TNX_REQUIRE(qtype == TNX_Q_INT4 || qtype == TNX_Q_NF4, "quantize_pack: bad qtype %d", qtype);
  if (interleave2) TNX_REQUIRE(N % 32 == 0, "quantize_pack: interleave2 needs N %% 32 == 0");
  dim3 grid((unsigned)cdiv(N, 128), (unsigned)(K / group));
  if (!(int4_bound > 0.f)) int4_bound = 7.0f;
  hipLaunchKernelGGL(quantize_pack_kernel, grid, dim3(128), 0, as_stream(stream), w, w_is_f32, K, N,
                     group, qtype, interleave2, int4_bound, codes, scales);
  TNX_CHECK_LAUNCH("quantize_pack");
  return TNX_OK;
}

extern "C" int tnx_qw_dequant(void* stream, const uint32_t* codes, const uint16_t* scales,
                              int64_t K, int64_t N, int group, int qtype, int interleave2,
                              float* w_out) {
  int rc = tnx_qw_sizes(K, N, group, nullptr, nullptr);
  if (rc) return rc;
  TNX_REQUIRE(codes && scales && w_out, "qw_dequant: null pointer");
  dim3 grid((unsigned)cdiv(N, 128), (unsigned)K);
  hipLaunchKernelGGL(qw_dequant_kernel, grid, dim3(128), 0, as_stream(stream), codes, scales, K, N,
                     group, qtype, interleave2, w_out);
  TNX_CHECK_LAUNCH("qw_dequant");
  return TNX_OK;
}

extern "C" size_t tnx_qw_expanded_bytes(int64_t K, int64_t N) {
  if (K <= 0 || N <= 0 || K % KTILE != 0) return 0;
  return (size_t)(cdiv(N, kWideCols) * (K / KTILE)) * 65536u;
}

extern "C" int tnx_qw_expand(void* stream, const uint32_t* codes, const uint16_t* scales, int64_t K, int64_t N,
                             int group, int qtype, uint16_t* w_expanded) {
  int rc = tnx_qw_sizes(K, N, group, nullptr, nullptr);
  if (rc) return rc;
  TNX_REQUIRE(codes && scales && w_expanded, "qw_expand: null pointer");
  TNX_REQUIRE(qtype == TNX_Q_INT4 || qtype == TNX_Q_NF4, "qw_expand: bad qtype %d", qtype);
  TNX_REQUIRE(((uintptr_t)w_expanded & 15) == 0, "qw_expand: the output must be 16-byte aligned");
  TNX_REQUIRE(K / KTILE <= 65535, "qw_expand: K=%lld too large", (long long)K);
  dim3 grid((unsigned)cdiv(N, kWideCols), (unsigned)(K / KTILE));
  hipLaunchKernelGGL(qw_expand_kernel, grid, dim3(256), 0, as_stream(stream), codes, scales, K, N, group, qtype,
                     reinterpret_cast<u32x4*>(w_expanded));
  TNX_CHECK_LAUNCH("qw_expand");
  return TNX_OK;
}

extern "C" int tnx_dense_expand(void* stream, const uint16_t* w_bf16, int64_t K, int64_t N, uint16_t* w_expanded) {
  TNX_REQUIRE(w_bf16 && w_expanded, "dense_expand: null pointer");
  TNX_REQUIRE(K > 0 && N > 0 && K % KTILE == 0 && K / KTILE <= 65535, "dense_expand: K=%lld must be a positive multiple of 128", (long long)K);
  TNX_REQUIRE(((uintptr_t)w_expanded & 15) == 0 && ((uintptr_t)w_bf16 & 15) == 0, "dense_expand: pointers must be 16-byte aligned");
  dim3 grid((unsigned)cdiv(N, kWideCols), (unsigned)(K / KTILE));
  hipLaunchKernelGGL(dense_expand_kernel, grid, dim3(256), 0, as_stream(stream), w_bf16, K, N,
                     reinterpret_cast<u32x4*>(w_expanded));
  TNX_CHECK_LAUNCH("dense_expand");
  return TNX_OK;
}

extern "C" int tnx_qlinear_lora(void* stream, const tnx_qlinear_desc* d) {
  int rc = check_desc(d);
  if (rc) return rc;
  const QLArgs a = to_args(d);
  hipStream_t st = as_stream(stream);
  // One kernel for every row count: 128 x 128 work-group tiles at 65+ rows, 16 / 32 / 64 rows for
  // decode batches that small (the weight stream and its dequantisation are the same; MFMA,
  // fragment and activation work shrink with the rows).  The 256-column variant (NT = 4) is not
  // dispatched: its accumulators need AGPRs, and the compiler wraps loops over AGPR accumulators
  // in register copies that cost more than the halved LDS traffic gains.
  const bool s2 = scales_per_tile(a.group) == 2;
  if (wide_shape(a)) return s2 ? launch_qgemm_wide<2>(st, a) : launch_qgemm_wide<4>(st, a);
  if (a.M <= 16) return s2 ? launch_qgemm128<2, 2, 1>(st, a) : launch_qgemm128<2, 4, 1>(st, a);
  if (a.M <= 32) return s2 ? launch_qgemm128<2, 2, 2>(st, a) : launch_qgemm128<2, 4, 2>(st, a);
  if (a.M <= 64) return s2 ? launch_qgemm128<2, 2, 4>(st, a) : launch_qgemm128<2, 4, 4>(st, a);
  return s2 ? launch_qgemm128<2, 2, 8>(st, a) : launch_qgemm128<2, 4, 8>(st, a);
}

// The quantised lm_head over many rows on the 128 x 256 kernel: per 128-column block statistics
// in the layout lmhead_kernel writes, so the same finishing kernel merges them.  Returns 1 when
// the shape is not one the kernel takes (the caller then uses its own kernel), 0 when launched.
int tnx_internal_wide_head(hipStream_t st, const tnx_lmhead_desc* d, float temperature, int64_t nvb,
                           float* part_ent) {
  if (d->forbidden || d->logits_fp32) return 1;   // (its tile is staged in bf16)
  // a dense head comes here only through its expanded copy (tnx_dense_expand)
  const bool dense = d->w_bf16 != nullptr;
  const bool pre_ok = d->w_expanded && d->D % KTILE == 0 &&
                      cdiv(d->V, kWideCols) * (d->D / KTILE) * 65536 < (int64_t)1 << 31;
  if (dense) {
    if (!pre_ok || d->V % 16 != 0 || d->lora_rank > 0) return 1;
  } else {
    if (d->group < 32 || d->group % 32 != 0 || (d->group <= KTILE ? KTILE % d->group != 0 : d->group % KTILE != 0) ||
        d->D % d->group != 0)
      return 1;
    if ((uint64_t)d->D * (uint64_t)d->V / 2 >= (1ull << 32)) return 1;
  }
  QLArgs a;
  memset(&a, 0, sizeof(a));
  a.M = d->M; a.K = d->D; a.N = d->V; a.group = dense ? KTILE : d->group; a.qtype = d->qtype;
  a.x = d->x; a.codes = d->codes; a.scales = d->scales;
  a.lora_rank = d->lora_rank; a.lora_nseg = 1; a.lora_seg_end[0] = d->V;
  a.t_ld = d->t_ld; a.t = d->t; a.lora_b = d->lora_b; a.lora_scale = d->lora_scale;
  a.epilogue = TNX_EPI_STORE; a.y = d->part;   // the shape test looks at a stored tile
  a.split_k = 1; a.ktiles_per_split = (int)(d->D / KTILE); a.x_div = 1;
  a.w_pre = pre_ok ? d->w_expanded : nullptr;
  // A dense head's copy is streamed at any row count: at a decode batch the launch is bound by
  // the weight stream, and this kernel re-reads the activations once per 256 columns where the
  // 128 x 128 head kernel re-reads them once per 128, as many bytes again as the weights.
  if (!wide_shape(a, dense ? 1 : 512)) return 1;
  a.y = nullptr;
  WideHead h{d->part, part_ent, d->targets, nvb, temperature, d->logits_out, nullptr, 0u, 0u, 0, nullptr, d->M};
  if (d->draw_id) {
    h.part_draw = d->part_draw; h.key0 = d->draw_key0; h.key1 = d->draw_key1; h.variant = d->draw_rng_variant;
    h.step_ptr = d->draw_step_ptr;
  }
  return scales_per_tile(a.group) == 2 ? launch_qgemm_wide<2>(st, a, h) : launch_qgemm_wide<4>(st, a, h);
}

extern "C" int tnx_splitk_finish(void* stream, const tnx_qlinear_desc* d) {
  int rc = check_desc(d);
  if (rc) return rc;
  TNX_REQUIRE(d->ws, "splitk_finish: null workspace");
  const QLArgs a = to_args(d);
  const bool mul = a.epilogue == TNX_EPI_SILU_MUL || a.epilogue == TNX_EPI_GELU_MUL;
  const int64_t n = a.M * (mul ? a.N / 2 : a.N);
  hipLaunchKernelGGL(splitk_finish_kernel, dim3((unsigned)cdiv(n, 256)), dim3(256), 0,
                     as_stream(stream), a);
  TNX_CHECK_LAUNCH("splitk_finish");
  return TNX_OK;
}

extern "C" int tnx_lora_reduce(void* stream, const float* tpart, int64_t M, int64_t n_col_blocks, int R,
                               uint16_t* t, int64_t t_ld) {
  TNX_REQUIRE(tpart && t, "lora_reduce: null pointer");
  TNX_REQUIRE(M > 0 && n_col_blocks > 0, "lora_reduce: bad shape");
  TNX_REQUIRE(R > 0 && R % 16 == 0 && R <= 64 && t_ld >= R, "lora_reduce: R=%d must be a multiple of 16, <= 64 and <= t_ld", R);
  hipLaunchKernelGGL(lora_reduce_kernel, dim3(256, (unsigned)cdiv(M, 128)), dim3(256), 0, as_stream(stream),
                     tpart, M, n_col_blocks, R, t, t_ld);
  TNX_CHECK_LAUNCH("lora_reduce");
  return TNX_OK;
}

extern "C" int tnx_lora_down(void* stream, const uint16_t* x, int64_t M, int64_t K,
                             const uint16_t* a_t, int R, uint16_t* t, int64_t t_ld) {
  TNX_REQUIRE(x && a_t && t, "lora_down: null pointer");
  TNX_REQUIRE(M > 0 && K > 0 && K % 32 == 0, "lora_down: K=%lld must be a multiple of 32", (long long)K);
  TNX_REQUIRE(R > 0 && R % 16 == 0 && t_ld >= R, "lora_down: R=%d must be a multiple of 16 and <= t_ld", R);
  if (M >= 512 && K % KTILE == 0 && (uint64_t)(M + 128) * (uint64_t)K * 2 < (1ull << 32) && R % 16 == 0 && R <= 192 &&
      (uint64_t)(R + 64) * (uint64_t)K * 2 < (1ull << 32)) {
    // many rows: both operands through LDS, all adapter columns per work-group
    auto launch = [&](auto MTc, auto NGc, auto NSc) -> int {
      constexpr int MT = decltype(MTc)::value, NG = decltype(NGc)::value, NS = decltype(NSc)::value;
      constexpr size_t kSmem = (size_t)NS * (MT * 16 * 256 + NG * 64 * 256);
      static_assert(kSmem <= 160 * 1024, "the stages fit LDS");
      static std::once_flag once;
      static int attr_rc = TNX_OK;
      std::call_once(once, [] { attr_rc = raise_lds_limit(&lora_down_rows_lds_kernel<MT, NG, NS>, kSmem); });
      if (attr_rc) return attr_rc;
      hipLaunchKernelGGL((lora_down_rows_lds_kernel<MT, NG, NS>), dim3((unsigned)cdiv(M, 16 * MT)), dim3(256), kSmem,
                         as_stream(stream), x, M, K, a_t, R, t, t_ld);
      TNX_CHECK_LAUNCH("lora_down_rows_lds");
      return TNX_OK;
    };
    // the tallest tile that still gives every compute unit a work-group; three k-tiles in LDS where
    // they fit, else two
    auto pick = [&](auto NGc) -> int {
      constexpr int NG = decltype(NGc)::value;
      using std::integral_constant;
      if (cdiv(M, 128) >= 256)
        return launch(integral_constant<int, 8>{}, NGc, integral_constant<int, (NG == 1 ? 3 : 2)>{});
      if (cdiv(M, 64) >= 256)
        return launch(integral_constant<int, 4>{}, NGc, integral_constant<int, (NG <= 2 ? 3 : 2)>{});
      return launch(integral_constant<int, 2>{}, NGc, integral_constant<int, (NG <= 2 ? 3 : 2)>{});
    };
    if (R <= 64) return pick(std::integral_constant<int, 1>{});
    if (R <= 128) return pick(std::integral_constant<int, 2>{});
    if (R <= 192) return pick(std::integral_constant<int, 3>{});
  }
  if (M >= 512 && K % KTILE == 0 && (uint64_t)(M + 128) * (uint64_t)K * 2 < (1ull << 32)) {
    // many rows: MFMA tiles of 128 rows, or of 64 / 32 where that is what it takes to fill the
    // device (32-bit buffer offsets: the activations must stay below 4 GiB)
    const int64_t cols = cdiv(R, 64);
    auto launch = [&](auto MTc) -> int {
      constexpr int MT = decltype(MTc)::value;
      constexpr size_t kSmem = 2 * (size_t)MT * 16 * A_LD * sizeof(uint16_t);
      static std::once_flag once;
      static int attr_rc = TNX_OK;
      std::call_once(once, [] { attr_rc = raise_lds_limit(&lora_down_rows_kernel<MT>, kSmem); });
      if (attr_rc) return attr_rc;
      dim3 grid((unsigned)cdiv(M, 16 * MT), (unsigned)cols);
      hipLaunchKernelGGL((lora_down_rows_kernel<MT>), grid, dim3(256), kSmem, as_stream(stream), x, M, K, a_t, R, t, t_ld);
      TNX_CHECK_LAUNCH("lora_down_rows");
      return TNX_OK;
    };
    if (cdiv(M, 128) * cols >= 192) return launch(std::integral_constant<int, 8>{});
    if (cdiv(M, 64) * cols >= 192) return launch(std::integral_constant<int, 4>{});
    return launch(std::integral_constant<int, 2>{});
  }
  // smallest tm + tn whose grid still fits the device once; 16 x 16 when nothing does
  int tm = 16, tn = 16;
  {
    static const int kTm[] = {4, 8, 16}, kTn[] = {4, 8, 12, 16};
    int best = 33;
    for (int a : kTm)
      for (int b : kTn)
        if (cdiv(M, a) * cdiv(R, b) <= 256 && a + b < best) {
          best = a + b;
          tm = a;
          tn = b;
        }
  }
  dim3 grid((unsigned)cdiv(M, tm), (unsigned)cdiv(R, tn));
  // the operand rows through LDS, whole (rows of K * 2 bytes rounded up to whole KB) or, when LDS
  // does not hold them, in pieces of kc elements (whole KB again)
  int64_t kc = K;
  if ((uint64_t)(tm + tn) * (uint64_t)cdiv(K * 2, 1024) * 1024 > 160 * 1024)
    kc = (160 * 1024 / ((tm + tn) * 2)) / 512 * 512;
  const uint64_t row_bytes = (uint64_t)cdiv(kc * 2, 1024) * 1024;
  const uint64_t lds = std::max<uint64_t>((uint64_t)(tm + tn) * row_bytes, 8192);
  if (K % 64 == 0 && kc >= 512 && lds <= 160 * 1024 && (uint64_t)(tm + 1) * (uint64_t)K * 2 < (1ull << 32)) {
    static std::once_flag once;
    static int attr_rc = TNX_OK;
    std::call_once(once, [] { attr_rc = raise_lds_limit(&lora_down_lds_kernel, 160 * 1024); });
    if (attr_rc) return attr_rc;
    hipLaunchKernelGGL(lora_down_lds_kernel, grid, dim3(512), (size_t)lds, as_stream(stream), x, M, K, a_t, R, t, t_ld,
                       tm, tn, (uint32_t)row_bytes, (int)kc);
    TNX_CHECK_LAUNCH("lora_down_lds");
    return TNX_OK;
  }
  hipLaunchKernelGGL(lora_down_kernel, grid, dim3(512), 0, as_stream(stream), x, M, K, a_t, R, t, t_ld, tm, tn);
  TNX_CHECK_LAUNCH("lora_down");
  return TNX_OK;
}

extern "C" int tnx_moe_int4_gmm(void* stream, const tnx_moe_gmm_desc* d) {
  TNX_REQUIRE(d, "moe_gmm: null descriptor");
  TNX_REQUIRE(d->n_routes > 0 && d->E > 0 && d->k > 0, "moe_gmm: bad shape");
  size_t cb = 0, sb = 0;
  int rc = tnx_qw_sizes(d->K, d->N, d->group, &cb, &sb);
  if (rc) return rc;
  TNX_REQUIRE(d->x && d->codes && d->scales && d->offsets && d->sorted_route && d->y, "moe_gmm: null pointer");
  TNX_REQUIRE(d->x_div >= 1, "moe_gmm: x_div must be >= 1");
  TNX_REQUIRE((uint64_t)(d->n_routes + 128) * (uint64_t)d->K * 2 < (1ull << 32),
              "moe_gmm: activations must stay below 4 GiB (32-bit buffer offsets)");
  TNX_REQUIRE(d->epilogue == TNX_EPI_STORE || d->epilogue == TNX_EPI_SILU_MUL, "moe_gmm: bad epilogue");
  if (d->epilogue == TNX_EPI_SILU_MUL) TNX_REQUIRE(d->N % 32 == 0, "moe_gmm: SILU_MUL needs N %% 32 == 0");
  QLArgs a;
  memset(&a, 0, sizeof(a));
  a.M = d->n_routes; a.K = d->K; a.N = d->N; a.group = d->group; a.qtype = d->qtype;
  a.x = d->x; a.codes = d->codes; a.scales = d->scales; a.epilogue = d->epilogue; a.y = d->y;
  a.split_k = 1; a.ktiles_per_split = (int)(d->K / KTILE);
  a.offsets = d->offsets; a.sorted_route = d->sorted_route; a.x_div = d->x_div;
  a.codes_stride = (int64_t)(cb / 4); a.scales_stride = (int64_t)(sb / 2);
  // Any expert can receive up to all rows (one route per token and expert): the grid covers
  // that bound and blocks past an expert's count exit at once.
  // The row tile follows the rows an expert gets on average (n_routes / E: 4 for a decode batch of
  // 64 with top-8 routing over 128 experts): the dequantisation per k-tile is the same for every
  // tile height, the MFMA, staging and LDS work is not, and two 16-row work-groups share a
  // compute unit.  An expert with more rows than one tile takes several (weights read again).
  const int64_t max_rows = d->n_routes / d->k;
  const int64_t avg_rows = cdiv(d->n_routes, (int64_t)d->E);
  hipStream_t st = as_stream(stream);
  a.n_experts = d->E;
  // Many rows per expert (a prefill, a per-token log-probability pass): the 128 x 256 tiles of
  // the many-row kernel, one expert's routes per row block.  From about 32 rows per expert on it
  // is faster than the 64-row tile kernel even with its row blocks three quarters empty (Qwen3-30B-
  // A3B shape, gate|up + down: 134 + 82 us against 152 + 102 us at 32 rows, 144 + 93 against
  // 271 + 179 us at 64; at 16 rows the 32-row tiles win, 97 + 60 against 130 + 76 us).
  const bool mul = d->epilogue == TNX_EPI_SILU_MUL;
  if (avg_rows > 24 && d->N % kWideCols == 0 && (mul ? d->N / 2 : d->N) % 8 == 0 && ((uintptr_t)d->y & 15) == 0 &&
      (uint64_t)(d->n_routes / d->x_div) * (uint64_t)d->K * 2 < 0xfffff000ull && d->n_routes % d->x_div == 0)
    return scales_per_tile(d->group) == 2 ? launch_qgemm_wide_grouped<2>(st, a) : launch_qgemm_wide_grouped<4>(st, a);
  // Up to about 12 rows per expert the streaming kernel (16-row blocks, an expert with more
  // rows streams its weights once per block) beats the 32-row tiles: 87 + 48 against 96 + 56 us
  // at 10 rows per expert, 90 + 49 against 96 + 58 us at 12, 112 + 54 against 98 + 60 us at 16.
  if (max_rows <= 16 || avg_rows <= 12) {
    const int cus = device_cus();
    if (moe16_shape(a, d->E, cb, sb, cus)) return launch_moe16(st, a, d->E, cus);
  }
  if (max_rows <= 16 || avg_rows <= 8) return launch_moe<1, 2>(st, a, d->E, max_rows);
  if (max_rows <= 32 || avg_rows <= 24) return launch_moe<2, 2>(st, a, d->E, max_rows);
  return launch_moe<4, 2>(st, a, d->E, max_rows);
}

#ifdef TNX_TIMING
// tuning aid (not part of the product build): the phase stamps of the last qgemm128 launch
extern "C" int tnx_debug_stamps(unsigned long long* out8) {
  return hipMemcpyFromSymbol(out8, HIP_SYMBOL(tnx_stamps), 8 * sizeof(unsigned long long)) == hipSuccess ? 0 : -1;
}
#endif
