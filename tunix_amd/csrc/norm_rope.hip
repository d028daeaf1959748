// Embedding gather, RMSNorm (three dtype flows), per-head q/k norm + RoPE + KV-cache write.
// All of these move a few bytes per decode step compared with the weights and the cache; they
// are written for exact dtype-flow parity and few launches, not for peak bandwidth.
#include <string.h>

#include "common.h"

namespace {

// ---- block reductions --------------------------------------------------------------------
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  if (nw == 1) return v;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
  for (int w = 0; w < nw; ++w) s += red[w];
  return s;
}

// One normalised element, given the row statistics.  `ms` is mean(x^2) (llama/qwen3: fp32 of
// fp32 squares; gemma3: bf16-rounded mean of bf16-rounded squares).
__device__ __forceinline__ float norm_elem(float x, float w, float ms, float eps, int flavor) {
  if (flavor == TNX_NORM_LLAMA) {
    // astype(w * x / rms): w*x is a bf16 product, the division is fp32.
    const float rms = sqrtf(ms + eps);
    return rbf(rbf(w * x) / rms);
  } else if (flavor == TNX_NORM_QWEN3) {
    const float rms = sqrtf(ms + eps);
    return rbf(w * (x / rms));
  } else {
    // gemma3: every op in bf16: x * rsqrt(var + eps) * (1 + scale)
    const float r = rbf(1.0f / sqrtf(rbf(ms + eps)));
    return rbf(rbf(x * r) * rbf(1.0f + w));
  }
}
__device__ __forceinline__ float sq_term(float x, int flavor) {
  return flavor == TNX_NORM_GEMMA3 ? rbf(x * x) : x * x;
}
__device__ __forceinline__ float finish_ms(float ss, float n, int flavor) {
  const float ms = ss / n;
  return flavor == TNX_NORM_GEMMA3 ? rbf(ms) : ms;
}

__global__ __launch_bounds__(256) void rmsnorm_kernel(const uint16_t* x, const uint16_t* res_pre,
                                                      uint16_t* h_out, const uint16_t* w,
                                                      const uint16_t* res_post, uint16_t* y,
                                                      int64_t D, float eps, int flavor) {
  __shared__ float red[4];
  extern __shared__ __align__(16) unsigned char smem_dyn[];
  float* hrow = reinterpret_cast<float*>(smem_dyn);  // [D]
  const int64_t row = blockIdx.x;
  const uint16_t* xr = x + row * D;
  float ss = 0.f;
  for (int64_t i = threadIdx.x; i < D; i += blockDim.x) {
    float h = bf2f(xr[i]);
    if (res_pre) h = rbf(h + bf2f(res_pre[row * D + i]));
    if (h_out) h_out[row * D + i] = f2bf(h);
    hrow[i] = h;
    ss += sq_term(h, flavor);
  }
  ss = block_sum(ss, red);
  const float ms = finish_ms(ss, (float)D, flavor);
  for (int64_t i = threadIdx.x; i < D; i += blockDim.x) {
    float v = norm_elem(hrow[i], bf2f(w[i]), ms, eps, flavor);
    if (res_post) v = rbf(v + bf2f(res_post[row * D + i]));
    y[row * D + i] = f2bf(v);
  }
}

// The same op for D % 8 == 0 (every model on the path): 16-byte loads and stores, the row stays
// in registers between the two passes (thread t owns the 8-element chunks t, t + 256, ...).
constexpr int kNormMaxChunks = 8;  // D <= 8 * 256 * 8 = 16384
__device__ __forceinline__ void unpack8(const u32x4& p, float (&f)[8]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = bflo(p[j]);
    f[2 * j + 1] = bfhi(p[j]);
  }
}
// The input row, by IN: kNormInRow -- x[row]; kNormInPlanes -- bf16(sum of the split_k fp32 partial
// planes ws[z][row][:]) of a split-k linear, added in split order: the linear's own finishing
// pass folded into the norm; kNormInRoutes -- bf16(sum_j cw[row, j] * x[row * split_k + j]) over
// the split_k routed rows of a token, j ascending: the weighted combine of an MoE layer folded
// into the norm (same arithmetic as moe_combine_vec_kernel).
constexpr int kNormInRow = 0, kNormInPlanes = 1, kNormInRoutes = 2;
template <int MAXC, int FLAVOR, int IN>
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(const uint16_t* x, const uint16_t* res_pre,
                                                          uint16_t* h_out, const uint16_t* w,
                                                          const uint16_t* res_post, uint16_t* y,
                                                          int64_t D, float eps, int /*flavor*/,
                                                          const float* ws, int split_k, int64_t plane,
                                                          const uint16_t* w2, uint16_t* y2, const uint16_t* cw) {
  constexpr bool PLANES = IN == kNormInPlanes, ROUTES = IN == kNormInRoutes;
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const int nchunks = (int)(D / 8);
  float h[MAXC][8];
  float ss = 0.f;
  // Chunks are taken two at a time with every load of the pair issued before the first sum (up
  // to eight planes per chunk at once, further planes in groups of eight): the kernel is a few
  // dependent memory round trips long, and each group of loads that waits for the previous sum
  // adds one.  The sum itself stays in split order.
#pragma unroll
  for (int c0 = 0; c0 < MAXC; c0 += 2) {
    if (c0 * 256 >= nchunks) break;   // uniform
    f32x4 p0[2][8], p1[2][8];
    u32x4 xin[2], rin[2], yin[2][8];
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      const int ch = (c0 + cc) * 256 + threadIdx.x;
      const int64_t o = row * D + (int64_t)min(ch, nchunks - 1) * 8;
      if (PLANES) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int64_t zo = (int64_t)min(u, split_k - 1) * plane + o;
          p0[cc][u] = *reinterpret_cast<const f32x4*>(ws + zo);
          p1[cc][u] = *reinterpret_cast<const f32x4*>(ws + zo + 4);
        }
      } else if (ROUTES) {
#pragma unroll
        for (int u = 0; u < 8; ++u)
          yin[cc][u] = *reinterpret_cast<const u32x4*>(
              x + (row * split_k + min(u, split_k - 1)) * D + (int64_t)min(ch, nchunks - 1) * 8);
      } else {
        xin[cc] = *reinterpret_cast<const u32x4*>(x + o);
      }
      if (res_pre) rin[cc] = *reinterpret_cast<const u32x4*>(res_pre + o);
    }
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      const int c = c0 + cc;
      const int ch = c * 256 + threadIdx.x;
      if (ch < nchunks) {
        const int64_t o = row * D + (int64_t)ch * 8;
        if (PLANES) {
#pragma unroll
          for (int j = 0; j < 8; ++j) h[c][j] = 0.f;
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (u < split_k) {
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                h[c][j] += p0[cc][u][j];
                h[c][4 + j] += p1[cc][u][j];
              }
            }
          for (int z0 = 8; z0 < split_k; z0 += 8) {   // more than eight planes: the rest in groups
            f32x4 q0[8], q1[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
              const int64_t zo = (int64_t)min(z0 + u, split_k - 1) * plane + o;
              q0[u] = *reinterpret_cast<const f32x4*>(ws + zo);
              q1[u] = *reinterpret_cast<const f32x4*>(ws + zo + 4);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
              if (z0 + u < split_k) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                  h[c][j] += q0[u][j];
                  h[c][4 + j] += q1[u][j];
                }
              }
          }
#pragma unroll
          for (int j = 0; j < 8; ++j) h[c][j] = rbf(h[c][j]);
        } else if (ROUTES) {
#pragma unroll
          for (int j = 0; j < 8; ++j) h[c][j] = 0.f;
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (u < split_k) {
              const float wt = bf2f(cw[row * split_k + u]);
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                h[c][2 * q] += wt * bflo(yin[cc][u][q]);
                h[c][2 * q + 1] += wt * bfhi(yin[cc][u][q]);
              }
            }
          for (int z0 = 8; z0 < split_k; z0 += 8) {   // more than eight routes per token: the rest in groups
            u32x4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
              v[u] = *reinterpret_cast<const u32x4*>(x + (row * split_k + min(z0 + u, split_k - 1)) * D + (int64_t)ch * 8);
#pragma unroll
            for (int u = 0; u < 8; ++u)
              if (z0 + u < split_k) {
                const float wt = bf2f(cw[row * split_k + z0 + u]);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                  h[c][2 * q] += wt * bflo(v[u][q]);
                  h[c][2 * q + 1] += wt * bfhi(v[u][q]);
                }
              }
          }
#pragma unroll
          for (int j = 0; j < 8; ++j) h[c][j] = rbf(h[c][j]);
        } else {
          unpack8(xin[cc], h[c]);
        }
        if (res_pre) {
          float r[8];
          unpack8(rin[cc], r);
#pragma unroll
          for (int j = 0; j < 8; ++j) h[c][j] = rbf(h[c][j] + r[j]);
        }
        if (h_out) {
          u32x4 q;
#pragma unroll
          for (int j = 0; j < 4; ++j) q[j] = pack2bf(h[c][2 * j], h[c][2 * j + 1]);
          *reinterpret_cast<u32x4*>(h_out + o) = q;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += sq_term(h[c][j], FLAVOR);
      }
    }
  }
  // the norm weights and the post-norm residual do not depend on the row statistics: fetch them
  // before the reduction instead of behind it
  u32x4 wpre[MAXC], rpost[MAXC];
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = c * 256 + threadIdx.x;
    if (ch < nchunks) {
      wpre[c] = *reinterpret_cast<const u32x4*>(w + (int64_t)ch * 8);
      if (res_post && res_post != h_out) rpost[c] = *reinterpret_cast<const u32x4*>(res_post + row * D + (int64_t)ch * 8);
    }
  }
  ss = block_sum(ss, red);
  const float ms = finish_ms(ss, (float)D, FLAVOR);
  float ss2 = 0.f;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = c * 256 + threadIdx.x;
    if (ch < nchunks) {
      const int64_t o = row * D + (int64_t)ch * 8;
      float wv[8], v[8];
      unpack8(wpre[c], wv);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = norm_elem(h[c][j], wv[j], ms, eps, FLAVOR);
      if (res_post) {
        float r[8];
        // (a residual that this launch itself rewrote as h_out is read back here, after the write)
        unpack8(res_post != h_out ? rpost[c] : *reinterpret_cast<const u32x4*>(res_post + o), r);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = rbf(v[j] + r[j]);
      }
      u32x4 q;
#pragma unroll
      for (int j = 0; j < 4; ++j) q[j] = pack2bf(v[2 * j], v[2 * j + 1]);
      *reinterpret_cast<u32x4*>(y + o) = q;
      if (w2) {   // the row just written is the input of a second norm: keep it, as rounded
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          h[c][j] = rbf(v[j]);
          ss2 += sq_term(h[c][j], FLAVOR);
        }
      }
    }
  }
  if (!w2) return;
  // y2 = norm(y) with its own weight, the row still in registers (same thread -> chunk map and
  // reduction order as a launch of its own would use: the results are identical)
  ss2 = block_sum(ss2, red);
  const float ms2 = finish_ms(ss2, (float)D, FLAVOR);
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = c * 256 + threadIdx.x;
    if (ch < nchunks) {
      float wv[8];
      unpack8(*reinterpret_cast<const u32x4*>(w2 + (int64_t)ch * 8), wv);
      u32x4 q;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        q[j] = pack2bf(norm_elem(h[c][2 * j], wv[2 * j], ms2, eps, FLAVOR),
                       norm_elem(h[c][2 * j + 1], wv[2 * j + 1], ms2, eps, FLAVOR));
      *reinterpret_cast<u32x4*>(y2 + row * D + (int64_t)ch * 8) = q;
    }
  }
}

// The kernel is unrolled over its chunks (256 threads x 8 elements each): instantiated for 2, 4
// and 8 chunks per thread so that the common widths (D <= 4096) run the small instance -- the
// code a wave walks through once is fetched cold at every launch.
template <int MAXC, class... Args>
void launch_rmsnorm_vec_c(hipStream_t st, int64_t M, int flavor, int in, Args... args) {
#define TNX_NORM_CASE(F)                                                                                   \
  if (in == kNormInPlanes) hipLaunchKernelGGL((rmsnorm_vec_kernel<MAXC, F, kNormInPlanes>), dim3((unsigned)M), dim3(256), 0, st, args...); \
  else if (in == kNormInRoutes) hipLaunchKernelGGL((rmsnorm_vec_kernel<MAXC, F, kNormInRoutes>), dim3((unsigned)M), dim3(256), 0, st, args...); \
  else hipLaunchKernelGGL((rmsnorm_vec_kernel<MAXC, F, kNormInRow>), dim3((unsigned)M), dim3(256), 0, st, args...)
  if (flavor == TNX_NORM_LLAMA) { TNX_NORM_CASE(TNX_NORM_LLAMA); }
  else if (flavor == TNX_NORM_QWEN3) { TNX_NORM_CASE(TNX_NORM_QWEN3); }
  else { TNX_NORM_CASE(TNX_NORM_GEMMA3); }
#undef TNX_NORM_CASE
}
template <class... Args>
void launch_rmsnorm_vec(hipStream_t st, int64_t M, int64_t D, int flavor, int in, Args... args) {
  if (D <= 8 * 256 * 2) launch_rmsnorm_vec_c<2>(st, M, flavor, in, args...);
  else if (D <= 8 * 256 * 4) launch_rmsnorm_vec_c<4>(st, M, flavor, in, args...);
  else launch_rmsnorm_vec_c<kNormMaxChunks>(st, M, flavor, in, args...);
}

__global__ void embed_kernel(const uint16_t* table, int64_t V, int64_t D, const int32_t* ids,
                             int64_t ids_ld, const int32_t* col_ptr, int64_t T, float scale_bf,
                             uint16_t* out) {
  const int64_t row = blockIdx.x;  // b*T + t
  const int64_t b = row / T, t = row % T;
  const int col = col_ptr ? *col_ptr : 0;
  int64_t id = ids[b * ids_ld + col + t];
  if (id < 0 || id >= V) id = 0;  // pad sentinels outside the vocabulary read row 0 (masked later)
  const uint16_t* src = table + id * D;
  if (D % 8 == 0) {   // 16 bytes per thread and turn
    for (int64_t i = (int64_t)threadIdx.x * 8; i < D; i += (int64_t)blockDim.x * 8) {
      u32x4 v = *reinterpret_cast<const u32x4*>(src + i);
      if (scale_bf != 1.0f) {
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = pack2bf(bflo(v[q]) * scale_bf, bfhi(v[q]) * scale_bf);
      }
      *reinterpret_cast<u32x4*>(out + row * D + i) = v;
    }
    return;
  }
  for (int64_t i = threadIdx.x; i < D; i += blockDim.x) {
    uint16_t v = src[i];
    if (scale_bf != 1.0f) v = f2bf(bf2f(v) * scale_bf);
    out[row * D + i] = v;
  }
}

struct RopeArgs {
  int64_t B, T, S;
  int Hq, Hkv, dh;
  int rope_flavor;
  float rope_scale;
  int qk_norm;
  float norm_eps;
  const uint16_t* q_norm_w;
  const uint16_t* k_norm_w;
  float q_prescale_bf;
  const uint16_t* qkv;
  const int32_t* positions;
  int64_t pos_ld;
  const int32_t* col_ptr;
  const float* timescale;
  uint16_t* q_out;
  uint16_t* kcache;
  uint16_t* vcache;
  const float* ws;   // split-k partial planes of the qkv linear instead of qkv, or null
  int split_k;
};

// grid (B*T, Hq + 2*Hkv); max(64, dh/2) threads: thread i < dh/2 owns elements i and i + dh/2
// of one head; the other threads only take part in the reductions.
__global__ void rope_kernel(const RopeArgs a) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const int64_t b = row / a.T, t = row % a.T;
  const int head = blockIdx.y;
  const int half = a.dh / 2, i = threadIdx.x;
  const bool live = i < half;
  const int col = *a.col_ptr;
  const int ld = (a.Hq + 2 * a.Hkv) * a.dh;
  const int64_t src_off = row * ld + (int64_t)head * a.dh;
  // element e of this head: from the finished linear output, or as the linear's own finishing
  // pass would produce it, bf16(sum of the split-k planes in split order)
  auto src_at = [&](int e) -> float {
    if (a.ws == nullptr) return bf2f(a.qkv[src_off + e]);
    const int64_t plane = a.B * a.T * (int64_t)ld;
    float v = 0.f;
    for (int z0 = 0; z0 < a.split_k; z0 += 8) {  // eight planes' loads in flight; sum in split order
      float p[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) p[u] = a.ws[(int64_t)min(z0 + u, a.split_k - 1) * plane + src_off + e];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (z0 + u < a.split_k) v += p[u];
    }
    return rbf(v);
  };
  const int slot = (int)((col + t) % a.S);
  if (head >= a.Hq + a.Hkv) {  // V: plain copy into the cache slot
    const int hk = head - a.Hq - a.Hkv;
    uint16_t* dst = a.vcache + (((b * a.Hkv + hk) * a.S) + slot) * a.dh;
    if (live) {
      dst[i] = f2bf(src_at(i));
      dst[i + half] = f2bf(src_at(i + half));
    }
    return;
  }
  const bool is_q = head < a.Hq;
  float x1 = live ? src_at(i) : 0.f, x2 = live ? src_at(i + half) : 0.f;
  if (a.qk_norm >= 0) {
    const float ss = block_sum(sq_term(x1, a.qk_norm) + sq_term(x2, a.qk_norm), red);
    const float ms = finish_ms(ss, (float)a.dh, a.qk_norm);
    const uint16_t* w = is_q ? a.q_norm_w : a.k_norm_w;
    if (live) {
      x1 = norm_elem(x1, bf2f(w[i]), ms, a.norm_eps, a.qk_norm);
      x2 = norm_elem(x2, bf2f(w[i + half]), ms, a.norm_eps, a.qk_norm);
    }
  }
  if (!live) return;
  const float pos = (float)a.positions[b * a.pos_ld + col + t];
  float ang = __fdiv_rn(pos, a.timescale[i]);
  if (a.rope_flavor == TNX_ROPE_GEMMA3) ang = __fdiv_rn(ang, a.rope_scale);
  float sn = sinf(ang), cs = cosf(ang);
  float o1, o2;
  if (a.rope_flavor == TNX_ROPE_QWEN3) {
    sn = rbf(sn);
    cs = rbf(cs);
    o1 = rbf(rbf(x1 * cs) - rbf(x2 * sn));
    o2 = rbf(rbf(x2 * cs) + rbf(x1 * sn));
  } else {
    // fp32 products and sum, one rounding at the end (no fused multiply-add)
    o1 = rbf(__fsub_rn(__fmul_rn(x1, cs), __fmul_rn(x2, sn)));
    o2 = rbf(__fadd_rn(__fmul_rn(x2, cs), __fmul_rn(x1, sn)));
  }
  if (is_q) {
    if (a.q_prescale_bf != 0.f) {
      o1 = rbf(o1 * a.q_prescale_bf);
      o2 = rbf(o2 * a.q_prescale_bf);
    }
    uint16_t* dst = a.q_out + (row * a.Hq + head) * a.dh;
    dst[i] = f2bf(o1);
    dst[i + half] = f2bf(o2);
  } else {
    const int hk = head - a.Hq;
    uint16_t* dst = a.kcache + (((b * a.Hkv + hk) * a.S) + slot) * a.dh;
    dst[i] = f2bf(o1);
    dst[i + half] = f2bf(o2);
  }
}

// Many rows, no q / k norm (a Llama prefill or whole-sequence pass): one work-group per token row,
// 16-byte accesses, and the sine / cosine of a (row, i) computed once for all heads instead of
// once per head.  Thread (ch, h0) owns the eight pairs i = 8 ch .. + 7 of heads h0, h0 + hstep, ...;
// the arithmetic per element is rope_kernel's, so the outputs are bit-identical.
__global__ __launch_bounds__(256) void rope_rows_kernel(const RopeArgs a) {
  const int64_t row = blockIdx.x;
  const int64_t b = row / a.T, t = row % a.T;
  const int half = a.dh / 2, CH = half / 8, heads = a.Hq + 2 * a.Hkv;
  const int ch = threadIdx.x % CH, h0 = threadIdx.x / CH, hstep = 256 / CH;
  const int col = *a.col_ptr;
  const int ld = heads * a.dh;
  const int slot = (int)((col + t) % a.S);
  const int i0 = ch * 8;
  const float pos = (float)a.positions[b * a.pos_ld + col + t];
  float sn[8], cs[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float ang = __fdiv_rn(pos, a.timescale[i0 + e]);
    if (a.rope_flavor == TNX_ROPE_GEMMA3) ang = __fdiv_rn(ang, a.rope_scale);
    sn[e] = sinf(ang);
    cs[e] = cosf(ang);
    if (a.rope_flavor == TNX_ROPE_QWEN3) {
      sn[e] = rbf(sn[e]);
      cs[e] = rbf(cs[e]);
    }
  }
  for (int head = h0; head < heads; head += hstep) {
    const uint16_t* src = a.qkv + row * ld + (int64_t)head * a.dh + i0;
    const u32x4 v1 = *reinterpret_cast<const u32x4*>(src), v2 = *reinterpret_cast<const u32x4*>(src + half);
    uint16_t* dst;
    if (head >= a.Hq + a.Hkv) {   // V: plain copy into the cache slot
      dst = a.vcache + (((b * a.Hkv + (head - a.Hq - a.Hkv)) * a.S) + slot) * a.dh + i0;
      *reinterpret_cast<u32x4*>(dst) = v1;
      *reinterpret_cast<u32x4*>(dst + half) = v2;
      continue;
    }
    const bool is_q = head < a.Hq;
    u32x4 o1v, o2v;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float o1[2], o2[2];
#pragma unroll
      for (int hsel = 0; hsel < 2; ++hsel) {
        const int e = 2 * r + hsel;
        const float x1 = hsel ? bfhi(v1[r]) : bflo(v1[r]), x2 = hsel ? bfhi(v2[r]) : bflo(v2[r]);
        if (a.rope_flavor == TNX_ROPE_QWEN3) {
          o1[hsel] = rbf(rbf(x1 * cs[e]) - rbf(x2 * sn[e]));
          o2[hsel] = rbf(rbf(x2 * cs[e]) + rbf(x1 * sn[e]));
        } else {
          o1[hsel] = rbf(__fsub_rn(__fmul_rn(x1, cs[e]), __fmul_rn(x2, sn[e])));
          o2[hsel] = rbf(__fadd_rn(__fmul_rn(x2, cs[e]), __fmul_rn(x1, sn[e])));
        }
        if (is_q && a.q_prescale_bf != 0.f) {
          o1[hsel] = rbf(o1[hsel] * a.q_prescale_bf);
          o2[hsel] = rbf(o2[hsel] * a.q_prescale_bf);
        }
      }
      o1v[r] = pack2bf(o1[0], o1[1]);
      o2v[r] = pack2bf(o2[0], o2[1]);
    }
    if (is_q) dst = a.q_out + (row * a.Hq + head) * a.dh + i0;
    else dst = a.kcache + (((b * a.Hkv + (head - a.Hq)) * a.S) + slot) * a.dh + i0;
    *reinterpret_cast<u32x4*>(dst) = o1v;
    *reinterpret_cast<u32x4*>(dst + half) = o2v;
  }
}

// sin / cos of angle = position / timescale[i] for the token in column *col_ptr of every row: the
// values rope_kernel computes for the Llama rotation, once per decode step instead of per layer.
__global__ void rope_table_kernel(const int32_t* positions, int64_t pos_ld, const int32_t* col_ptr,
                                  const float* timescale, int half, float* sin_out, float* cos_out) {
  const int64_t b = blockIdx.x;
  const int i = threadIdx.x;
  if (i >= half) return;
  const float pos = (float)positions[b * pos_ld + *col_ptr];
  const float ang = __fdiv_rn(pos, timescale[i]);
  sin_out[b * half + i] = sinf(ang);
  cos_out[b * half + i] = cosf(ang);
}

float host_round_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
  memcpy(&f, &u, 4);
  return f;
}

}  // namespace

extern "C" int tnx_embed(void* stream, const uint16_t* table, int64_t V, int64_t D,
                         const int32_t* ids, int64_t ids_ld, const int32_t* col_ptr, int64_t B,
                         int64_t T, float scale, uint16_t* out) {
  TNX_REQUIRE(table && ids && out, "embed: null pointer");
  TNX_REQUIRE(V > 0 && D > 0 && B > 0 && T > 0, "embed: bad shape");
  hipLaunchKernelGGL(embed_kernel, dim3((unsigned)(B * T)), dim3(256), 0, as_stream(stream), table,
                     V, D, ids, ids_ld, col_ptr, T, host_round_bf16(scale), out);
  TNX_CHECK_LAUNCH("embed");
  return TNX_OK;
}

extern "C" int tnx_rmsnorm(void* stream, const uint16_t* x, const uint16_t* res_pre,
                           uint16_t* h_out, const uint16_t* w, const uint16_t* res_post,
                           uint16_t* y, int64_t M, int64_t D, float eps, int flavor) {
  TNX_REQUIRE(x && w && y, "rmsnorm: null pointer");
  TNX_REQUIRE(M > 0 && D > 0 && D <= 16384, "rmsnorm: D=%lld out of range (1..16384)", (long long)D);
  TNX_REQUIRE(flavor >= TNX_NORM_LLAMA && flavor <= TNX_NORM_GEMMA3, "rmsnorm: bad flavor %d", flavor);
  if (D % 8 == 0 && D <= 8 * 256 * kNormMaxChunks)
    launch_rmsnorm_vec(as_stream(stream), M, D, flavor, kNormInRow, x, res_pre, h_out, w, res_post, y, D, eps, flavor,
                       (const float*)nullptr, 0, (int64_t)0, (const uint16_t*)nullptr, (uint16_t*)nullptr,
                       (const uint16_t*)nullptr);
  else
    hipLaunchKernelGGL(rmsnorm_kernel, dim3((unsigned)M), dim3(256), (size_t)D * sizeof(float),
                       as_stream(stream), x, res_pre, h_out, w, res_post, y, D, eps, flavor);
  TNX_CHECK_LAUNCH("rmsnorm");
  return TNX_OK;
}

extern "C" int tnx_rmsnorm_splitk(void* stream, const float* ws, int split_k, const uint16_t* res_pre,
                                  uint16_t* h_out, const uint16_t* w, const uint16_t* res_post,
                                  uint16_t* y, int64_t M, int64_t D, float eps, int flavor) {
  TNX_REQUIRE(ws && w && y, "rmsnorm_splitk: null pointer");
  TNX_REQUIRE(split_k >= 1, "rmsnorm_splitk: split_k must be >= 1");
  TNX_REQUIRE(M > 0 && D > 0 && D % 8 == 0 && D <= 8 * 256 * kNormMaxChunks,
              "rmsnorm_splitk: D=%lld must be a multiple of 8 and <= 16384", (long long)D);
  TNX_REQUIRE(flavor >= TNX_NORM_LLAMA && flavor <= TNX_NORM_GEMMA3, "rmsnorm_splitk: bad flavor %d", flavor);
  launch_rmsnorm_vec(as_stream(stream), M, D, flavor, kNormInPlanes, (const uint16_t*)nullptr, res_pre, h_out, w, res_post, y,
                     D, eps, flavor, ws, split_k, (int64_t)(M * D), (const uint16_t*)nullptr, (uint16_t*)nullptr,
                     (const uint16_t*)nullptr);
  TNX_CHECK_LAUNCH("rmsnorm_splitk");
  return TNX_OK;
}

extern "C" int tnx_rmsnorm_moe_combine(void* stream, const uint16_t* y_route, const uint16_t* topk_w, int k,
                                       const uint16_t* res_pre, uint16_t* h_out, const uint16_t* w,
                                       const uint16_t* res_post, uint16_t* y, int64_t M, int64_t D, float eps,
                                       int flavor) {
  TNX_REQUIRE(y_route && topk_w && w && y, "rmsnorm_moe_combine: null pointer");
  TNX_REQUIRE(k >= 1, "rmsnorm_moe_combine: k must be >= 1");
  TNX_REQUIRE(M > 0 && D > 0 && D % 8 == 0 && D <= 8 * 256 * kNormMaxChunks,
              "rmsnorm_moe_combine: D=%lld must be a multiple of 8 and <= 16384", (long long)D);
  TNX_REQUIRE(flavor >= TNX_NORM_LLAMA && flavor <= TNX_NORM_GEMMA3, "rmsnorm_moe_combine: bad flavor %d", flavor);
  launch_rmsnorm_vec(as_stream(stream), M, D, flavor, kNormInRoutes, y_route, res_pre, h_out, w, res_post, y, D, eps, flavor,
                     (const float*)nullptr, k, (int64_t)0, (const uint16_t*)nullptr, (uint16_t*)nullptr, topk_w);
  TNX_CHECK_LAUNCH("rmsnorm_moe_combine");
  return TNX_OK;
}

extern "C" int tnx_rmsnorm_pair(void* stream, const uint16_t* x, const float* ws, int split_k,
                                const uint16_t* res_pre, uint16_t* h_out, const uint16_t* w,
                                const uint16_t* res_post, uint16_t* y, const uint16_t* w2, uint16_t* y2,
                                int64_t M, int64_t D, float eps, int flavor) {
  TNX_REQUIRE((x != nullptr) != (ws != nullptr), "rmsnorm_pair: exactly one of x and ws must be given");
  TNX_REQUIRE(w && y && w2 && y2, "rmsnorm_pair: null pointer");
  if (ws) TNX_REQUIRE(split_k >= 1, "rmsnorm_pair: split_k must be >= 1");
  TNX_REQUIRE(M > 0 && D > 0 && D % 8 == 0 && D <= 8 * 256 * kNormMaxChunks,
              "rmsnorm_pair: D=%lld must be a multiple of 8 and <= 16384", (long long)D);
  TNX_REQUIRE(flavor >= TNX_NORM_LLAMA && flavor <= TNX_NORM_GEMMA3, "rmsnorm_pair: bad flavor %d", flavor);
  launch_rmsnorm_vec(as_stream(stream), M, D, flavor, ws ? kNormInPlanes : kNormInRow, x, res_pre, h_out, w, res_post, y, D,
                     eps, flavor, ws, ws ? split_k : 0, (int64_t)(M * D), w2, y2, (const uint16_t*)nullptr);
  TNX_CHECK_LAUNCH("rmsnorm_pair");
  return TNX_OK;
}

extern "C" int tnx_rope_table(void* stream, const int32_t* positions, int64_t pos_ld, const int32_t* col_ptr,
                              int64_t B, const float* timescale, int dh, float* sin_out, float* cos_out) {
  TNX_REQUIRE(positions && col_ptr && timescale && sin_out && cos_out, "rope_table: null pointer");
  TNX_REQUIRE(B > 0 && dh % 2 == 0 && dh >= 2 && dh <= 2048, "rope_table: bad shape");
  hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)B), dim3((unsigned)(dh / 2 < 64 ? 64 : dh / 2)), 0,
                     as_stream(stream), positions, pos_ld, col_ptr, timescale, dh / 2, sin_out, cos_out);
  TNX_CHECK_LAUNCH("rope_table");
  return TNX_OK;
}

extern "C" int tnx_qknorm_rope_kvwrite(void* stream, const tnx_rope_desc* d) {
  TNX_REQUIRE(d, "rope: null descriptor");
  TNX_REQUIRE(d->B > 0 && d->T > 0 && d->S > 0, "rope: bad shape");
  TNX_REQUIRE(d->dh % 2 == 0 && d->dh >= 2 && d->dh <= 512, "rope: bad head_dim %d", d->dh);
  TNX_REQUIRE((d->qkv || d->qkv_ws) && d->positions && d->col_ptr && d->timescale && d->q_out &&
                  d->kcache && d->vcache,
              "rope: null pointer");
  if (d->qkv_ws) TNX_REQUIRE(d->split_k >= 1 && d->split_k <= 64, "rope: split_k=%d out of range", d->split_k);
  TNX_REQUIRE(d->rope_flavor >= TNX_ROPE_LLAMA && d->rope_flavor <= TNX_ROPE_GEMMA3, "rope: bad flavor");
  TNX_REQUIRE(d->qk_norm >= -1 && d->qk_norm <= TNX_NORM_GEMMA3, "rope: bad qk_norm");
  if (d->qk_norm >= 0) TNX_REQUIRE(d->q_norm_w && d->k_norm_w, "rope: qk_norm weights are null");
  if (d->rope_flavor == TNX_ROPE_GEMMA3)
    TNX_REQUIRE(d->rope_scale >= 1.0f, "rope: scale_factor must be >= 1.0, got %f", d->rope_scale);
  RopeArgs a;
  a.B = d->B; a.T = d->T; a.S = d->S; a.Hq = d->Hq; a.Hkv = d->Hkv; a.dh = d->dh;
  a.rope_flavor = d->rope_flavor; a.rope_scale = d->rope_scale; a.qk_norm = d->qk_norm;
  a.norm_eps = d->norm_eps; a.q_norm_w = d->q_norm_w; a.k_norm_w = d->k_norm_w;
  a.q_prescale_bf = d->q_prescale != 0.f ? host_round_bf16(d->q_prescale) : 0.f;
  a.qkv = d->qkv; a.positions = d->positions; a.pos_ld = d->pos_ld; a.col_ptr = d->col_ptr;
  a.timescale = d->timescale; a.q_out = d->q_out; a.kcache = d->kcache; a.vcache = d->vcache;
  a.ws = d->qkv_ws; a.split_k = d->split_k;
  // many rows of a model without q / k norm, from the finished linear output: the row kernel
  const int chunks = d->dh / 16;
  const bool aligned = (((uintptr_t)d->qkv | (uintptr_t)d->q_out | (uintptr_t)d->kcache | (uintptr_t)d->vcache) & 15) == 0;
  if (d->qk_norm < 0 && !d->qkv_ws && d->B * d->T >= 256 && d->dh % 16 == 0 && chunks <= 256 && 256 % chunks == 0 &&
      aligned) {
    hipLaunchKernelGGL(rope_rows_kernel, dim3((unsigned)(d->B * d->T)), dim3(256), 0, as_stream(stream), a);
    TNX_CHECK_LAUNCH("qknorm_rope_kvwrite (rows)");
    return TNX_OK;
  }
  dim3 grid((unsigned)(d->B * d->T), (unsigned)(d->Hq + 2 * d->Hkv));
  hipLaunchKernelGGL(rope_kernel, grid, dim3(d->dh / 2 < 64 ? 64 : d->dh / 2), 0, as_stream(stream), a);
  TNX_CHECK_LAUNCH("qknorm_rope_kvwrite");
  return TNX_OK;
}
