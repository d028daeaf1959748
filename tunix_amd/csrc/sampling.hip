// Top-k / top-p sampling from materialised fp32 logits with the threefry2x32 bit stream of
// jax.random (fold_in -> random_bits -> uniform -> gumbel -> argmax), one work-group per row.
#include <mutex>

#include "common.h"
#include "rng.h"

namespace {

constexpr int NTH = 1024;
constexpr float kNegInf = -__builtin_inff();

__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct ArgMax {
  float v;
  int i;
};
__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {  // larger value, then lower index
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

__device__ ArgMax block_argmax(ArgMax x, ArgMax* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    ArgMax y;
    y.v = __shfl_xor(x.v, o, 64);
    y.i = __shfl_xor(x.i, o, 64);
    x = better(x, y);
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = x;
  __syncthreads();
  ArgMax r = red[0];
  for (int w = 1; w < NTH / 64; ++w) r = better(r, red[w]);
  __syncthreads();
  return r;
}

__device__ float block_sum_f(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
  for (int w = 0; w < NTH / 64; ++w) s += red[w];
  __syncthreads();
  return s;
}

__global__ __launch_bounds__(NTH) void sample_topk_kernel(const float* logits, int64_t V, int k,
                                                          float top_p, uint32_t key0, uint32_t key1,
                                                          int variant, const int32_t* step_ptr,
                                                          int64_t M, float temperature,
                                                          const int32_t* forbidden, int n_forbidden,
                                                          int32_t* ids_out, float* logp_out) {
  __shared__ uint32_t hist[256];
  __shared__ float cval[NTH];
  __shared__ int cidx[NTH];
  __shared__ ArgMax red_am[NTH / 64];
  __shared__ float red_f[NTH / 64];
  __shared__ uint32_t s_sel, s_rem, s_cnt, s_base;
  __shared__ uint32_t wave_cnt[NTH / 64];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  const float* lr = logits + row * V;
  // the caller passes raw logits; sampling works on f32(logit) / temperature
  auto lg = [lr, temperature, forbidden, n_forbidden](int64_t v) {
    for (int f = 0; f < n_forbidden; ++f)
      if (forbidden[f] == (int32_t)v) return kNegInf;
    return __fdiv_rn(lr[v], temperature);
  };

  // fold_in(key, step): threefry of the key over the counter pair (0, step)
  uint32_t ks0 = 0u, ks1 = (uint32_t)(*step_ptr);
  threefry2x32(key0, key1, ks0, ks1);

  // ---- log-sum-exp of the row (for the log-probability of the drawn token) ----
  ArgMax am;
  am.v = kNegInf;
  am.i = 0x7fffffff;
  for (int64_t v = tid; v < V; v += NTH) {
    ArgMax c;
    c.v = lg(v);
    c.i = (int)v;
    am = better(am, c);
  }
  am = block_argmax(am, red_am);
  float se = 0.f;
  for (int64_t v = tid; v < V; v += NTH) se += expf(lg(v) - am.v);
  se = block_sum_f(se, red_f);
  const float lse = am.v + logf(se);

  if (k <= 0) {
    // categorical over the whole vocabulary: arg-max of logit + gumbel noise
    ArgMax g;
    g.v = kNegInf;
    g.i = 0x7fffffff;
    for (int64_t v = tid; v < V; v += NTH) {
      ArgMax c;
      c.v = lg(v) + gumbel_from_bits(random_bits(ks0, ks1, (uint64_t)(row * V + v), (uint64_t)(M * V), variant));
      c.i = (int)v;
      g = better(g, c);
    }
    g = block_argmax(g, red_am);
    if (tid == 0) {
      ids_out[row] = g.i;
      if (logp_out) logp_out[row] = lg(g.i) - lse;
    }
    return;
  }

  // ---- radix select: key of the k-th largest logit ----
  uint32_t prefix = 0, mask = 0;
  if (tid == 0) s_rem = (uint32_t)k;
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    for (int64_t v = tid; v < V; v += NTH) {
      const uint32_t kk = order_key(lg(v));
      if ((kk & mask) == prefix) atomicAdd(&hist[(kk >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (tid == 0) {
      uint32_t cum = 0, rem = s_rem;
      int b = 255;
      for (; b > 0; --b) {
        if (cum + hist[b] >= rem) break;
        cum += hist[b];
      }
      s_sel = (uint32_t)b;
      s_rem = rem - cum;
    }
    __syncthreads();
    prefix |= s_sel << shift;
    mask |= 0xffu << shift;
  }
  const uint32_t thr = prefix;
  const uint32_t r_eq = s_rem;  // how many elements equal to the threshold are taken
  if (tid == 0) {
    s_cnt = 0;
    s_base = 0;
  }
  cval[tid] = kNegInf;
  cidx[tid] = 0x7fffffff;
  __syncthreads();
  // elements above the threshold: any order (sorted below)
  for (int64_t v = tid; v < V; v += NTH) {
    const float x = lg(v);
    if (order_key(x) > thr) {
      const uint32_t p = atomicAdd(&s_cnt, 1u);
      cval[p] = x;
      cidx[p] = (int)v;
    }
  }
  __syncthreads();
  const uint32_t n_gt = s_cnt;
  // elements equal to the threshold: the r_eq lowest indices, by an ordered block scan
  for (int64_t v0 = 0; v0 < V; v0 += NTH) {
    if (s_base >= r_eq) break;
    const int64_t v = v0 + tid;
    const bool eq = v < V && order_key(lg(v)) == thr;
    const uint64_t bal = __ballot(eq);
    const int lane = tid & 63, wave = tid >> 6;
    const uint32_t before = (uint32_t)__popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) wave_cnt[wave] = (uint32_t)__popcll(bal);
    __syncthreads();
    uint32_t woff = 0, tot = 0;
    for (int w = 0; w < NTH / 64; ++w) {
      if (w < wave) woff += wave_cnt[w];
      tot += wave_cnt[w];
    }
    const uint32_t pos = s_base + woff + before;
    if (eq && pos < r_eq) {
      cval[n_gt + pos] = lg(v);
      cidx[n_gt + pos] = (int)v;
    }
    __syncthreads();
    if (tid == 0) s_base += tot;
    __syncthreads();
  }
  __syncthreads();
  // ---- bitonic sort of the candidates: descending value, ascending index ----
  for (int size = 2; size <= NTH; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      const int partner = tid ^ stride;
      if (partner > tid) {
        ArgMax a{cval[tid], cidx[tid]}, b{cval[partner], cidx[partner]};
        const bool a_first = (a.v > b.v) || (a.v == b.v && a.i < b.i);
        const bool up = (tid & size) == 0;  // this pair sorts "best first" when up
        if (up != a_first) {
          cval[tid] = b.v; cidx[tid] = b.i;
          cval[partner] = a.v; cidx[partner] = a.i;
        }
      }
      __syncthreads();
    }
  }
  // ---- softmax over the k sorted logits, top-p cut, gumbel arg-max ----
  const float mx = cval[0];
  float e = tid < k ? expf(cval[tid] - mx) : 0.f;
  const float tot = block_sum_f(e, red_f);
  __shared__ float prob[NTH];
  prob[tid] = e / tot;
  __syncthreads();
  __shared__ float excl[NTH];
  if (tid == 0) {
    float c = 0.f;
    for (int j = 0; j < k; ++j) {
      c += prob[j];
      excl[j] = c - prob[j];  // cumsum - p, as in the reference
    }
  }
  __syncthreads();
  ArgMax g;
  g.v = kNegInf;
  g.i = 0x7fffffff;
  if (tid < k) {
    const float lg = excl[tid] > top_p ? kNegInf : cval[tid];
    g.v = lg + gumbel_from_bits(random_bits(ks0, ks1, (uint64_t)(row * k + tid), (uint64_t)(M * k), variant));
    g.i = tid;
  }
  g = block_argmax(g, red_am);
  if (tid == 0) {
    const int tokid = cidx[g.i];
    ids_out[row] = tokid;
    if (logp_out) logp_out[row] = lg(tokid) - lse;
  }
}


// ---- top-k in two launches ---------------------------------------------------------------
// One work-group per row makes nine passes over half a megabyte through a single compute
// unit.  With a workspace the row is cut into segments of at most kSegElems logits, one
// work-group each: the segment is read from HBM once into LDS, reduced to (max, sum of
// exponentials) and to its own k best candidates (same order: larger value, then lower index),
// and a second kernel merges the segments' candidates and statistics and draws the token.  The
// k best of the row are among the k best of the segments, ties included, so the result is the
// one of the single-launch kernel.
constexpr int kSegElems = 8192;    // 32 KiB of LDS: three work-groups per compute unit
constexpr int kSegThreads = 512;
constexpr int kListMax = 2048;     // candidates at or above the pivot kept for the exact ranking
constexpr int kMergeMax = 4096;    // candidates (segments x k) the merging launch can rank

__global__ __launch_bounds__(kSegThreads) void topk_segment_kernel(
    const float* logits, int64_t V, int k, int seg_len, float temperature, const int32_t* forbidden,
    int n_forbidden, float* ws, uint32_t key0, uint32_t key1, int variant, const int32_t* step_ptr,
    int64_t M) {
  extern __shared__ __align__(16) float seg[];   // [seg_len]
  __shared__ uint32_t hist[256];
  __shared__ float red_f[kSegThreads / 64];
  __shared__ uint32_t wave_cnt[kSegThreads / 64];
  __shared__ uint32_t s_sel, s_rem, s_cnt, s_base;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nseg = gridDim.x, sidx = blockIdx.x;
  const int64_t row = blockIdx.y;
  const int64_t v0 = (int64_t)sidx * seg_len;
  const int n = (int)max((int64_t)0, min((int64_t)seg_len, V - v0));
  const float* lr = logits + row * V + v0;
  float* stats = ws + (row * nseg + sidx) * (k > 0 ? 2 + 2 * (int64_t)k : 5);
  float* cand_v = stats + 2;
  int* cand_i = reinterpret_cast<int*>(stats + 2 + k);

  // the segment, scaled and masked, into LDS (16-byte loads where the row allows them)
  float mx = kNegInf;
  const bool vec = ((reinterpret_cast<uintptr_t>(lr) & 15) == 0);
  for (int i = tid * 4; i < n; i += kSegThreads * 4) {
    float x[4];
    if (vec && i + 4 <= n) {
      const f32x4 q = *reinterpret_cast<const f32x4*>(lr + i);
      x[0] = q[0]; x[1] = q[1]; x[2] = q[2]; x[3] = q[3];
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) x[j] = i + j < n ? lr[i + j] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (i + j >= n) break;
      float y = __fdiv_rn(x[j], temperature);
      for (int f = 0; f < n_forbidden; ++f)
        if (forbidden[f] == (int32_t)(v0 + i + j)) y = kNegInf;
      seg[i + j] = y;
      mx = fmaxf(mx, y);
    }
  }
  // maximum and sum of exponentials of the segment
  mx = wave_max(mx);
  __syncthreads();
  if (lane == 0) red_f[wave] = mx;
  __syncthreads();
  mx = red_f[0];
  for (int w = 1; w < kSegThreads / 64; ++w) mx = fmaxf(mx, red_f[w]);
  __syncthreads();
  float se = 0.f;
  if (mx != kNegInf)
    for (int i = tid; i < n; i += kSegThreads) se += expf(seg[i] - mx);
  se = wave_sum(se);
  if (lane == 0) red_f[wave] = se;
  __syncthreads();
  if (tid == 0) {
    float t = 0.f;
    for (int w = 0; w < kSegThreads / 64; ++w) t += red_f[w];
    stats[0] = mx;
    stats[1] = t;
  }
  if (k <= 0) {
    // categorical over the whole vocabulary: this segment's arg-max of logit + gumbel noise
    // (noise of element v of the row: counter row * V + v of M * V, as one draw over [M, V])
    __shared__ ArgMax red_g[kSegThreads / 64];
    uint32_t ks0 = 0u, ks1 = (uint32_t)(*step_ptr);
    threefry2x32(key0, key1, ks0, ks1);
    ArgMax g;
    g.v = kNegInf;
    g.i = 0x7fffffff;
    for (int i = tid; i < n; i += kSegThreads) {
      ArgMax c;
      c.v = seg[i] + gumbel_from_bits(random_bits(ks0, ks1, (uint64_t)(row * V + v0 + i), (uint64_t)(M * V), variant));
      c.i = (int)(v0 + i);
      g = better(g, c);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      ArgMax y;
      y.v = __shfl_xor(g.v, o, 64);
      y.i = __shfl_xor(g.i, o, 64);
      g = better(g, y);
    }
    if (lane == 0) red_g[wave] = g;
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < kSegThreads / 64; ++w) g = better(g, red_g[w]);
      stats[2] = g.v;
      reinterpret_cast<int*>(stats)[3] = g.i;
      stats[4] = g.i == 0x7fffffff ? kNegInf : seg[g.i - (int)v0];
    }
    return;
  }
  for (int i = tid; i < k; i += kSegThreads) {   // fewer than k elements: the rest never wins
    cand_v[i] = kNegInf;
    cand_i[i] = 0x7fffffff;
  }
  if (n <= k) {
    for (int i = tid; i < n; i += kSegThreads) {
      cand_v[i] = seg[i];
      cand_i[i] = (int)(v0 + i);
    }
    return;
  }
  // Pivot: every wave sorts its 64 per-thread maxima (each over a strided subset) and offers its
  // j-th largest, j = ceil(k / waves); at least waves * j >= k elements lie at or above the
  // smallest offer, so {x >= pivot} contains the k best including every tie at the k-th value.
  // For all but adversarial data that set holds a few k elements, which are compacted and
  // ranked by counting.  (A histogram of the key bytes in LDS, the textbook radix select,
  // serialises here: almost all logits share their exponent byte.)
  {
    __shared__ float lst_v[kListMax];
    __shared__ int lst_i[kListMax];
    constexpr int kWaves = kSegThreads / 64;
    float lm = kNegInf;
    for (int i = tid; i < n; i += kSegThreads) lm = fmaxf(lm, seg[i]);
#pragma unroll
    for (int size = 2; size <= 64; size <<= 1)               // bitonic in the wave, descending
#pragma unroll
      for (int st = size >> 1; st > 0; st >>= 1) {
        const float y = __shfl_xor(lm, st, 64);
        const bool up = (lane & size) == 0, low = (lane & st) == 0;
        lm = (up == low) ? fmaxf(lm, y) : fminf(lm, y);
      }
    const int j = (k + kWaves - 1) / kWaves;                 // <= 64: k <= kSegThreads
    const float offer = __shfl(lm, j - 1, 64);
    __syncthreads();
    if (lane == 0) red_f[wave] = offer;
    if (tid == 0) s_cnt = 0;
    __syncthreads();
    float pivot = red_f[0];
    for (int w = 1; w < kWaves; ++w) pivot = fminf(pivot, red_f[w]);
    for (int i = tid; i < n; i += kSegThreads) {
      const float x = seg[i];
      if (x >= pivot) {
        const uint32_t p = atomicAdd(&s_cnt, 1u);
        if (p < kListMax) {
          lst_v[p] = x;
          lst_i[p] = (int)(v0 + i);
        }
      }
    }
    __syncthreads();
    const int c = (int)s_cnt;
    if (c <= kListMax) {
      // rank = number of better candidates (larger value, then lower index): a strict order
      for (int t = tid; t < c; t += kSegThreads) {
        const ArgMax me{lst_v[t], lst_i[t]};
        int r = 0;
        for (int q = 0; q < c; ++q) {
          const float v = lst_v[q];
          r += (v > me.v || (v == me.v && lst_i[q] < me.i)) ? 1 : 0;
        }
        if (r < k) {
          cand_v[r] = me.v;
          cand_i[r] = me.i;
        }
      }
      return;
    }
  }
  // more than kListMax elements at or above the pivot (many equal values): exact radix select
  uint32_t prefix = 0, mask = 0;
  if (tid == 0) s_rem = (uint32_t)k;
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    for (int i = tid; i < n; i += kSegThreads) {
      const uint32_t kk = order_key(seg[i]);
      if ((kk & mask) == prefix) atomicAdd(&hist[(kk >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (tid == 0) {
      uint32_t cum = 0, rem = s_rem;
      int b = 255;
      for (; b > 0; --b) {
        if (cum + hist[b] >= rem) break;
        cum += hist[b];
      }
      s_sel = (uint32_t)b;
      s_rem = rem - cum;
    }
    __syncthreads();
    prefix |= s_sel << shift;
    mask |= 0xffu << shift;
  }
  const uint32_t thr = prefix;
  const uint32_t r_eq = s_rem;  // how many elements equal to the threshold are taken
  if (tid == 0) {
    s_cnt = 0;
    s_base = 0;
  }
  __syncthreads();
  for (int i = tid; i < n; i += kSegThreads) {   // above the threshold: any order
    const float x = seg[i];
    if (order_key(x) > thr) {
      const uint32_t p = atomicAdd(&s_cnt, 1u);
      cand_v[p] = x;
      cand_i[p] = (int)(v0 + i);
    }
  }
  __syncthreads();
  const uint32_t n_gt = s_cnt;
  for (int i0 = 0; i0 < n; i0 += kSegThreads) {   // equal to it: the r_eq lowest indices
    if (s_base >= r_eq) break;
    const int i = i0 + tid;
    const bool eq = i < n && order_key(seg[i]) == thr;
    const uint64_t bal = __ballot(eq);
    const uint32_t before = (uint32_t)__popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) wave_cnt[wave] = (uint32_t)__popcll(bal);
    __syncthreads();
    uint32_t woff = 0, tot = 0;
    for (int w = 0; w < kSegThreads / 64; ++w) {
      if (w < wave) woff += wave_cnt[w];
      tot += wave_cnt[w];
    }
    const uint32_t pos = s_base + woff + before;
    if (eq && pos < r_eq) {
      cand_v[n_gt + pos] = seg[i];
      cand_i[n_gt + pos] = (int)(v0 + i);
    }
    __syncthreads();
    if (tid == 0) s_base += tot;
    __syncthreads();
  }
}

__global__ __launch_bounds__(NTH) void topk_merge_sample_kernel(
    const float* ws, int nseg, int k, float top_p, uint32_t key0, uint32_t key1, int variant,
    const int32_t* step_ptr, int64_t M, int32_t* ids_out, float* logp_out) {
  __shared__ float cval[NTH];
  __shared__ int cidx[NTH];
  __shared__ float mval[kMergeMax];
  __shared__ int midx[kMergeMax];
  __shared__ ArgMax red_am[NTH / 64];
  __shared__ float red_f[NTH / 64];
  __shared__ float prob[NTH];
  __shared__ float excl[NTH];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  const int64_t stride = k > 0 ? 2 + 2 * (int64_t)k : 5;
  const float* rw = ws + row * nseg * stride;
  uint32_t ks0 = 0u, ks1 = (uint32_t)(*step_ptr);
  threefry2x32(key0, key1, ks0, ks1);
  // log-sum-exp of the row from the segments' (max, sum)
  float gm = kNegInf;
  for (int sg = 0; sg < nseg; ++sg) gm = fmaxf(gm, rw[sg * stride]);
  float se = 0.f;
  for (int sg = 0; sg < nseg; ++sg) {
    const float m = rw[sg * stride];
    if (m != kNegInf) se += rw[sg * stride + 1] * expf(m - gm);
  }
  const float lse = gm + logf(se);
  if (k <= 0) {  // whole-vocabulary draw: best (logit + noise) over the segments
    if (tid == 0) {
      ArgMax g;
      g.v = kNegInf;
      g.i = 0x7fffffff;
      float lgt = kNegInf;
      for (int sg = 0; sg < nseg; ++sg) {
        ArgMax c;
        c.v = rw[sg * stride + 2];
        c.i = reinterpret_cast<const int*>(rw + sg * stride)[3];
        const ArgMax w = better(g, c);
        if (w.i != g.i) lgt = rw[sg * stride + 4];
        g = w;
      }
      ids_out[row] = g.i;
      if (logp_out) logp_out[row] = lgt - lse;
    }
    return;
  }
  // all candidates into LDS, bitonic sort (best first: larger value, then lower index); only as
  // many slots as there are candidates take part, padded to a power of two with -inf
  const int nc = nseg * k;
  int m2 = 64;
  while (m2 < nc) m2 <<= 1;
  for (int t = tid; t < m2; t += NTH) {
    const int sg = t / k, j = t % k;
    mval[t] = t < nc ? rw[sg * stride + 2 + j] : kNegInf;
    midx[t] = t < nc ? reinterpret_cast<const int*>(rw + sg * stride + 2 + k)[j] : 0x7fffffff;
  }
  __syncthreads();
  for (int size = 2; size <= m2; size <<= 1) {
    for (int st = size >> 1; st > 0; st >>= 1) {
      for (int t = tid; t < m2; t += NTH) {
        const int partner = t ^ st;
        if (partner > t) {
          ArgMax x{mval[t], midx[t]}, y{mval[partner], midx[partner]};
          const bool x_first = (x.v > y.v) || (x.v == y.v && x.i < y.i);
          const bool up = (t & size) == 0;
          if (up != x_first) {
            mval[t] = y.v; midx[t] = y.i;
            mval[partner] = x.v; midx[partner] = x.i;
          }
        }
      }
      __syncthreads();
    }
  }
  cval[tid] = tid < m2 ? mval[tid] : kNegInf;
  cidx[tid] = tid < m2 ? midx[tid] : 0x7fffffff;
  __syncthreads();
  // softmax over the k sorted logits, top-p cut, gumbel arg-max (as in sample_topk_kernel)
  const float mx = cval[0];
  float e = tid < k ? expf(cval[tid] - mx) : 0.f;
  const float tot = block_sum_f(e, red_f);
  prob[tid] = e / tot;
  __syncthreads();
  if (tid == 0) {
    float c = 0.f;
    for (int j = 0; j < k; ++j) {
      c += prob[j];
      excl[j] = c - prob[j];
    }
  }
  __syncthreads();
  ArgMax g;
  g.v = kNegInf;
  g.i = 0x7fffffff;
  if (tid < k) {
    const float lgt = excl[tid] > top_p ? kNegInf : cval[tid];
    g.v = lgt + gumbel_from_bits(random_bits(ks0, ks1, (uint64_t)(row * k + tid), (uint64_t)(M * k), variant));
    g.i = tid;
  }
  g = block_argmax(g, red_am);
  if (tid == 0) {
    ids_out[row] = cidx[g.i];
    if (logp_out) logp_out[row] = cval[g.i] - lse;
  }
}


// ---- top-k from the head's own block statistics, one launch -----------------------------------
// The head leaves, per row and 128-column block, the block's largest scaled logit.  Under the
// order of the selection (larger value, then lower index) the k best elements of a row lie in
// the k best blocks ordered by (block maximum, then lower block): a block outside them has k
// blocks whose best element comes before every one of its own.  So one work-group per row picks
// those blocks from the statistics, fetches only their logits (k x 128 instead of the row), and
// selects, ranks and draws as the two launches above do: same candidates, same draw.  The
// log-probability is taken against the head's own log-sum-exp of the row.
constexpr int kBlkCols = 128;        // columns per statistics block (tnx_lmhead_nblocks)
constexpr int kBlkThreads = 512;
constexpr int kBlkMaxBlocks = 4096;  // block maxima of a row held in LDS
constexpr int kBlkMaxK = kSegElems / kBlkCols;

struct SelectScratch {
  float lst_v[kListMax];
  int lst_i[kListMax];
  uint32_t hist[256];
  float red_f[kBlkThreads / 64];
  uint32_t wave_cnt[kBlkThreads / 64];
  uint32_t sel, rem, cnt, base;
};

// The k best of v[0..n) (LDS) under (larger value, then lower id), id of position i = gi(i),
// positions in id order; result ranked best first in cv / ci [0..k) (LDS), padded with
// (-inf, 0x7fffffff) when n < k.  Every thread of the work-group calls it; it ends on a barrier.
template <class IdxFn>
__device__ void select_best(const float* v, int n, int k, IdxFn gi, float* cv, int* ci, SelectScratch& s) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr int kWaves = kBlkThreads / 64;
  auto rank_list = [&](const float* lv, const int* li, int c) {   // c <= kListMax candidates -> ranks
    for (int t = tid; t < c; t += kBlkThreads) {
      const float mv = lv[t];
      const int mi = li[t];
      int r = 0;
      for (int q = 0; q < c; ++q) {
        const float x = lv[q];
        r += (x > mv || (x == mv && li[q] < mi)) ? 1 : 0;
      }
      if (r < k) {
        cv[r] = mv;
        ci[r] = mi;
      }
    }
  };
  __syncthreads();
  for (int i = tid; i < k; i += kBlkThreads) {
    cv[i] = kNegInf;
    ci[i] = 0x7fffffff;
  }
  if (tid == 0) s.cnt = 0;
  // pivot: every wave offers the j-th largest of its threads' maxima, j = ceil(k / waves); at
  // least k elements lie at or above the smallest offer, every tie at the k-th value included
  float lm = kNegInf;
  for (int i = tid; i < n; i += kBlkThreads) lm = fmaxf(lm, v[i]);
#pragma unroll
  for (int size = 2; size <= 64; size <<= 1)
#pragma unroll
    for (int st = size >> 1; st > 0; st >>= 1) {
      const float y = __shfl_xor(lm, st, 64);
      const bool up = (lane & size) == 0, low = (lane & st) == 0;
      lm = (up == low) ? fmaxf(lm, y) : fminf(lm, y);
    }
  const int j = (k + kWaves - 1) / kWaves;
  const float offer = __shfl(lm, j - 1, 64);
  if (lane == 0) s.red_f[wave] = offer;
  __syncthreads();
  float pivot = s.red_f[0];
  for (int w = 1; w < kWaves; ++w) pivot = fminf(pivot, s.red_f[w]);
  for (int i = tid; i < n; i += kBlkThreads) {
    const float x = v[i];
    if (x >= pivot) {
      const uint32_t p = atomicAdd(&s.cnt, 1u);
      if (p < kListMax) {
        s.lst_v[p] = x;
        s.lst_i[p] = gi(i);
      }
    }
  }
  __syncthreads();
  const int c = (int)s.cnt;
  if (c <= kListMax) {
    rank_list(s.lst_v, s.lst_i, c);
    __syncthreads();
    return;
  }
  // more than kListMax elements at or above the pivot (many equal values): exact radix select of
  // the k-th key, the elements above it in any order, those equal to it by lowest position
  uint32_t prefix = 0, mask = 0;
  if (tid == 0) s.rem = (uint32_t)k;
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    if (tid < 256) s.hist[tid] = 0;
    __syncthreads();
    for (int i = tid; i < n; i += kBlkThreads) {
      const uint32_t kk = order_key(v[i]);
      if ((kk & mask) == prefix) atomicAdd(&s.hist[(kk >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (tid == 0) {
      uint32_t cum = 0, rem = s.rem;
      int b = 255;
      for (; b > 0; --b) {
        if (cum + s.hist[b] >= rem) break;
        cum += s.hist[b];
      }
      s.sel = (uint32_t)b;
      s.rem = rem - cum;
    }
    __syncthreads();
    prefix |= s.sel << shift;
    mask |= 0xffu << shift;
  }
  const uint32_t thr = prefix, r_eq = s.rem;
  if (tid == 0) {
    s.cnt = 0;
    s.base = 0;
  }
  __syncthreads();
  for (int i = tid; i < n; i += kBlkThreads) {
    const float x = v[i];
    if (order_key(x) > thr) {
      const uint32_t p = atomicAdd(&s.cnt, 1u);
      s.lst_v[p] = x;
      s.lst_i[p] = gi(i);
    }
  }
  __syncthreads();
  const uint32_t n_gt = s.cnt;   // < k
  for (int i0 = 0; i0 < n; i0 += kBlkThreads) {
    if (s.base >= r_eq) break;
    const int i = i0 + tid;
    const bool eq = i < n && order_key(v[i]) == thr;
    const uint64_t bal = __ballot(eq);
    const uint32_t before = (uint32_t)__popcll(bal & ((1ull << lane) - 1ull));
    if (lane == 0) s.wave_cnt[wave] = (uint32_t)__popcll(bal);
    __syncthreads();
    uint32_t woff = 0, tot = 0;
    for (int w = 0; w < kWaves; ++w) {
      if (w < wave) woff += s.wave_cnt[w];
      tot += s.wave_cnt[w];
    }
    const uint32_t pos = s.base + woff + before;
    if (eq && pos < r_eq) {
      s.lst_v[n_gt + pos] = v[i];
      s.lst_i[n_gt + pos] = gi(i);
    }
    __syncthreads();
    if (tid == 0) s.base += tot;
    __syncthreads();
  }
  __syncthreads();
  rank_list(s.lst_v, s.lst_i, k);
  __syncthreads();
}

__global__ __launch_bounds__(kBlkThreads) void topk_blocks_sample_kernel(
    const float* logits, const float* part, const float* lse, int64_t V, int nvb, int k, float top_p,
    float temperature, const int32_t* forbidden, int n_forbidden, uint32_t key0, uint32_t key1, int variant,
    const int32_t* step_ptr, int64_t M, int32_t* ids_out, float* logp_out) {
  __shared__ __align__(16) float buf[kSegElems];   // the block maxima, then the gathered logits
  __shared__ SelectScratch sc;
  __shared__ float cv[kBlkMaxK];
  __shared__ int ci[kBlkMaxK];
  __shared__ int blk[kBlkMaxK];
  __shared__ float prob[kBlkMaxK], excl[kBlkMaxK];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t row = blockIdx.x;
  // 1. the k best blocks by (maximum, then lower block)
  for (int b = tid; b < nvb; b += kBlkThreads) buf[b] = part[(row * nvb + b) * 4];
  const int kb = min(k, nvb);
  select_best(buf, nvb, kb, [](int i) { return i; }, cv, ci, sc);
  // 2. in block order, so that positions in LDS are in id order
  if (tid < kb) {
    const int me = ci[tid];
    int r = 0;
    for (int q = 0; q < kb; ++q) r += ci[q] < me ? 1 : 0;
    blk[r] = me;
  }
  __syncthreads();
  // 3. their logits, scaled and masked as the sampling launches do
  const float* lr = logits + row * V;
  const int n2 = kb * kBlkCols;
  const bool vec = (reinterpret_cast<uintptr_t>(lr) & 15) == 0 && V % 4 == 0;
  for (int e = tid * 4; e < n2; e += kBlkThreads * 4) {
    const int64_t col = (int64_t)blk[e >> 7] * kBlkCols + (e & 127);
    float x[4];
    if (vec && col + 4 <= V) {
      const f32x4 q = *reinterpret_cast<const f32x4*>(lr + col);
      x[0] = q[0]; x[1] = q[1]; x[2] = q[2]; x[3] = q[3];
    } else {
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) x[jj] = col + jj < V ? lr[col + jj] : 0.f;
    }
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      float y = col + jj < V ? __fdiv_rn(x[jj], temperature) : kNegInf;
      for (int f = 0; f < n_forbidden; ++f)
        if (forbidden[f] == (int32_t)(col + jj)) y = kNegInf;
      buf[e + jj] = y;
    }
  }
  // 4. the k best of those (select_best starts on a barrier)
  select_best(buf, n2, k, [&](int i) { return blk[i >> 7] * kBlkCols + (i & 127); }, cv, ci, sc);
  // 5. softmax over the k sorted logits, top-p cut, gumbel arg-max (as topk_merge_sample_kernel)
  uint32_t ks0 = 0u, ks1 = (uint32_t)(*step_ptr);
  threefry2x32(key0, key1, ks0, ks1);
  const float mx = cv[0];
  if (wave == 0) {
    const float e = lane < k ? expf(cv[lane] - mx) : 0.f;
    const float tot = wave_sum(e);
    prob[lane] = e / tot;
  }
  __syncthreads();
  if (tid == 0) {
    float c = 0.f;
    for (int jj = 0; jj < k; ++jj) {
      c += prob[jj];
      excl[jj] = c - prob[jj];
    }
  }
  __syncthreads();
  if (wave == 0) {
    ArgMax g;
    g.v = kNegInf;
    g.i = 0x7fffffff;
    if (lane < k) {
      const float lgt = excl[lane] > top_p ? kNegInf : cv[lane];
      g.v = lgt + gumbel_from_bits(random_bits(ks0, ks1, (uint64_t)(row * k + lane), (uint64_t)(M * k), variant));
      g.i = lane;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      ArgMax y;
      y.v = __shfl_xor(g.v, o, 64);
      y.i = __shfl_xor(g.i, o, 64);
      g = better(g, y);
    }
    if (lane == 0) {
      const int w = g.i < k ? g.i : 0;   // (no finite candidate at all: the best-ranked one)
      ids_out[row] = ci[w];
      if (logp_out) logp_out[row] = cv[w] - lse[row];
    }
  }
}


// ---- top-p over the whole vocabulary (top_k absent with top_p < 1, or top_k == V) -------------
// sample_top_p then sorts the full row (jax.lax.top_k with k = V: descending, the lower index first
// among equal values): a stable least-significant-digit radix sort per row, written here (four
// passes of eight bits over order-preserving keys), then one work-group per row that soft-maxes
// the sorted row, keeps the entries whose exclusive cumulative probability is <= top_p and draws
// by Gumbel-max with the noise of the SORTED position, as jax.random.categorical over the sorted
// logits does.
//
// The sort: one work-group of kSortThreads threads per row.  Thread t owns the contiguous chunk
// [t * per, (t + 1) * per) of the row, so "thread order, then position inside the chunk" is the
// row's order and a counting sort that hands out positions in that order is stable.  Per pass:
// every thread counts its chunk's digits into its own column of an LDS table [256 digits][threads]
// (no atomics), the table is turned into exclusive offsets in (digit, thread) order -- each pair
// of digit rows summed by one thread, the 256 digit totals scanned, the rows rewritten -- and
// every thread walks its chunk again and moves each element to offset[digit][t]++.  Keys are the
// bit patterns of the scaled logits mapped so that unsigned order is descending float order; the
// first pass reads the logits themselves (dividing by the temperature and masking forbidden ids
// on the way), the last one writes floats back.  Two (key, id) buffer pairs alternate; after the
// fourth pass the sorted row is in the first pair.
constexpr int kSortThreads = 128;
constexpr int kSortLd = kSortThreads + 1;              // padded row of the table: bank-conflict-free scans
constexpr size_t kSortLdsBytes = 256 * (size_t)kSortLd * sizeof(uint32_t);

__device__ __forceinline__ uint32_t desc_key(float f) { return ~order_key(f); }   // ascending unsigned = descending float
__device__ __forceinline__ float desc_key_inv(uint32_t k) {
  const uint32_t o = ~k;
  return __uint_as_float((o & 0x80000000u) ? (o & 0x7fffffffu) : ~o);
}

__global__ __launch_bounds__(kSortThreads) void fullsort_kernel(const float* logits, int64_t V, float temperature,
                                                                const int32_t* forbidden, int n_forbidden,
                                                                uint32_t* k0, int* i0, uint32_t* k1, int* i1) {
  extern __shared__ uint32_t cnt[];                    // [256][kSortLd]
  __shared__ uint32_t digit_base[256];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  const int64_t per = (V + kSortThreads - 1) / kSortThreads;
  const int64_t j0 = min(V, tid * per), j1 = min(V, j0 + per);
  const float* lrow = logits + row * V;
  uint32_t* ka = k0 + row * V;
  int* ia = i0 + row * V;
  uint32_t* kb = k1 + row * V;
  int* ib = i1 + row * V;
  // key of element j in pass 0: the scaled, masked logit (what tnx_sample_topk's other paths draw from)
  auto first_key = [&](int64_t j) -> uint32_t {
    float y = __fdiv_rn(lrow[j], temperature);
    for (int f = 0; f < n_forbidden; ++f)
      if (forbidden[f] == (int)j) y = kNegInf;
    return desc_key(y);
  };
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 8 * pass;
    const uint32_t* src_k = (pass & 1) ? kb : ka;      // passes 1, 3 read the second pair
    const int* src_i = (pass & 1) ? ib : ia;
    uint32_t* dst_k = (pass & 1) ? ka : kb;
    int* dst_i = (pass & 1) ? ia : ib;
    for (int d = 0; d < 256; ++d) cnt[d * kSortLd + tid] = 0;
    // (a thread touches only its own column until the barrier)
    for (int64_t j = j0; j < j1; ++j) {
      const uint32_t key = pass == 0 ? first_key(j) : src_k[j];
      ++cnt[((key >> shift) & 255u) * kSortLd + tid];
    }
    __syncthreads();
    // exclusive offsets in (digit, thread) order: the two digit rows of this thread summed, ...
    uint32_t tot[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int d = 2 * tid + h;
      uint32_t run = 0;
      for (int t = 0; t < kSortThreads; ++t) {
        const uint32_t c = cnt[d * kSortLd + t];
        cnt[d * kSortLd + t] = run;
        run += c;
      }
      tot[h] = run;
      digit_base[d] = run;
    }
    __syncthreads();
    // ... the digit totals scanned (256 values: every thread walks the ones below its own two), ...
    uint32_t base = 0;
    for (int d = 0; d < 2 * tid; ++d) base += digit_base[d];
    __syncthreads();
    digit_base[2 * tid] = base;
    digit_base[2 * tid + 1] = base + tot[0];
    __syncthreads();
    // ... and every element moved to its digit's base + its (thread, position) rank
    for (int64_t j = j0; j < j1; ++j) {
      const uint32_t key = pass == 0 ? first_key(j) : src_k[j];
      const int id = pass == 0 ? (int)j : src_i[j];
      const uint32_t d = (key >> shift) & 255u;
      const uint32_t pos = digit_base[d] + cnt[d * kSortLd + tid]++;
      dst_k[pos] = pass == 3 ? __float_as_uint(desc_key_inv(key)) : key;
      dst_i[pos] = id;
    }
    __syncthreads();   // the pass's writes are visible to the work-group's next pass; the table is free
  }
}

__global__ __launch_bounds__(NTH) void fullsort_sample_kernel(const float* skeys, const int* sids, int64_t V,
                                                              float top_p, uint32_t key0, uint32_t key1,
                                                              int variant, const int32_t* step_ptr, int64_t M,
                                                              int32_t* ids_out, float* logp_out) {
  __shared__ ArgMax red_am[NTH / 64];
  __shared__ float red_f[NTH / 64];
  __shared__ float chunk_sum[NTH];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  const float* sk = skeys + row * V;
  uint32_t ks0 = 0u, ks1 = (uint32_t)(*step_ptr);
  threefry2x32(key0, key1, ks0, ks1);
  const float mx = sk[0];
  // every thread owns a contiguous chunk of the sorted row
  const int64_t per = (V + NTH - 1) / NTH;
  const int64_t j0 = min(V, tid * per), j1 = min(V, j0 + per);
  float se = 0.f;
  for (int64_t j = j0; j < j1; ++j) se += expf(sk[j] - mx);
  chunk_sum[tid] = se;
  const float tot = block_sum_f(se, red_f);
  // exclusive prefix of the chunk sums (in probability units), then the scan inside the chunk
  __syncthreads();
  float before = 0.f;
  for (int t = 0; t < tid; ++t) before += chunk_sum[t];
  float c = before / tot;
  ArgMax g;
  g.v = kNegInf;
  g.i = 0x7fffffff;
  for (int64_t j = j0; j < j1; ++j) {
    const float pj = expf(sk[j] - mx) / tot;
    const float lg = c > top_p ? kNegInf : sk[j];          // cumsum - p > top_p is dropped
    c += pj;
    ArgMax x;
    x.v = lg + gumbel_from_bits(random_bits(ks0, ks1, (uint64_t)(row * V + j), (uint64_t)(M * V), variant));
    x.i = (int)j;
    g = better(g, x);
  }
  g = block_argmax(g, red_am);
  if (tid == 0) {
    ids_out[row] = sids[row * V + g.i];
    if (logp_out) logp_out[row] = sk[g.i] - (mx + logf(tot));
  }
}

struct FullSortWs {
  size_t keys_a, keys_b, ids_a, ids_b, total;
};
void fullsort_layout(int64_t M, int64_t V, FullSortWs* w) {
  const size_t n = (size_t)(M * V);
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  size_t o = 0;
  w->keys_a = o; o += up(n * 4);
  w->keys_b = o; o += up(n * 4);
  w->ids_a = o; o += up(n * 4);
  w->ids_b = o; o += up(n * 4);
  w->total = o;
}

}  // namespace

extern "C" size_t tnx_sample_fullsort_ws_bytes(int64_t M, int64_t V) {
  FullSortWs w;
  if (M <= 0 || V <= 0 || M * V >= (1ll << 31)) return 0;
  fullsort_layout(M, V, &w);
  return w.total;
}

extern "C" size_t tnx_sample_topk_ws_bytes(int64_t M, int64_t V, int k) {
  if (M <= 0 || V <= 0) return 0;
  if (k <= 0 || k >= V) k = 0;  // whole-vocabulary draw: (max, sum, noisy best, its id, its logit); k == V takes the full sort
  return (size_t)(M * cdiv(V, kSegElems) * (k > 0 ? 2 + 2 * (int64_t)k : 5)) * sizeof(float);
}

extern "C" int tnx_sample_topk(void* stream, const float* logits, int64_t M, int64_t V, int k,
                               float top_p, float temperature, uint32_t key0, uint32_t key1,
                               int rng_variant, const int32_t* forbidden, int n_forbidden,
                               const int32_t* step_ptr, float* ws, int32_t* ids_out,
                               float* logp_out) {
  TNX_REQUIRE(logits && step_ptr && ids_out, "sample_topk: null pointer");
  TNX_REQUIRE(M > 0 && V > 0 && V < (1ll << 31), "sample_topk: bad shape");
  TNX_REQUIRE(rng_variant == 0 || rng_variant == 1, "sample_topk: rng_variant must be 0 or 1");
  TNX_REQUIRE(temperature > 0.f, "sample_topk: temperature must be positive, got %f", temperature);
  // jax.lax.top_k refuses k beyond the last axis (sampler.py:126-127)
  TNX_REQUIRE(k <= V, "sample_topk: top_k=%d exceeds the vocabulary (%lld)", k, (long long)V);
  if (k <= 0 || k == V) {
    // no top-k with top_p < 1, or a top-k of the whole vocabulary (whatever top_p): the reference
    // sorts the row and draws over SORTED positions; only top_k absent with top_p >= 1 draws over
    // vocabulary ids (sampler.py:118-127)
    if (top_p < 1.0f || k == V) {
      TNX_REQUIRE(ws, "sample_topk: top_p < 1 without top_k (or top_k == V) sorts the whole row and needs a "
                      "workspace of tnx_sample_fullsort_ws_bytes(M, V) bytes");
      TNX_REQUIRE(M * V < (1ll << 31), "sample_topk: M * V too large for the full-row sort");
      FullSortWs w;
      fullsort_layout(M, V, &w);
      unsigned char* base = reinterpret_cast<unsigned char*>(ws);
      uint32_t* ka = reinterpret_cast<uint32_t*>(base + w.keys_a);
      uint32_t* kb = reinterpret_cast<uint32_t*>(base + w.keys_b);
      int* ia = reinterpret_cast<int*>(base + w.ids_a);
      int* ib = reinterpret_cast<int*>(base + w.ids_b);
      static std::once_flag sort_once;
      static hipError_t sort_rc = hipSuccess;
      std::call_once(sort_once, [] {
        sort_rc = hipFuncSetAttribute(reinterpret_cast<const void*>(fullsort_kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSortLdsBytes);
      });
      TNX_REQUIRE(sort_rc == hipSuccess, "sample_topk: cannot raise the dynamic LDS limit of the sort");
      hipLaunchKernelGGL(fullsort_kernel, dim3((unsigned)M), dim3(kSortThreads), kSortLdsBytes, as_stream(stream), logits,
                         V, temperature, forbidden, forbidden ? n_forbidden : 0, ka, ia, kb, ib);
      TNX_CHECK_LAUNCH("sample_topk (sort)");
      // (four passes: the sorted floats and their ids are back in the first pair)
      hipLaunchKernelGGL(fullsort_sample_kernel, dim3((unsigned)M), dim3(NTH), 0, as_stream(stream),
                         reinterpret_cast<const float*>(ka), ia, V,
                         top_p, key0, key1, rng_variant, step_ptr, M, ids_out, logp_out);
      TNX_CHECK_LAUNCH("sample_topk (sorted draw)");
      return TNX_OK;
    }
    k = 0;
  }
  TNX_REQUIRE(k <= NTH, "sample_topk: top_k=%d exceeds %d", k, NTH);
  const int nseg = (int)cdiv(V, kSegElems);
  if (ws && (k == 0 || (k <= kSegThreads && (int64_t)nseg * k <= kMergeMax))) {
    // segments of equal length, a multiple of 4 so that aligned rows stay aligned
    const int seg_len = (int)(cdiv(cdiv(V, nseg), 4) * 4);
    static std::once_flag once;
    static hipError_t attr_rc = hipSuccess;
    std::call_once(once, [] {
      attr_rc = hipFuncSetAttribute(reinterpret_cast<const void*>(topk_segment_kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kSegElems * 4);
    });
    TNX_REQUIRE(attr_rc == hipSuccess, "sample_topk: cannot raise the dynamic LDS limit");
    hipLaunchKernelGGL(topk_segment_kernel, dim3((unsigned)nseg, (unsigned)M), dim3(kSegThreads),
                       (size_t)seg_len * 4, as_stream(stream), logits, V, k, seg_len, temperature, forbidden,
                       forbidden ? n_forbidden : 0, ws, key0, key1, rng_variant, step_ptr, M);
    TNX_CHECK_LAUNCH("sample_topk (segments)");
    hipLaunchKernelGGL(topk_merge_sample_kernel, dim3((unsigned)M), dim3(NTH), 0, as_stream(stream), ws, nseg,
                       k, top_p, key0, key1, rng_variant, step_ptr, M, ids_out, logp_out);
    TNX_CHECK_LAUNCH("sample_topk (merge)");
    return TNX_OK;
  }
  hipLaunchKernelGGL(sample_topk_kernel, dim3((unsigned)M), dim3(NTH), 0, as_stream(stream), logits,
                     V, k, top_p, key0, key1, rng_variant, step_ptr, M, temperature, forbidden,
                     forbidden ? n_forbidden : 0, ids_out, logp_out);
  TNX_CHECK_LAUNCH("sample_topk");
  return TNX_OK;
}

extern "C" int tnx_sample_topk_head_ok(int64_t V, int k) {
  return k > 0 && k < V && k <= kBlkMaxK && cdiv(V, kBlkCols) <= kBlkMaxBlocks ? 1 : 0;
}

extern "C" int tnx_sample_topk_head(void* stream, const float* logits, const float* part, const float* lse,
                                    int64_t M, int64_t V, int k, float top_p, float temperature, uint32_t key0,
                                    uint32_t key1, int rng_variant, const int32_t* forbidden, int n_forbidden,
                                    const int32_t* step_ptr, int32_t* ids_out, float* logp_out) {
  TNX_REQUIRE(logits && part && step_ptr && ids_out, "sample_topk_head: null pointer");
  TNX_REQUIRE(!logp_out || lse, "sample_topk_head: log-probabilities need the head's log-sum-exp");
  TNX_REQUIRE(M > 0 && V > 0 && V < (1ll << 31), "sample_topk_head: bad shape");
  TNX_REQUIRE(rng_variant == 0 || rng_variant == 1, "sample_topk_head: rng_variant must be 0 or 1");
  TNX_REQUIRE(temperature > 0.f, "sample_topk_head: temperature must be positive, got %f", temperature);
  TNX_REQUIRE(tnx_sample_topk_head_ok(V, k),
              "sample_topk_head: needs 0 < top_k <= %d, top_k < V and V <= %d (top_k=%d, V=%lld): use tnx_sample_topk",
              kBlkMaxK, kBlkMaxBlocks * kBlkCols, k, (long long)V);
  hipLaunchKernelGGL(topk_blocks_sample_kernel, dim3((unsigned)M), dim3(kBlkThreads), 0, as_stream(stream), logits,
                     part, lse, V, (int)cdiv(V, kBlkCols), k, top_p, temperature, forbidden, forbidden ? n_forbidden : 0,
                     key0, key1, rng_variant, step_ptr, M, ids_out, logp_out);
  TNX_CHECK_LAUNCH("sample_topk_head");
  return TNX_OK;
}
