// Error plumbing, small element-wise kernels (fill, sampler bookkeeping, GRPO ratio) and the
// MoE routing helpers.
#include <stdarg.h>
#include <string.h>

#include <mutex>

#include "common.h"

namespace {
thread_local char g_err[512] = "";
}

void tnx_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char* tnx_last_error(void) { return g_err; }
extern "C" int tnx_version(void) { return TNX_ABI_VERSION; }

namespace {

__global__ void fill_kernel(uint32_t* p, int64_t n, uint32_t v) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

__global__ void sample_commit_kernel(const int32_t* ids, const float* logp, int64_t B,
                                     int32_t* tokens, int64_t tok_ld, float* logprobs,
                                     int32_t* done, const int32_t* eos, int n_eos,
                                     int32_t* step_ptr) {
  // single work-group: every thread reads the step before anyone advances it
  const int col = *step_ptr;
  __syncthreads();
  for (int64_t b = threadIdx.x; b < B; b += blockDim.x) {
    const int32_t id = ids[b];
    tokens[b * tok_ld + col + 1] = id;
    if (logprobs && logp) logprobs[b * tok_ld + col + 1] = logp[b];
    if (done) {
      int hit = 0;
      for (int e = 0; e < n_eos; ++e) hit |= (id == eos[e]);
      if (hit) done[b] = 1;
    }
  }
  if (threadIdx.x == 0) *step_ptr = col + 1;
}

__global__ void grpo_ratio_kernel(const float* logp, const float* old_logp, const float* adv,
                                  int64_t N, int64_t tokens_per_seq, float eps_lo, float eps_hi,
                                  float* ratio, float* loss, int32_t* clipped) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N) return;
  float lr = logp[i] - (old_logp ? old_logp[i] : logp[i]);
  lr = fminf(fmaxf(lr, -20.0f), 20.0f);
  const float r = expf(lr);
  const float a = adv[i / tokens_per_seq];
  const float l1 = -a * r;
  const float l2 = -a * fminf(fmaxf(r, 1.0f - eps_lo), 1.0f + eps_hi);
  if (ratio) ratio[i] = r;
  if (loss) loss[i] = fmaxf(l1, l2);
  if (clipped) clipped[i] = l2 > l1 ? 1 : 0;
}

// Per-token KL estimators: logp - ref ("kl"), half the squared difference ("mse_kl"),
// exp(d) - d - 1 with d = ref - logp ("low_var_kl"); optional symmetric clamp.
__global__ void kl_divergence_kernel(const float* logp, const float* ref_logp, int64_t N, int method,
                                     float clamp, float* kl) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N) return;
  const float p = logp[i], q = ref_logp[i];
  float v;
  if (method == TNX_KL_KL) {
    v = p - q;
  } else if (method == TNX_KL_MSE) {
    const float d = p - q;
    v = 0.5f * (d * d);
  } else {
    const float d = q - p;
    v = expf(d) - d - 1.0f;
  }
  if (clamp >= 0.f) v = fminf(fmaxf(v, -clamp), clamp);
  kl[i] = v;
}

// Sum of 256 values, one per thread, in a fixed order: every launch adds the same numbers in
// the same tree, so the aggregates do not change between runs.
__device__ __forceinline__ float block_sum256(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();   // red may still be read from an earlier call
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

// Row b: (sum of loss * mask, sum of mask) -> row_ws[b][0..1].
__global__ __launch_bounds__(256) void agg_rows_kernel(const float* loss, const float* mask, int64_t T,
                                                       float* row_ws) {
  __shared__ float red[4];
  const int64_t b = blockIdx.x;
  float s = 0.f, c = 0.f;
  for (int64_t t = threadIdx.x; t < T; t += 256) {
    const float m = mask[b * T + t];
    s += loss[b * T + t] * m;
    c += m;
  }
  s = block_sum256(s, red);
  c = block_sum256(c, red);
  if (threadIdx.x == 0) {
    row_ws[2 * b] = s;
    row_ws[2 * b + 1] = c;
  }
}

// The rows' sums -> (unreduced sum, denominator) of the aggregation mode.
__global__ __launch_bounds__(256) void agg_finish_kernel(const float* row_ws, int64_t B, int mode,
                                                         float norm, float* out) {
  __shared__ float red[4];
  float num = 0.f, den = 0.f;
  for (int64_t b = threadIdx.x; b < B; b += 256) {
    const float s = row_ws[2 * b], c = row_ws[2 * b + 1];
    const float nonempty = c > 0.f ? 1.f : 0.f;
    if (mode == TNX_AGG_TOKEN_MEAN) {
      num += s;
      den += c;
    } else if (mode == TNX_AGG_SEQ_MEAN_TOKEN_MEAN) {
      num += s / fmaxf(c, 1.0f);
      den += nonempty;
    } else if (mode == TNX_AGG_SEQ_MEAN_TOKEN_SCALE) {
      num += s / fmaxf(norm, 1e-6f);
      den += nonempty;
    } else if (mode == TNX_AGG_SEQ_MEAN_TOKEN_SUM) {
      num += s * nonempty;
      den += nonempty;
    } else {
      num += s;
    }
  }
  num = block_sum256(num, red);
  den = block_sum256(den, red);
  if (threadIdx.x == 0) {
    out[0] = num;
    out[1] = mode == TNX_AGG_SEQ_MEAN_TOKEN_SUM_NORM ? norm : den;
  }
}

// Packed batches: row b holds several sequences told apart by segment_ids[b][t] (0 = padding).
// Per row and segment s: (sum of loss * mask, sum of mask) -> seg_ws[b][s][0..1], each sum taken
// over the row's tokens in order by ONE thread (thread s % 256 handles segment s), so the result
// does not depend on the launch.  The row is staged through LDS 1024 tokens at a time; ids outside
// [0, S) belong to no segment.
__global__ __launch_bounds__(256) void agg_segments_kernel(const float* loss, const float* mask,
                                                           const int32_t* seg, int64_t T, int S, float* seg_ws) {
  __shared__ float s_lm[1024], s_m[1024];
  __shared__ int32_t s_seg[1024];
  const int64_t b = blockIdx.x;
  for (int s0 = 0; s0 < S; s0 += 256) {
    const int sid = s0 + threadIdx.x;
    float l = 0.f, c = 0.f;
    for (int64_t t0 = 0; t0 < T; t0 += 1024) {
      __syncthreads();   // the stage may still be read from the turn before
      for (int i = threadIdx.x; i < 1024; i += 256) {
        const int64_t t = t0 + i;
        const float m = t < T ? mask[b * T + t] : 0.f;
        s_m[i] = m;
        s_lm[i] = t < T ? loss[b * T + t] * m : 0.f;
        s_seg[i] = t < T ? seg[b * T + t] : -1;
      }
      __syncthreads();
      const int n = (int)min((int64_t)1024, T - t0);
      if (sid < S) {
        for (int i = 0; i < n; ++i)
          if (s_seg[i] == sid) {
            l += s_lm[i];
            c += s_m[i];
          }
      }
    }
    if (sid < S) {
      seg_ws[(b * S + sid) * 2] = l;
      seg_ws[(b * S + sid) * 2 + 1] = c;
    }
  }
}

// (unreduced sum, denominator) of the mode from the per-segment sums (segment 0 excluded, a
// segment counts when it has a scored token) and, for the two modes that ignore segments, from
// the per-row sums.  norm <= 0 in the sum-norm mode means the reference's default there: the
// number of active segments.
__global__ __launch_bounds__(256) void agg_segments_finish_kernel(const float* seg_ws, const float* row_ws, int64_t B,
                                                                  int S, int mode, float norm, float* out) {
  __shared__ float red[4];
  float num = 0.f, act = 0.f, tot = 0.f, cnt = 0.f;
  for (int64_t i = threadIdx.x; i < B * S; i += 256) {
    if (i % S == 0) continue;   // the padding bucket
    const float l = seg_ws[2 * i], c = seg_ws[2 * i + 1];
    if (c > 0.f) {
      act += 1.f;
      if (mode == TNX_AGG_SEQ_MEAN_TOKEN_MEAN) num += l / fmaxf(c, 1.0f);
      else if (mode == TNX_AGG_SEQ_MEAN_TOKEN_SCALE) num += l / fmaxf(norm, 1e-6f);
      else if (mode == TNX_AGG_SEQ_MEAN_TOKEN_SUM) num += l;
    }
  }
  for (int64_t b = threadIdx.x; b < B; b += 256) {
    tot += row_ws[2 * b];
    cnt += row_ws[2 * b + 1];
  }
  num = block_sum256(num, red);
  act = block_sum256(act, red);
  tot = block_sum256(tot, red);
  cnt = block_sum256(cnt, red);
  if (threadIdx.x == 0) {
    if (mode == TNX_AGG_TOKEN_MEAN) {
      out[0] = tot;
      out[1] = cnt;
    } else if (mode == TNX_AGG_SEQ_MEAN_TOKEN_SUM_NORM) {
      out[0] = tot;
      out[1] = norm > 0.f ? norm : act;
    } else {
      out[0] = num;
      out[1] = act;
    }
  }
}

// Agreement of two sets of per-token log-probabilities under a mask.  Row pass: eight masked
// sums in double (count, |dlogp|, |dp|, p_r, p_t, p_r^2, p_t^2, p_r * p_t) and two maxima per
// row; the finishing work-group adds the rows in order and forms the five figures.
constexpr int kDriftSums = 8;
__device__ __forceinline__ double block_sum256d(double v, double* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}
__device__ __forceinline__ float block_max256(float v, float* red) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

__global__ __launch_bounds__(256) void drift_rows_kernel(const float* a, const float* b, const float* mask,
                                                         int64_t T, double* row_ws) {
  __shared__ double redd[4];
  __shared__ float redf[4];
  const int64_t row = blockIdx.x;
  double s[kDriftSums] = {0, 0, 0, 0, 0, 0, 0, 0};
  float mx_d = 0.f, mx_p = 0.f;
  for (int64_t t = threadIdx.x; t < T; t += 256) {
    if (mask[row * T + t] == 0.f) continue;
    const float la = a[row * T + t], lb = b[row * T + t];
    const float d = fabsf(la - lb);
    const float pa = expf(la), pb = expf(lb);
    const float dp = fabsf(pa - pb);
    s[0] += 1.0;
    s[1] += d;
    s[2] += dp;
    s[3] += pa;
    s[4] += pb;
    s[5] += (double)pa * pa;
    s[6] += (double)pb * pb;
    s[7] += (double)pa * pb;
    mx_d = fmaxf(mx_d, d);
    mx_p = fmaxf(mx_p, dp);
  }
#pragma unroll
  for (int i = 0; i < kDriftSums; ++i) s[i] = block_sum256d(s[i], redd);
  mx_d = block_max256(mx_d, redf);
  mx_p = block_max256(mx_p, redf);
  if (threadIdx.x == 0) {
    double* o = row_ws + row * (kDriftSums + 2);
#pragma unroll
    for (int i = 0; i < kDriftSums; ++i) o[i] = s[i];
    o[kDriftSums] = mx_d;
    o[kDriftSums + 1] = mx_p;
  }
}

__global__ __launch_bounds__(256) void drift_finish_kernel(const double* row_ws, int64_t B, float* out) {
  __shared__ double redd[4];
  __shared__ float redf[4];
  double s[kDriftSums] = {0, 0, 0, 0, 0, 0, 0, 0};
  float mx_d = 0.f, mx_p = 0.f;
  for (int64_t r = threadIdx.x; r < B; r += 256) {
    const double* o = row_ws + r * (kDriftSums + 2);
#pragma unroll
    for (int i = 0; i < kDriftSums; ++i) s[i] += o[i];
    mx_d = fmaxf(mx_d, (float)o[kDriftSums]);
    mx_p = fmaxf(mx_p, (float)o[kDriftSums + 1]);
  }
#pragma unroll
  for (int i = 0; i < kDriftSums; ++i) s[i] = block_sum256d(s[i], redd);
  mx_d = block_max256(mx_d, redf);
  mx_p = block_max256(mx_p, redf);
  if (threadIdx.x == 0) {
    const double n = s[0] > 1.0 ? s[0] : 1.0;   // max(mask sum, 1)
    const double ma = s[3] / n, mb = s[4] / n;
    // sums of (p - mean)^2 * mask and of the cross term, from the raw moments (in double)
    const double va = (s[5] - 2.0 * ma * s[3] + ma * ma * s[0]) / n;
    const double vb = (s[6] - 2.0 * mb * s[4] + mb * mb * s[0]) / n;
    const double cov = (s[7] - ma * s[4] - mb * s[3] + ma * mb * s[0]) / n;
    const double vv = va * vb > 1e-12 ? va * vb : 1e-12;
    out[0] = (float)(s[1] / n);
    out[1] = mx_d;
    out[2] = (float)(s[2] / n);
    out[3] = mx_p;
    out[4] = (float)(cov / sqrt(vv));
  }
}

// Router: fp32 softmax of the bf16 scores, top-k (descending, lower expert id first among
// equals), renormalise, cast to bf16.  One wave per token; E <= 1024.
__global__ __launch_bounds__(64) void moe_route_kernel(const uint16_t* scores, int E, int k,
                                                       uint16_t* topk_w, int32_t* topk_id) {
  __shared__ float prob[1024];
  const int64_t m = blockIdx.x;
  const int lane = threadIdx.x;
  const uint16_t* sr = scores + m * E;
  float mx = -__builtin_inff();
  for (int e = lane; e < E; e += 64) mx = fmaxf(mx, bf2f(sr[e]));
  mx = wave_max(mx);
  float sum = 0.f;
  for (int e = lane; e < E; e += 64) {
    const float p = expf(bf2f(sr[e]) - mx);
    prob[e] = p;
    sum += p;
  }
  sum = wave_sum(sum);
  __syncthreads();
  // A NaN score makes every probability of the row NaN.  The selection below must still pick k
  // distinct experts inside [0, E) (the route sort and the grouped GEMM index memory with them), so
  // NaNs are ranked as -0.5: below every real probability, above the -1 that marks a taken
  // expert.  The row's weights are then written as NaN, and the NaN reaches the layer's output.
  bool bad = false;
  for (int e = lane; e < E; e += 64) {
    const float p = prob[e] / sum;
    const bool ok = p >= 0.f;
    bad |= !ok;
    prob[e] = ok ? p : -0.5f;
  }
  bad = __any(bad);
  __syncthreads();
  float wsum = 0.f;
  float sel_w = 0.f;   // lane j keeps the j-th selected weight (k <= 64)
  int sel_id = 0;
  for (int j = 0; j < k; ++j) {
    float best = -1.f;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float p = prob[e];
      if (p > best) { best = p; bi = e; }
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    if (lane == j) { sel_w = best; sel_id = bi; }
    wsum += best;
    if (lane == 0) prob[bi] = -1.f;
    __syncthreads();
  }
  if (lane < k) {
    topk_w[m * k + lane] = bad ? (uint16_t)0x7fc0 : f2bf(sel_w / wsum);
    topk_id[m * k + lane] = sel_id;
  }
}

// Counting sort of routes by expert; single work-group, stable in route order.  General form
// (any E): one thread per expert scans the routes.
__global__ __launch_bounds__(1024) void moe_sort_scan_kernel(const int32_t* topk_id, int64_t n_routes,
                                                             int E, int32_t* counts, int32_t* offsets,
                                                             int32_t* sorted_route) {
  extern __shared__ int32_t sh[];  // [E] counts, then [E] cursors
  int32_t* cnt = sh;
  int32_t* cur = sh + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int64_t r = threadIdx.x; r < n_routes; r += blockDim.x) atomicAdd(&cnt[topk_id[r]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t acc = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = acc;
      cur[e] = acc;
      counts[e] = cnt[e];
      acc += cnt[e];
    }
    offsets[E] = acc;
  }
  __syncthreads();
  // stable placement: expert e's routes in increasing route id, one thread per expert
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    int32_t pos = cur[e];
    for (int64_t r = 0; r < n_routes; ++r)
      if (topk_id[r] == e) sorted_route[pos++] = (int32_t)r;
  }
}

// The same for E <= 512 (every model on the path), one thread per ROUTE: the routes are walked
// 1024 at a time; within a wave, lanes of the same expert find each other by ballots and number
// themselves; a per-wave, per-expert count table in LDS gives each wave the routes of its
// expert in the waves before it; a cursor per expert carries over from one batch of 1024 to
// the next.  Three barriers per batch, no scan over the routes per expert.
constexpr int kSortMaxE = 512;
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int32_t* topk_id, int64_t n_routes,
                                                        int E, int32_t* counts, int32_t* offsets,
                                                        int32_t* sorted_route) {
  extern __shared__ int32_t sh[];  // [E] cursors, [16][E] per-wave counts of the current batch
  int32_t* cur = sh;
  int32_t* wcnt = sh + E;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < 17 * E; i += 1024) sh[i] = 0;
  __syncthreads();
  for (int64_t r = tid; r < n_routes; r += 1024) atomicAdd(&cur[topk_id[r]], 1);
  __syncthreads();
  if (tid == 0) {   // counts -> exclusive offsets (E <= 512: a few microseconds)
    int32_t acc = 0;
    for (int e = 0; e < E; ++e) {
      const int32_t c = cur[e];
      counts[e] = c;
      offsets[e] = acc;
      cur[e] = acc;
      acc += c;
    }
    offsets[E] = acc;
  }
  __syncthreads();
  const uint64_t below = lane ? (~0ull >> (64 - lane)) : 0ull;
  for (int64_t r0 = 0; r0 < n_routes; r0 += 1024) {
    const int64_t r = r0 + tid;
    const int e = r < n_routes ? topk_id[r] : -1;
    int rank = 0, mine = 0;
    bool leader = false;
    uint64_t todo = __ballot(e >= 0);
    while (todo) {   // wave-uniform: one turn per distinct expert in the wave
      const int l = __builtin_amdgcn_readfirstlane(__ffsll((long long)todo) - 1);
      const int le = __builtin_amdgcn_readlane(e, l);
      const uint64_t m = __ballot(e == le);
      if (e == le) {
        rank = __popcll(m & below);
        mine = __popcll(m);
        leader = lane == l;
      }
      todo &= ~m;
    }
    if (leader) wcnt[wave * E + e] = mine;
    __syncthreads();
    if (e >= 0) {
      int32_t base = cur[e];
      for (int w = 0; w < wave; ++w) base += wcnt[w * E + e];
      sorted_route[base + rank] = (int32_t)r;
    }
    __syncthreads();
    for (int x = tid; x < E; x += 1024) {
      int32_t s = 0;
#pragma unroll
      for (int w = 0; w < 16; ++w) s += wcnt[w * E + x];
      cur[x] += s;
    }
    __syncthreads();
    if (leader) wcnt[wave * E + e] = 0;
  }
}

__global__ void moe_combine_kernel(const uint16_t* y, const uint16_t* topk_w, int k, int64_t D,
                                   const uint16_t* residual, uint16_t* out) {
  const int64_t m = blockIdx.x;
  for (int64_t d = threadIdx.x; d < D; d += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < k; ++j) acc += bf2f(topk_w[m * k + j]) * bf2f(y[(m * k + j) * D + d]);
    float v = rbf(acc);
    if (residual) v = rbf(v + bf2f(residual[m * D + d]));
    out[m * D + d] = f2bf(v);
  }
}

// The same for D % 8 == 0 and k <= 16: eight columns per thread, the k expert rows fetched with
// independent 16-byte loads (same summation order per element: j ascending).
__global__ __launch_bounds__(256) void moe_combine_vec_kernel(const uint16_t* y, const uint16_t* topk_w, int k,
                                                              int64_t D, const uint16_t* residual,
                                                              uint16_t* out) {
  const int64_t m = blockIdx.x;
  const int64_t d0 = ((int64_t)blockIdx.y * 256 + threadIdx.x) * 8;
  if (d0 >= D) return;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  for (int j0 = 0; j0 < k; j0 += 8) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      v[u] = *reinterpret_cast<const u32x4*>(y + (m * k + min(j0 + u, k - 1)) * D + d0);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (j0 + u < k) {
        const float w = bf2f(topk_w[m * k + j0 + u]);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          acc[2 * q] += w * bflo(v[u][q]);
          acc[2 * q + 1] += w * bfhi(v[u][q]);
        }
      }
    }
  }
  u32x4 r = {0, 0, 0, 0};
  if (residual) r = *reinterpret_cast<const u32x4*>(residual + m * D + d0);
  u32x4 o;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    float lo = rbf(acc[2 * q]), hi = rbf(acc[2 * q + 1]);
    if (residual) {
      lo = rbf(lo + bflo(r[q]));
      hi = rbf(hi + bfhi(r[q]));
    }
    o[q] = pack2bf(lo, hi);
  }
  *reinterpret_cast<u32x4*>(out + m * D + d0) = o;
}

}  // namespace

extern "C" int tnx_fill_u32(void* stream, uint32_t* p, int64_t n, uint32_t value) {
  TNX_REQUIRE(p && n >= 0, "fill: bad arguments");
  if (n == 0) return TNX_OK;
  hipLaunchKernelGGL(fill_kernel, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, as_stream(stream), p, n, value);
  TNX_CHECK_LAUNCH("fill");
  return TNX_OK;
}

extern "C" int tnx_sample_commit(void* stream, const int32_t* ids, const float* logp, int64_t B,
                                 int32_t* tokens, int64_t tok_ld, float* logprobs, int32_t* done,
                                 const int32_t* eos, int n_eos, int32_t* step_ptr) {
  TNX_REQUIRE(ids && tokens && step_ptr && B > 0, "sample_commit: bad arguments");
  TNX_REQUIRE(n_eos == 0 || eos, "sample_commit: eos list is null");
  hipLaunchKernelGGL(sample_commit_kernel, dim3(1), dim3(256), 0, as_stream(stream), ids, logp, B,
                     tokens, tok_ld, logprobs, done, eos, n_eos, step_ptr);
  TNX_CHECK_LAUNCH("sample_commit");
  return TNX_OK;
}

extern "C" int tnx_grpo_ratio(void* stream, const float* logp, const float* old_logp,
                              const float* adv, int64_t N, int64_t tokens_per_seq, float eps_lo,
                              float eps_hi, float* ratio, float* loss, int32_t* clipped) {
  TNX_REQUIRE(logp && adv && N > 0 && tokens_per_seq > 0, "grpo_ratio: bad arguments");
  hipLaunchKernelGGL(grpo_ratio_kernel, dim3((unsigned)cdiv(N, 256)), dim3(256), 0,
                     as_stream(stream), logp, old_logp, adv, N, tokens_per_seq, eps_lo, eps_hi,
                     ratio, loss, clipped);
  TNX_CHECK_LAUNCH("grpo_ratio");
  return TNX_OK;
}

extern "C" int tnx_kl_divergence(void* stream, const float* logp, const float* ref_logp, int64_t N,
                                 int method, float clamp, float* kl) {
  TNX_REQUIRE(logp && ref_logp && kl && N > 0, "kl_divergence: bad arguments");
  TNX_REQUIRE(method >= TNX_KL_KL && method <= TNX_KL_LOW_VAR, "kl_divergence: bad method %d", method);
  hipLaunchKernelGGL(kl_divergence_kernel, dim3((unsigned)cdiv(N, 256)), dim3(256), 0, as_stream(stream),
                     logp, ref_logp, N, method, clamp, kl);
  TNX_CHECK_LAUNCH("kl_divergence");
  return TNX_OK;
}

extern "C" int tnx_aggregate_loss(void* stream, const float* per_token_loss, const float* mask, int64_t B,
                                  int64_t T, int mode, float norm, float* row_ws, float* out) {
  TNX_REQUIRE(per_token_loss && mask && row_ws && out, "aggregate_loss: null pointer");
  TNX_REQUIRE(B > 0 && T > 0 && B <= 0x7fffffffLL, "aggregate_loss: bad shape");
  TNX_REQUIRE(mode >= TNX_AGG_TOKEN_MEAN && mode <= TNX_AGG_SEQ_MEAN_TOKEN_SUM_NORM, "aggregate_loss: bad mode %d", mode);
  if (mode == TNX_AGG_SEQ_MEAN_TOKEN_SCALE || mode == TNX_AGG_SEQ_MEAN_TOKEN_SUM_NORM)
    TNX_REQUIRE(norm > 0.f, "aggregate_loss: norm must be positive");
  hipLaunchKernelGGL(agg_rows_kernel, dim3((unsigned)B), dim3(256), 0, as_stream(stream), per_token_loss, mask,
                     T, row_ws);
  TNX_CHECK_LAUNCH("aggregate_loss rows");
  hipLaunchKernelGGL(agg_finish_kernel, dim3(1), dim3(256), 0, as_stream(stream), row_ws, B, mode, norm, out);
  TNX_CHECK_LAUNCH("aggregate_loss finish");
  return TNX_OK;
}

extern "C" size_t tnx_aggregate_loss_segmented_ws_bytes(int64_t B, int num_segments) {
  return B > 0 && num_segments > 0 ? (size_t)B * ((size_t)num_segments + 1) * 2 * sizeof(float) : 0;
}

extern "C" int tnx_aggregate_loss_segmented(void* stream, const float* per_token_loss, const float* mask,
                                            const int32_t* segment_ids, int64_t B, int64_t T, int num_segments,
                                            int mode, float norm, float* ws, float* out) {
  TNX_REQUIRE(per_token_loss && mask && segment_ids && ws && out, "aggregate_loss_segmented: null pointer");
  TNX_REQUIRE(B > 0 && T > 0 && B <= 0x7fffffffLL, "aggregate_loss_segmented: bad shape");
  TNX_REQUIRE(num_segments >= 1 && num_segments <= (1 << 20), "aggregate_loss_segmented: num_segments=%d out of range", num_segments);
  TNX_REQUIRE(mode >= TNX_AGG_TOKEN_MEAN && mode <= TNX_AGG_SEQ_MEAN_TOKEN_SUM_NORM, "aggregate_loss_segmented: bad mode %d", mode);
  if (mode == TNX_AGG_SEQ_MEAN_TOKEN_SCALE)
    TNX_REQUIRE(norm > 0.f, "aggregate_loss_segmented: sequence-mean-token-scale needs an explicit positive norm");
  float* seg_ws = ws;
  float* row_ws = ws + (size_t)B * num_segments * 2;
  hipStream_t st = as_stream(stream);
  hipLaunchKernelGGL(agg_rows_kernel, dim3((unsigned)B), dim3(256), 0, st, per_token_loss, mask, T, row_ws);
  TNX_CHECK_LAUNCH("aggregate_loss_segmented rows");
  hipLaunchKernelGGL(agg_segments_kernel, dim3((unsigned)B), dim3(256), 0, st, per_token_loss, mask, segment_ids, T,
                     num_segments, seg_ws);
  TNX_CHECK_LAUNCH("aggregate_loss_segmented segments");
  hipLaunchKernelGGL(agg_segments_finish_kernel, dim3(1), dim3(256), 0, st, seg_ws, row_ws, B, num_segments, mode,
                     norm, out);
  TNX_CHECK_LAUNCH("aggregate_loss_segmented finish");
  return TNX_OK;
}

extern "C" size_t tnx_logp_drift_ws_bytes(int64_t B) {
  return B > 0 ? (size_t)B * (kDriftSums + 2) * sizeof(double) : 0;
}

extern "C" int tnx_logp_drift(void* stream, const float* rollout_logp, const float* trainer_logp,
                              const float* mask, int64_t B, int64_t T, void* ws, float* out5) {
  TNX_REQUIRE(rollout_logp && trainer_logp && mask && ws && out5, "logp_drift: null pointer");
  TNX_REQUIRE(B > 0 && T > 0 && B <= 0x7fffffffLL, "logp_drift: bad shape");
  TNX_REQUIRE(((uintptr_t)ws & 7) == 0, "logp_drift: the workspace must be 8-byte aligned");
  hipLaunchKernelGGL(drift_rows_kernel, dim3((unsigned)B), dim3(256), 0, as_stream(stream), rollout_logp,
                     trainer_logp, mask, T, (double*)ws);
  TNX_CHECK_LAUNCH("logp_drift rows");
  hipLaunchKernelGGL(drift_finish_kernel, dim3(1), dim3(256), 0, as_stream(stream), (const double*)ws, B, out5);
  TNX_CHECK_LAUNCH("logp_drift finish");
  return TNX_OK;
}

// The row moments of tnx_logp_drift_static live in this array instead of a caller's workspace.
// Each GPU the library runs on holds its own copy (kDriftStaticMaxRows * 10 doubles = 320 KiB)
// until the process ends.  Host code never uses the array's name as an address: the device
// address is looked up once per device and kept in g_drift_scratch_ptr.
constexpr int64_t kDriftStaticMaxRows = 4096;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) double drift_scratch[kDriftStaticMaxRows * (kDriftSums + 2)];
static double* g_drift_scratch_ptr[kMaxDevices] = {};
static std::mutex g_drift_scratch_mu;

extern "C" int64_t tnx_logp_drift_static_max_rows(void) { return kDriftStaticMaxRows; }

extern "C" int tnx_logp_drift_static(void* stream, const float* rollout_logp, const float* trainer_logp,
                                     const float* mask, int64_t B, int64_t T, float* out5) {
  TNX_REQUIRE(rollout_logp && trainer_logp && mask && out5, "logp_drift_static: null pointer");
  TNX_REQUIRE(B > 0 && T > 0, "logp_drift_static: bad shape");
  TNX_REQUIRE(B <= kDriftStaticMaxRows,
              "logp_drift_static: %lld rows exceed the built-in scratch of %lld rows; use tnx_logp_drift "
              "with a workspace", (long long)B, (long long)kDriftStaticMaxRows);
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    tnx_set_error("logp_drift_static: no current device (or its ordinal is above %d)", kMaxDevices - 1);
    return TNX_EINVAL;
  }
  double* ws = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_drift_scratch_mu);
    if (!g_drift_scratch_ptr[dev]) {   // first call on this device: look its copy of the array up
      void* p = nullptr;
      const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(drift_scratch));
      if (e != hipSuccess || !p) {
        tnx_set_error("logp_drift_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        return TNX_ELAUNCH;
      }
      g_drift_scratch_ptr[dev] = (double*)p;
    }
    ws = g_drift_scratch_ptr[dev];
  }
  // every row slot the finishing kernel reads is written by the row kernel of this call: nothing
  // has to be cleared between calls
  hipLaunchKernelGGL(drift_rows_kernel, dim3((unsigned)B), dim3(256), 0, as_stream(stream), rollout_logp,
                     trainer_logp, mask, T, ws);
  TNX_CHECK_LAUNCH("logp_drift_static rows");
  hipLaunchKernelGGL(drift_finish_kernel, dim3(1), dim3(256), 0, as_stream(stream), (const double*)ws, B, out5);
  TNX_CHECK_LAUNCH("logp_drift_static finish");
  return TNX_OK;
}

extern "C" int tnx_moe_route_topk(void* stream, const uint16_t* scores, int64_t M, int E, int k,
                                  uint16_t* topk_w, int32_t* topk_id) {
  TNX_REQUIRE(scores && topk_w && topk_id, "moe_route: null pointer");
  TNX_REQUIRE(M > 0 && E > 0 && E <= 1024 && k > 0 && k <= 64 && k <= E, "moe_route: bad shape E=%d k=%d", E, k);
  hipLaunchKernelGGL(moe_route_kernel, dim3((unsigned)M), dim3(64), 0, as_stream(stream), scores, E,
                     k, topk_w, topk_id);
  TNX_CHECK_LAUNCH("moe_route");
  return TNX_OK;
}

extern "C" int tnx_moe_sort_routes(void* stream, const int32_t* topk_id, int64_t M, int k, int E,
                                   int32_t* counts, int32_t* offsets, int32_t* sorted_route) {
  TNX_REQUIRE(topk_id && counts && offsets && sorted_route, "moe_sort: null pointer");
  TNX_REQUIRE(M > 0 && k > 0 && E > 0 && E <= 4096 && M * k <= (1 << 20), "moe_sort: bad shape");
  if (E <= kSortMaxE)
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), (size_t)(17 * E) * sizeof(int32_t),
                       as_stream(stream), topk_id, M * k, E, counts, offsets, sorted_route);
  else
    hipLaunchKernelGGL(moe_sort_scan_kernel, dim3(1), dim3(1024), (size_t)(2 * E) * sizeof(int32_t),
                       as_stream(stream), topk_id, M * k, E, counts, offsets, sorted_route);
  TNX_CHECK_LAUNCH("moe_sort");
  return TNX_OK;
}

extern "C" int tnx_moe_combine(void* stream, const uint16_t* y, const uint16_t* topk_w, int64_t M,
                               int k, int64_t D, const uint16_t* residual, uint16_t* out) {
  TNX_REQUIRE(y && topk_w && out && M > 0 && k > 0 && D > 0, "moe_combine: bad arguments");
  if (D % 8 == 0 && D <= 2048 * 65535)
    hipLaunchKernelGGL(moe_combine_vec_kernel, dim3((unsigned)M, (unsigned)cdiv(D, 2048)), dim3(256), 0,
                       as_stream(stream), y, topk_w, k, D, residual, out);
  else
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)M), dim3(256), 0, as_stream(stream), y,
                       topk_w, k, D, residual, out);
  TNX_CHECK_LAUNCH("moe_combine");
  return TNX_OK;
}
