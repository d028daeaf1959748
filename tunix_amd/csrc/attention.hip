// GQA attention over the KV cache with a wavefront-level online softmax.
//
// One wave owns a tile of 16 query vectors that share a (batch row, kv head): the G query
// heads of the group (decode), or G heads x 16/G consecutive positions (prefill).  Scores are
// computed transposed, S^T[key, query] = K . q^T, so that every lane ends up holding the
// probabilities of ONE query column for 8 keys -- exactly the A fragment of the P.V MFMA --
// and the max / sum of the online softmax are per-lane scalars reduced over 4 lanes.  V rows
// are loaded in their natural [key][dh] layout (256 B contiguous per key) and transposed
// inside each lane with v_perm_b32 to form B fragments; nothing goes through LDS.
#include <string.h>

#include <mutex>
#include <type_traits>

#include "common.h"
#include "gemm_tile.h"   // dma16, raw_rsrc, tnx_wait_vm

// Register stages of the key-block ring (head_dim <= 128).  Two: one block in flight while one is
// computed.  A compute unit draws 21-28 GB/s from memory whatever its waves request, so a
// third stage adds nothing to the stream, and its 72 registers push ring registers into AGPRs,
// whose copies wait on loads in flight (measured: 46.5 / 64.8 us with two stages against
// 47.9 / 67.3 us with three at contexts 528 / 768).
#ifndef TNX_ATTN_NS
#define TNX_ATTN_NS 2
#endif

namespace {

struct AttnArgs {
  int64_t B, T, S;
  int Hq, Hkv, dh, G, Gp;
  int gp_shift;                // Gp = 1 << gp_shift (the query group padded to a power of two)
  unsigned QT;                 // query tiles per row: ceil(T / (16 / Gp))
  unsigned QTG;                // (attn_tiles_kernel) groups of QW query tiles per row
  float scale_bf;  // bf16-rounded scale, 0 = none
  int window;
  int32_t pad_id;
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  const int32_t* tokens;       // token ids, or (seg_mode) the segment ids of a packed batch
  int64_t tok_ld;
  int seg_mode;                // 0: a key counts when its token != pad_id; 1: when its segment id equals the query's
  const int32_t* col_ptr;
  int kv_chunk, n_chunks;
  float* ws;
  uint16_t* out;
  // fused RoPE + cache write of the step's own token (decode, T == 1, no q/k norm, Llama
  // rotation): the query, key and value come from the qkv linear's output instead of q / the cache
  const float* qkv_ws;        // split-k partial planes [qkv_split][B][(Hq + 2 Hkv) * dh], or null
  const uint16_t* qkv;        // ... or the finished bf16 output
  int qkv_split;
  const float* rope_sin;      // fp32 [B, dh/2] of this step's positions; non-null switches the mode on
  const float* rope_cos;
};

constexpr float kNegBig = -1.0e30f;

// FUSE: 0 = q comes rotated, keys and values are in the cache; 1 = the fused rotation and cache
// write of a decode step (below), qkv taken from the finished output or from any number of
// partial planes; 2 = the same from at most eight partial planes and at most four query heads per
// kv head (one set of 3 x 64 lanes x 16 bytes per plane), all fetched in one round trip.
template <int DH, int FUSE, bool TOKVEC>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(DH > 128 ? 2 : 1, DH > 128 ? 2 : 1))) void attn_kernel(const AttnArgs a) {
  constexpr int KS = DH / 32;                 // k-steps of the QK product
  constexpr int NH = DH > 128 ? DH / 128 : 1; // 128-column halves of V / O
  constexpr int NS = DH > 128 ? 1 : TNX_ATTN_NS;        // register stages of the key-block pipeline
  const int lane = threadIdx.x, lm = lane & 15, lq = lane >> 4;
  const int chunk = blockIdx.x, hkv = blockIdx.y;
  // (shifts and one unsigned division: a general integer division costs some forty instructions,
  // and the chain in front of this kernel's first loads had several of them)
  const int PT = 16 >> a.gp_shift;                       // positions per query tile
  const unsigned bz = blockIdx.z;
  const int64_t b = FUSE != 0 ? bz : bz / a.QT;          // (the fused decode step has one query tile per row)
  const int qt = FUSE != 0 ? 0 : (int)(bz - (unsigned)b * a.QT);
  const int col0 = *a.col_ptr;

  // query column of this lane (as B-fragment column and as softmax owner)
  const int g = lm & (a.Gp - 1), tq = qt * PT + (lm >> a.gp_shift);
  const bool qvalid = g < a.G && tq < a.T;
  const int c_n = col0 + tq;                              // cache slot of the query token
  const int lo_n = a.window > 0 ? max(0, c_n - a.window + 1) : 0;
  const int64_t qvec = (b * a.T + (qvalid ? tq : 0)) * a.Hq + hkv * a.G + (qvalid ? g : 0);

  // key range of the tile
  const int t_last = min((int)a.T - 1, qt * PT + PT - 1);
  int k_hi = col0 + t_last;                               // inclusive
  int k_lo = a.window > 0 ? max(0, col0 + qt * PT - a.window + 1) : 0;
  if (a.kv_chunk > 0) {
    k_lo = max(k_lo, chunk * a.kv_chunk);
    k_hi = min(k_hi, chunk * a.kv_chunk + a.kv_chunk - 1);
  }

  constexpr bool fused = FUSE != 0;                         // T == 1: c_n = col0 for every lane
  u32x4 qf[KS];
#pragma unroll
  for (int j = 0; j < KS; ++j) {
    qf[j] = u32x4{0, 0, 0, 0};
    if (qvalid && !fused) qf[j] = *reinterpret_cast<const u32x4*>(a.q + qvec * DH + j * 32 + lq * 8);
  }
  // in fused mode the step's own key / value never come from the cache: the loop stops one key
  // short and they are added from registers at the end
  int key_hi = fused ? c_n - 1 : c_n;
  const bool writer = fused && col0 >= k_lo && col0 <= k_hi;   // the chunk that owns the new token
  if (fused) k_hi = min(k_hi, col0 - 1);

  f32x4 O[NH][8];
#pragma unroll
  for (int h = 0; h < NH; ++h)
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) O[h][jj] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = kNegBig, l_run = 0.f;

  const uint16_t* kbase = a.k + ((b * a.Hkv + hkv) * a.S) * DH;
  const uint16_t* vbase = a.v + ((b * a.Hkv + hkv) * a.S) * DH;
  const int32_t* tok = a.tokens + b * a.tok_ld;
  // what a key's id is compared with: the pad id (the key counts when it differs), or, for packed
  // batches, the segment id of this lane's query token (the key counts when it is equal).  The
  // query's id is fetched behind the first key blocks and planes (a load in front of them would
  // hold them back until the step counter it depends on has arrived), in both modes: a branch
  // around a load would make the counted waits behind it inexact.
  int32_t id_ref = a.pad_id;
  const bool id_equal = a.seg_mode != 0;
  auto fetch_query_id = [&]() {
    const int32_t id_q = tok[min((int64_t)c_n, a.tok_ld - 1)];
    id_ref = a.seg_mode ? id_q : a.pad_id;
  };
  const int vcol = (8 * lm) % (DH < 128 ? DH : 128);     // DH=64: upper lanes duplicate
  // TOKVEC: 16-byte token loads; the host chooses them when rows are 16-byte aligned and hold
  // whole groups of four slots (keys beyond the range are masked by the range test anyway).  A
  // compile-time choice: a branch around loads would make every wait behind it assume that the
  // shorter side was taken.

  // A ring of NS register stages: the loads of the next NS-1 key blocks are in flight while a
  // block is computed, so the memory system is never left idle behind a wave's softmax and
  // MFMAs.  One wave per SIMD owns the whole register file for this (nothing else hides the
  // latency: a wave has no second wave to alternate with).  Prefetches past the last block are
  // redirected to the last block (cache hits) rather than skipped: with every load issued
  // unconditionally the number of loads in flight is static, and the wait for a stage's data
  // does not have to drain the younger stages.
  struct Stage {
    u32x4 kf[2][KS];
    u32x4 vf[NH][8];
    int tk[8];
  };
  // K / V of this (row, kv head) and the row's token ids as buffer resources: a lane's byte
  // offset is a per-kernel constant plus the block's first key, so a block costs a handful of
  // address instructions, and keys past the cache (S not a multiple of 32, or a prefetch past
  // the end) read zeros; they are masked by the range test anyway.
  const uint32_t slab_bytes = (uint32_t)a.S * DH * 2u;
  const rsrc_t rk = make_rsrc(kbase, slab_bytes), rv = make_rsrc(vbase, slab_bytes);
  // (the row holds tok_ld ids: slots past them read zeros, and the range test masks them)
  const rsrc_t rtok = make_rsrc(tok, (uint64_t)min(a.S, a.tok_ld) * 4);
  const uint32_t koff = (uint32_t)(lm * DH + lq * 8) * 2u;           // + tt * 16 keys, + j * 64 B
  const uint32_t voff = (uint32_t)(4 * lq * DH + vcol) * 2u;         // + s keys, + 16 keys, + h * 256 B
  auto load_block = [&](int kb, Stage& sg) {
    const uint32_t kb_bytes = (uint32_t)kb * (DH * 2u);
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      const uint32_t o = koff + kb_bytes + (uint32_t)(tt * 16 * DH * 2);
#pragma unroll
      for (int j = 0; j < KS; ++j) sg.kf[tt][j] = __builtin_amdgcn_raw_buffer_load_b128(rk, o + (uint32_t)(j * 64), 0, kStreamOnce);
    }
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const uint32_t o = voff + kb_bytes + (uint32_t)(((s < 4 ? s : 12 + s)) * DH * 2);
#pragma unroll
      for (int h = 0; h < NH; ++h) sg.vf[h][s] = __builtin_amdgcn_raw_buffer_load_b128(rv, o + (uint32_t)(h * 256), 0, kStreamOnce);
    }
    // token ids of this lane's 8 keys (two runs of 4 consecutive slots), fetched unconditionally
    // together with K and V: a predicated load per key would serialise eight memory latencies
    if constexpr (TOKVEC) {
      const u32x4 t0 = __builtin_amdgcn_raw_buffer_load_b128(rtok, (uint32_t)(kb + 4 * lq) * 4u, 0, 0);
      const u32x4 t1 = __builtin_amdgcn_raw_buffer_load_b128(rtok, (uint32_t)(kb + 16 + 4 * lq) * 4u, 0, 0);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        sg.tk[s] = (int)t0[s];
        sg.tk[4 + s] = (int)t1[s];
      }
    } else {
#pragma unroll
      for (int s = 0; s < 8; ++s)
        sg.tk[s] = (int)__builtin_amdgcn_raw_buffer_load_b32(
            rtok, (uint32_t)(kb + (s < 4 ? 4 * lq + s : 16 + 4 * lq + (s - 4))) * 4u, 0, 0);
    }
  };
  auto compute_block = [&](int kb, const Stage& sg) {
    bool kvalid[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int key = kb + (s < 4 ? 4 * lq + s : 16 + 4 * lq + (s - 4));
      kvalid[s] = qvalid && key >= max(k_lo, lo_n) && key <= min(k_hi, key_hi) && ((sg.tk[s] == id_ref) == id_equal);
    }
    // ---- S^T = K . q^T ----
    f32x4 st[2];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      st[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < KS; ++j) st[tt] = mfma16(sg.kf[tt][j], qf[j], st[tt]);
    }
    float sv[8];
    float bmax = kNegBig;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      float x = rbf(st[s >> 2][s & 3]);
      if (a.scale_bf != 0.f) x = rbf(x * a.scale_bf);
      sv[s] = x;
      if (kvalid[s]) bmax = fmaxf(bmax, x);
    }
    bmax = fmaxf(bmax, __shfl_xor(bmax, 16, 64));
    bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
    const float m_new = fmaxf(m_run, bmax);
    const float alpha = __expf(m_run - m_new);
    m_run = m_new;
    float p[8], psum = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      p[s] = kvalid[s] ? __expf(sv[s] - m_new) : 0.f;
      psum += p[s];
    }
    l_run = l_run * alpha + psum;
    u32x4 pa;
    pa[0] = pack2bf(p[0], p[1]);
    pa[1] = pack2bf(p[2], p[3]);
    pa[2] = pack2bf(p[4], p[5]);
    pa[3] = pack2bf(p[6], p[7]);
    // ---- O = O * alpha + P . V ----
    // the running maximum settles after a few blocks: rescale O only when some column moved
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
      float ar[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) ar[i] = __shfl(alpha, 4 * lq + i, 64);
#pragma unroll
      for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int jj = 0; jj < 8; ++jj)
#pragma unroll
          for (int i = 0; i < 4; ++i) O[h][jj][i] *= ar[i];
    }
#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) {
        const uint32_t sel = (jj & 1) ? 0x07060302u : 0x05040100u;
        u32x4 bfrag;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          bfrag[r] = __builtin_amdgcn_perm(sg.vf[h][2 * r + 1][jj >> 1], sg.vf[h][2 * r][jj >> 1], sel);
        O[h][jj] = mfma16(pa, bfrag, O[h][jj]);
      }
  };
  {
    Stage sg[NS];
    const int kb0 = k_lo & ~31;
    const int kb_last = k_hi & ~31;
    const bool any = kb0 <= k_hi;
    // (issued even when the key range is empty: a block outside the slab reads zeros, and an
    // unconditional load keeps the counted waits behind it exact)
    auto issue_stage = [&](int u) { load_block(min(kb0 + 32 * u, kb_last), sg[u]); };
    auto issue_ring = [&]() {
#pragma unroll
      for (int u = 0; u < NS - 1; ++u) issue_stage(u);
    };
    // Without the fused rotation the first key blocks are requested right away.  With it the
    // partial planes of this step's q / k / v go first: a wave's loads return in order, so
    // planes requested behind 32 KiB of keys and values would only be usable once those have
    // arrived, and the rotation would start late instead of running while the blocks stream in.
    if constexpr (!fused) {
      issue_ring();
      fetch_query_id();
    }
    // the step's own key / value wait in LDS while the cached keys stream through the registers
    __shared__ u32x4 park[FUSE ? KS + NH : 1][64];
    if constexpr (fused) {
      u32x4 kn[KS], vn[NH];
      // ---- this step's q (G heads), k and v of the kv head from the qkv linear's output, RoPE
      // applied as the stand-alone kernel does; the first key blocks are already in flight ----
      const int ld = (a.Hq + 2 * a.Hkv) * DH;
      const int64_t plane = a.B * (int64_t)ld;
      const int64_t rowoff = b * (int64_t)ld;
      // The G query heads, the key head and the value head of this (row, kv head), (G + 2) * DH
      // values, are fetched once by the whole wave (16 bytes per lane and plane, all planes of
      // a group in flight together), summed in split order, rounded to bf16 and staged in LDS,
      // from where every lane picks the elements of its fragments.
      __shared__ float xs[18 * DH];
      // sine / cosine of this row's position: a per-step table (tnx_rope_table), computed with
      // the arithmetic of the stand-alone kernel; fetched together with the planes
      float sn[KS / 2][8], cs[KS / 2][8];
      {
        f32x4 s0[KS / 2], s1[KS / 2], c0[KS / 2], c1[KS / 2];
#pragma unroll
        for (int j = 0; j < KS / 2; ++j) {
          const int64_t o = b * (DH / 2) + j * 32 + lq * 8;
          s0[j] = *reinterpret_cast<const f32x4*>(a.rope_sin + o);
          s1[j] = *reinterpret_cast<const f32x4*>(a.rope_sin + o + 4);
          c0[j] = *reinterpret_cast<const f32x4*>(a.rope_cos + o);
          c1[j] = *reinterpret_cast<const f32x4*>(a.rope_cos + o + 4);
        }
        // three turns of 64 lanes x 16 bytes at a time (one turn set covers G = 4), every load of
        // the set issued before the first sum: a set costs one memory round trip, not one per turn
        const int n4 = (a.G + 2) * (DH / 4);
        constexpr bool planes_first = FUSE == 2;   // (the host checks qkv_ws, qkv_split <= 8 and G <= 4)
        // (called inside each of the two paths below, not behind their join: a use of the
        // oldest loads after a join of paths with different load sequences waits for everything)
        auto take_sincos = [&]() {
#pragma unroll
          for (int j = 0; j < KS / 2; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              sn[j][e] = s0[j][e]; sn[j][4 + e] = s1[j][e];
              cs[j][e] = c0[j][e]; cs[j][4 + e] = c1[j][e];
            }
        };
        auto load_planes = [&](int base, f32x4 (&p)[3][8]) {
#pragma unroll
          for (int tsel = 0; tsel < 3; ++tsel) {
            const int i4 = min(base + tsel * 64 + lane, n4 - 1);
            const int hsel = i4 / (DH / 4), d = (i4 % (DH / 4)) * 4;
            const int head = hsel < a.G ? hkv * a.G + hsel : (hsel == a.G ? a.Hq + hkv : a.Hq + a.Hkv + hkv);
            const int64_t o = rowoff + (int64_t)head * DH + d;
#pragma unroll
            for (int u = 0; u < 8; ++u)
              p[tsel][u] = *reinterpret_cast<const f32x4*>(a.qkv_ws + (int64_t)min(u, a.qkv_split - 1) * plane + o);
          }
        };
        auto sum_planes = [&](int base, const f32x4 (&p)[3][8]) {
#pragma unroll
          for (int tsel = 0; tsel < 3; ++tsel) {
            const int i4 = base + tsel * 64 + lane;
            f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < 8; ++u)
              if (u < a.qkv_split) acc += p[tsel][u];
            if (i4 < n4) *reinterpret_cast<f32x4*>(&xs[i4 * 4]) = f32x4{rbf(acc[0]), rbf(acc[1]), rbf(acc[2]), rbf(acc[3])};
          }
        };
        if constexpr (planes_first) {
          // the plane set, then the first block of the key / value ring, then the sums:
          // straight-line, so that the wait for the planes counts the ring's loads behind them
          // (the second block of the ring follows once the planes' registers are free: with
          // both in flight next to 24 plane vectors the ring would not get the registers it keeps
          // in the loop, and moving a register that is still being loaded waits for the load)
          f32x4 p[3][8];
          load_planes(0, p);
          __builtin_amdgcn_sched_barrier(0);
          issue_stage(0);
          fetch_query_id();
          __builtin_amdgcn_sched_barrier(0);
          sum_planes(0, p);
          take_sincos();
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int u = 1; u < NS - 1; ++u) issue_stage(u);
          __builtin_amdgcn_sched_barrier(0);
        } else {
          issue_ring();
          fetch_query_id();
          take_sincos();
          for (int i4 = lane; i4 < n4; i4 += 64) {
              const int hsel = i4 / (DH / 4), d = (i4 % (DH / 4)) * 4;
              const int head = hsel < a.G ? hkv * a.G + hsel : (hsel == a.G ? a.Hq + hkv : a.Hq + a.Hkv + hkv);
              const int64_t o = rowoff + (int64_t)head * DH + d;
              f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
              if (a.qkv_ws) {
                for (int z0 = 0; z0 < a.qkv_split; z0 += 8) {
                  f32x4 p[8];
#pragma unroll
                  for (int u = 0; u < 8; ++u)
                    p[u] = *reinterpret_cast<const f32x4*>(a.qkv_ws + (int64_t)min(z0 + u, a.qkv_split - 1) * plane + o);
#pragma unroll
                  for (int u = 0; u < 8; ++u)
                    if (z0 + u < a.qkv_split) acc += p[u];
                }
              } else {
                const u32x2 q = *reinterpret_cast<const u32x2*>(a.qkv + o);
                acc = f32x4{bflo(q[0]), bfhi(q[0]), bflo(q[1]), bfhi(q[1])};
              }
              *reinterpret_cast<f32x4*>(&xs[i4 * 4]) = f32x4{rbf(acc[0]), rbf(acc[1]), rbf(acc[2]), rbf(acc[3])};
          }
        }
        // the work-group is this one wave: LDS executes a wave's accesses in order, so the staged
        // values only need the compiler to keep the reads behind the writes (a work-group
        // barrier would also wait for the key / value loads in flight)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
      auto fetch8 = [&](int hsel, int d, float (&x)[8]) {
        const f32x4 v0 = *reinterpret_cast<const f32x4*>(&xs[hsel * DH + d]);
        const f32x4 v1 = *reinterpret_cast<const f32x4*>(&xs[hsel * DH + d + 4]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          x[e] = v0[e];
          x[4 + e] = v1[e];
        }
      };
      // rotate the head whose first column is `col`: pairs (d, d + DH/2) sit in k-steps j, j + KS/2
      auto rotated = [&](int hsel, u32x4 (&dst)[KS]) {
        float x[KS][8];
#pragma unroll
        for (int j = 0; j < KS; ++j) fetch8(hsel, j * 32 + lq * 8, x[j]);
#pragma unroll
        for (int j = 0; j < KS / 2; ++j) {
          float o1[8], o2[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float x1 = x[j][e], x2 = x[j + KS / 2][e];
            o1[e] = rbf(__fsub_rn(__fmul_rn(x1, cs[j][e]), __fmul_rn(x2, sn[j][e])));
            o2[e] = rbf(__fadd_rn(__fmul_rn(x2, cs[j][e]), __fmul_rn(x1, sn[j][e])));
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            dst[j][e] = pack2bf(o1[2 * e], o1[2 * e + 1]);
            dst[j + KS / 2][e] = pack2bf(o2[2 * e], o2[2 * e + 1]);
          }
        }
      };
      if (qvalid) rotated(g, qf);
#pragma unroll
      for (int j = 0; j < KS; ++j) kn[j] = u32x4{0, 0, 0, 0};
#pragma unroll
      for (int h = 0; h < NH; ++h) vn[h] = u32x4{0, 0, 0, 0};
      if (writer) {
        const int64_t slot = ((b * a.Hkv + hkv) * a.S + (col0 % (int)a.S)) * DH;
        if (lm == 0) {   // lanes (0, lq) hold the key as row 0 of an A fragment
          rotated(a.G, kn);
#pragma unroll
          for (int j = 0; j < KS; ++j)
            *reinterpret_cast<u32x4*>(const_cast<uint16_t*>(a.k) + slot + j * 32 + lq * 8) = kn[j];
        }
        if (lq == 0 && 8 * lm < (DH < 128 ? DH : 128)) {   // lanes (lm, 0) hold the value row of key 0
#pragma unroll
          for (int h = 0; h < NH; ++h) {
            float x[8];
            fetch8(a.G + 1, h * 128 + 8 * lm, x);
#pragma unroll
            for (int e = 0; e < 4; ++e) vn[h][e] = pack2bf(x[2 * e], x[2 * e + 1]);
            *reinterpret_cast<u32x4*>(const_cast<uint16_t*>(a.v) + slot + h * 128 + 8 * lm) = vn[h];
          }
        }
      }
#pragma unroll
      for (int j = 0; j < KS; ++j) park[j][lane] = kn[j];
#pragma unroll
      for (int h = 0; h < NH; ++h) park[KS + h][lane] = vn[h];
    }
    if (any) {
      // Whole turns of the ring without a branch inside (an exit in the middle of a turn makes
      // the compiler merge the stages' registers on the exit edges, and a copy of a register
      // that is still being loaded waits for everything in flight), then the last one or two
      // blocks, whose loads were issued by the turn before them.
      const int nblk = ((kb_last - kb0) >> 5) + 1;
      int i = 0;
      for (; i + NS <= nblk; i += NS) {
#pragma unroll
        for (int u = 0; u < NS; ++u) {
          const int kbu = kb0 + 32 * (i + u);
          load_block(min(kbu + 32 * (NS - 1), kb_last), sg[(u + NS - 1) % NS]);
          __builtin_amdgcn_sched_barrier(0);
          compute_block(kbu, sg[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < NS - 1; ++u)
        if (i + u < nblk) compute_block(kb0 + 32 * (i + u), sg[u]);
    }
    if (writer) {
      // the step's own key / value as a block of one key (at position col0) from registers
      Stage& one = sg[0];
#pragma unroll
      for (int j = 0; j < KS; ++j) {
        one.kf[0][j] = park[j][lane];
        one.kf[1][j] = u32x4{0, 0, 0, 0};
      }
#pragma unroll
      for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int sidx = 0; sidx < 8; ++sidx) one.vf[h][sidx] = sidx == 0 ? park[KS + h][lane] : u32x4{0, 0, 0, 0};
      const int own_tok = tok[col0];
#pragma unroll
      for (int sidx = 0; sidx < 8; ++sidx) one.tk[sidx] = own_tok;
      k_hi = col0;
      key_hi = col0;
      compute_block(col0, one);
    }
  }

  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);

  // O rows are query columns 4*lq + i; columns are d = h*128 + 8*lm + jj.
  const bool dvalid = 8 * lm < (DH < 128 ? DH : 128);
  if (a.kv_chunk <= 0 || a.n_chunks == 1) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = 4 * lq + i;
      const float l = __shfl(l_run, n, 64);
      const int gi = n & (a.Gp - 1), ti = qt * PT + (n >> a.gp_shift);
      if (!(gi < a.G && ti < a.T) || !dvalid) continue;
      const float inv = l > 0.f ? 1.0f / l : 0.f;
      uint16_t* o = a.out + ((b * a.T + ti) * a.Hq + hkv * a.G + gi) * DH;
#pragma unroll
      for (int h = 0; h < NH; ++h) {
        u32x4 w;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          w[r] = pack2bf(O[h][2 * r][i] * inv, O[h][2 * r + 1][i] * inv);
        *reinterpret_cast<u32x4*>(o + h * 128 + 8 * lm) = w;
      }
    }
    return;
  }
  // split: partial (m, l, O[dh]) per (query vector, chunk)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = 4 * lq + i;
    const float l = __shfl(l_run, n, 64);
    const float m = __shfl(m_run, n, 64);
    const int gi = n & (a.Gp - 1), ti = qt * PT + (n >> a.gp_shift);
    if (!(gi < a.G && ti < a.T)) continue;
    const int64_t qv = (b * a.T + ti) * a.Hq + hkv * a.G + gi;
    float* p = a.ws + (qv * a.n_chunks + chunk) * (DH + 2);
    if (lm == 0) {
      p[0] = m;
      p[1] = l;
    }
    if (!dvalid || l <= 0.f) continue;
#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) p[2 + h * 128 + 8 * lm + jj] = O[h][jj][i];
  }
}

// Many query positions per row (prefill, whole-sequence log-probability passes): the wave above
// loads 16 KB of keys and values per 32-key block for sixteen MFMAs, i.e. it runs at what a
// compute unit can draw from L2, not at its matrix rate.  This form gives one wave QW
// consecutive query tiles: every loaded block, and the in-lane transposition of its value rows,
// serves QW x 16 query columns.  Each tile sees the same 32-key blocks in the same order with
// the same arithmetic as it would in a wave of its own (a block wholly before a tile's window
// or after its causal limit leaves its running maximum, sum and output untouched: p = 0,
// alpha = exp(0)), so results are bit-identical to the kernel above.  No fused rotation, no key
// split (those are decode modes).
template <int DH, bool TOKVEC, int QW>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(1, 1))) void attn_tiles_kernel(const AttnArgs a) {
  constexpr int KS = DH / 32;
  constexpr int NH = DH > 128 ? DH / 128 : 1;
  constexpr int NS = 2;
  const int lane = threadIdx.x, lm = lane & 15, lq = lane >> 4;
  const int hkv = blockIdx.y;
  const int PT = 16 >> a.gp_shift;
  const unsigned bz = blockIdx.z;
  const int64_t b = bz / a.QTG;
  // (the longest tiles of a row are handed out first: a tile's work grows with its position)
  const int qt0 = ((int)a.QTG - 1 - (int)(bz - (unsigned)b * a.QTG)) * QW;
  const int col0 = *a.col_ptr;
  const int g = lm & (a.Gp - 1);

  int c_n[QW], lo_n[QW];
  bool qvalid[QW];
  u32x4 qf[QW][KS];
#pragma unroll
  for (int w = 0; w < QW; ++w) {
    const int tq = (qt0 + w) * PT + (lm >> a.gp_shift);
    qvalid[w] = g < a.G && tq < a.T;
    c_n[w] = col0 + tq;
    lo_n[w] = a.window > 0 ? max(0, c_n[w] - a.window + 1) : 0;
    const int64_t qvec = (b * a.T + (qvalid[w] ? tq : 0)) * a.Hq + hkv * a.G + (qvalid[w] ? g : 0);
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      qf[w][j] = u32x4{0, 0, 0, 0};
      if (qvalid[w]) qf[w][j] = *reinterpret_cast<const u32x4*>(a.q + qvec * DH + j * 32 + lq * 8);
    }
  }
  // key range of the QW tiles together
  const int t_last = min((int)a.T - 1, (qt0 + QW) * PT - 1);
  const int k_hi = col0 + t_last;
  const int k_lo = a.window > 0 ? max(0, col0 + qt0 * PT - a.window + 1) : 0;

  f32x4 O[QW][NH][8];
  float m_run[QW], l_run[QW];
#pragma unroll
  for (int w = 0; w < QW; ++w) {
    m_run[w] = kNegBig;
    l_run[w] = 0.f;
#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) O[w][h][jj] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const uint16_t* kbase = a.k + ((b * a.Hkv + hkv) * a.S) * DH;
  const uint16_t* vbase = a.v + ((b * a.Hkv + hkv) * a.S) * DH;
  const int32_t* tok = a.tokens + b * a.tok_ld;
  int32_t id_ref[QW];
  const bool id_equal = a.seg_mode != 0;
  const int vcol = (8 * lm) % (DH < 128 ? DH : 128);
  struct Stage {
    u32x4 kf[2][KS];
    u32x4 vf[NH][8];
    int tk[8];
  };
  const uint32_t slab_bytes = (uint32_t)a.S * DH * 2u;
  const rsrc_t rk = make_rsrc(kbase, slab_bytes), rv = make_rsrc(vbase, slab_bytes);
  const rsrc_t rtok = make_rsrc(tok, (uint64_t)min(a.S, a.tok_ld) * 4);
  const uint32_t koff = (uint32_t)(lm * DH + lq * 8) * 2u;
  const uint32_t voff = (uint32_t)(4 * lq * DH + vcol) * 2u;
  // (the blocks are re-read by the waves of the later tiles of this row: default cache policy)
  auto load_block = [&](int kb, Stage& sg) {
    const uint32_t kb_bytes = (uint32_t)kb * (DH * 2u);
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      const uint32_t o = koff + kb_bytes + (uint32_t)(tt * 16 * DH * 2);
#pragma unroll
      for (int j = 0; j < KS; ++j) sg.kf[tt][j] = __builtin_amdgcn_raw_buffer_load_b128(rk, o + (uint32_t)(j * 64), 0, 0);
    }
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const uint32_t o = voff + kb_bytes + (uint32_t)(((s < 4 ? s : 12 + s)) * DH * 2);
#pragma unroll
      for (int h = 0; h < NH; ++h) sg.vf[h][s] = __builtin_amdgcn_raw_buffer_load_b128(rv, o + (uint32_t)(h * 256), 0, 0);
    }
    if constexpr (TOKVEC) {
      const u32x4 t0 = __builtin_amdgcn_raw_buffer_load_b128(rtok, (uint32_t)(kb + 4 * lq) * 4u, 0, 0);
      const u32x4 t1 = __builtin_amdgcn_raw_buffer_load_b128(rtok, (uint32_t)(kb + 16 + 4 * lq) * 4u, 0, 0);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        sg.tk[s] = (int)t0[s];
        sg.tk[4 + s] = (int)t1[s];
      }
    } else {
#pragma unroll
      for (int s = 0; s < 8; ++s)
        sg.tk[s] = (int)__builtin_amdgcn_raw_buffer_load_b32(
            rtok, (uint32_t)(kb + (s < 4 ? 4 * lq + s : 16 + 4 * lq + (s - 4))) * 4u, 0, 0);
    }
  };
  auto compute_block = [&](int kb, const Stage& sg) {
    u32x4 pa[QW];
#pragma unroll
    for (int w = 0; w < QW; ++w) {
      bool kvalid[8];
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        const int key = kb + (s < 4 ? 4 * lq + s : 16 + 4 * lq + (s - 4));
        kvalid[s] = qvalid[w] && key >= max(k_lo, lo_n[w]) && key <= min(k_hi, c_n[w]) &&
                    ((sg.tk[s] == id_ref[w]) == id_equal);
      }
      f32x4 st[2];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        st[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < KS; ++j) st[tt] = mfma16(sg.kf[tt][j], qf[w][j], st[tt]);
      }
      float sv[8];
      float bmax = kNegBig;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        float x = rbf(st[s >> 2][s & 3]);
        if (a.scale_bf != 0.f) x = rbf(x * a.scale_bf);
        sv[s] = x;
        if (kvalid[s]) bmax = fmaxf(bmax, x);
      }
      bmax = fmaxf(bmax, __shfl_xor(bmax, 16, 64));
      bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
      const float m_new = fmaxf(m_run[w], bmax);
      const float alpha = __expf(m_run[w] - m_new);
      m_run[w] = m_new;
      float p[8], psum = 0.f;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        p[s] = kvalid[s] ? __expf(sv[s] - m_new) : 0.f;
        psum += p[s];
      }
      l_run[w] = l_run[w] * alpha + psum;
      pa[w][0] = pack2bf(p[0], p[1]);
      pa[w][1] = pack2bf(p[2], p[3]);
      pa[w][2] = pack2bf(p[4], p[5]);
      pa[w][3] = pack2bf(p[6], p[7]);
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
        float ar[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) ar[i] = __shfl(alpha, 4 * lq + i, 64);
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
          for (int jj = 0; jj < 8; ++jj)
#pragma unroll
            for (int i = 0; i < 4; ++i) O[w][h][jj][i] *= ar[i];
      }
    }
    // O += P . V: a value fragment is transposed once and multiplied with every tile's P
#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) {
        const uint32_t sel = (jj & 1) ? 0x07060302u : 0x05040100u;
        u32x4 bfrag;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          bfrag[r] = __builtin_amdgcn_perm(sg.vf[h][2 * r + 1][jj >> 1], sg.vf[h][2 * r][jj >> 1], sel);
#pragma unroll
        for (int w = 0; w < QW; ++w) O[w][h][jj] = mfma16(pa[w], bfrag, O[w][h][jj]);
      }
  };
  {
    Stage sg[NS];
    const int kb0 = k_lo & ~31;
    const int kb_last = k_hi & ~31;
    const bool any = kb0 <= k_hi;
#pragma unroll
    for (int u = 0; u < NS - 1; ++u) load_block(min(kb0 + 32 * u, kb_last), sg[u]);
#pragma unroll
    for (int w = 0; w < QW; ++w) {
      const int32_t id_q = tok[min((int64_t)c_n[w], a.tok_ld - 1)];
      id_ref[w] = a.seg_mode ? id_q : a.pad_id;
    }
    if (any) {
      const int nblk = ((kb_last - kb0) >> 5) + 1;
      int i = 0;
      for (; i + NS <= nblk; i += NS) {
#pragma unroll
        for (int u = 0; u < NS; ++u) {
          const int kbu = kb0 + 32 * (i + u);
          load_block(min(kbu + 32 * (NS - 1), kb_last), sg[(u + NS - 1) % NS]);
          __builtin_amdgcn_sched_barrier(0);
          compute_block(kbu, sg[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < NS - 1; ++u)
        if (i + u < nblk) compute_block(kb0 + 32 * (i + u), sg[u]);
    }
  }
  const bool dvalid = 8 * lm < (DH < 128 ? DH : 128);
#pragma unroll
  for (int w = 0; w < QW; ++w) {
    float lr = l_run[w];
    lr += __shfl_xor(lr, 16, 64);
    lr += __shfl_xor(lr, 32, 64);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = 4 * lq + i;
      const float l = __shfl(lr, n, 64);
      const int gi = n & (a.Gp - 1), ti = (qt0 + w) * PT + (n >> a.gp_shift);
      if (!(gi < a.G && ti < a.T) || !dvalid) continue;
      const float inv = l > 0.f ? 1.0f / l : 0.f;
      uint16_t* o = a.out + ((b * a.T + ti) * a.Hq + hkv * a.G + gi) * DH;
#pragma unroll
      for (int h = 0; h < NH; ++h) {
        u32x4 wv;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          wv[r] = pack2bf(O[w][h][2 * r][i] * inv, O[w][h][2 * r + 1][i] * inv);
        *reinterpret_cast<u32x4*>(o + h * 128 + 8 * lm) = wv;
      }
    }
  }
}

// The same for head_dim 128 with keys and values staged through LDS: a work-group of four waves
// takes 4 x QW consecutive query tiles of one (row, kv head), and every 32-key block is requested
// once per work-group straight into LDS (16 bytes per lane, key rows with their 16-byte chunks
// XOR-swizzled by row so that the fragment reads of 16 rows hit 16 bank groups; value rows as they
// are; the block's 32 token / segment ids next to them), two blocks in flight.  A wave reads its
// fragments from there instead of drawing them through its own loads in the MFMA operand layout,
// which the memory path serves a few lanes at a time, and two such work-groups per compute unit
// (227 registers per lane, 68 KB of LDS) put the softmax arithmetic of one wave under the MFMAs of
// another.  Two query tiles per wave: with three the kernel spills.  Every wave computes exactly
// the blocks attn_tiles_kernel would give it, in the same order with the same arithmetic: outputs
// are bit-identical.
typedef uint32_t __attribute__((address_space(3))) lds_word_t;
typedef u32x4 __attribute__((address_space(3))) lds_vec_t;
__device__ __forceinline__ u32x4 attn_lds128(uint32_t addr) {
  return *reinterpret_cast<const lds_vec_t*>(static_cast<uintptr_t>(addr));
}
constexpr uint32_t kWgStageBytes = 8192 + 8192 + 1024;   // 32 keys x 256 B, 32 values x 256 B, ids
// blocks in LDS: one computed, three in flight (three / six measured 3 % / 50 % slower: with six a
// compute unit holds one work-group instead of two)
constexpr int kWgStages = 4;
template <int QW>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_wg_kernel(const AttnArgs a) {
  constexpr int DH = 128, KS = 4;
  extern __shared__ __align__(16) unsigned char smem_a[];
  const uint32_t lds0 = lds_addr(smem_a);
  const int tid = threadIdx.x, lane = tid & 63, lm = lane & 15, lq = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hkv = blockIdx.y;
  const int PT = 16 >> a.gp_shift;
  const unsigned bz = blockIdx.z;
  const int64_t b = bz / a.QTG;
  // (the longest groups of a row are handed out first: a tile's work grows with its position)
  const int qt_wg = ((int)a.QTG - 1 - (int)(bz - (unsigned)b * a.QTG)) * (4 * QW);
  const int qt0 = qt_wg + wave * QW;
  const int col0 = *a.col_ptr;
  const int g = lm & (a.Gp - 1);

  int c_n[QW], lo_n[QW];
  bool qvalid[QW];
  u32x4 qf[QW][KS];
#pragma unroll
  for (int w = 0; w < QW; ++w) {
    const int tq = (qt0 + w) * PT + (lm >> a.gp_shift);
    qvalid[w] = g < a.G && tq < a.T;
    c_n[w] = col0 + tq;
    lo_n[w] = a.window > 0 ? max(0, c_n[w] - a.window + 1) : 0;
    const int64_t qvec = (b * a.T + (qvalid[w] ? tq : 0)) * a.Hq + hkv * a.G + (qvalid[w] ? g : 0);
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      qf[w][j] = u32x4{0, 0, 0, 0};
      if (qvalid[w]) qf[w][j] = *reinterpret_cast<const u32x4*>(a.q + qvec * DH + j * 32 + lq * 8);
    }
  }
  // key range of this wave's QW tiles (as in attn_tiles_kernel) and of the work-group's 4 QW
  const bool wave_live = qt0 * PT < a.T;
  const int k_hi = col0 + min((int)a.T - 1, (qt0 + QW) * PT - 1);
  const int k_lo = a.window > 0 ? max(0, col0 + qt0 * PT - a.window + 1) : 0;
  const int k_hi_wg = col0 + min((int)a.T - 1, (qt_wg + 4 * QW) * PT - 1);
  const int k_lo_wg = a.window > 0 ? max(0, col0 + qt_wg * PT - a.window + 1) : 0;
  const int kb0_wg = k_lo_wg & ~31;
  const int nblk_wg = (((k_hi_wg & ~31) - kb0_wg) >> 5) + 1;
  const int kb0 = k_lo & ~31, kb_last = k_hi & ~31;
  const bool any = wave_live && kb0 <= k_hi;

  f32x4 O[QW][8];
  float m_run[QW], l_run[QW];
#pragma unroll
  for (int w = 0; w < QW; ++w) {
    m_run[w] = kNegBig;
    l_run[w] = 0.f;
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) O[w][jj] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const uint16_t* kbase = a.k + ((b * a.Hkv + hkv) * a.S) * DH;
  const uint16_t* vbase = a.v + ((b * a.Hkv + hkv) * a.S) * DH;
  const int32_t* tok = a.tokens + b * a.tok_ld;
  const bool id_equal = a.seg_mode != 0;
  int32_t id_ref[QW];
#pragma unroll
  for (int w = 0; w < QW; ++w) {
    const int32_t id_q = tok[min((int64_t)c_n[w], a.tok_ld - 1)];
    id_ref[w] = a.seg_mode ? id_q : a.pad_id;
  }
  // A block that lies wholly inside every query's range of a tile, with no id to mask, takes the
  // same arithmetic without the per-key tests: the bounds of that, uniform over the wave.
  // (Packed batches compare ids per query and always take the general form.)
  int lo_max[QW], hi_min[QW];
#pragma unroll
  for (int w = 0; w < QW; ++w) {
    int lo = max(k_lo, lo_n[w]), hi = min(k_hi, c_n[w]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      lo = max(lo, __shfl_xor(lo, o, 64));
      hi = min(hi, __shfl_xor(hi, o, 64));
    }
    const bool full = __builtin_amdgcn_ballot_w64(qvalid[w]) == ~0ull && !id_equal;
    lo_max[w] = __builtin_amdgcn_readfirstlane(full ? lo : 0x7fffffff);
    hi_min[w] = __builtin_amdgcn_readfirstlane(hi);
  }
  const uint32_t slab_bytes = (uint32_t)a.S * DH * 2u;
  const u32x4 rk = raw_rsrc(kbase, slab_bytes), rv = raw_rsrc(vbase, slab_bytes);
  const u32x4 rtok = raw_rsrc(tok, (uint64_t)min(a.S, a.tok_ld) * 4);
  // thread t requests, per 16-row half of a block, the 16 bytes that land at byte 16 t of the half:
  // row t / 16, and of the key row the chunk (t % 16) ^ (row % 16)
  const uint32_t krow = (uint32_t)(tid >> 4);
  const uint32_t kreq = krow * 256u + ((uint32_t)(tid & 15) ^ krow) * 16u;
  const uint32_t vreq = krow * 256u + (uint32_t)(tid & 15) * 16u;
  auto request_block = [&](int i) {   // five requests per wave (the ids by every wave: same bytes, one count)
    const uint32_t base = lds0 + (uint32_t)(i % kWgStages) * kWgStageBytes + (uint32_t)wave * 1024u;
    const uint32_t kb_bytes = (uint32_t)(kb0_wg + 32 * i) * 256u;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      dma16(base + (uint32_t)c * 4096u, rk, kb_bytes + (uint32_t)c * 4096u + kreq, 0);
      dma16(base + 8192u + (uint32_t)c * 4096u, rv, kb_bytes + (uint32_t)c * 4096u + vreq, 0);
    }
    // ids kb .. kb + 255 (the block's 32 and whatever follows them; past the row: zeros)
    dma16(lds0 + (uint32_t)(i % kWgStages) * kWgStageBytes + 16384u, rtok, (uint32_t)(kb0_wg + 32 * i + 4 * lane) * 4u, 0);
  };
  auto compute_block = [&](int kb, uint32_t base) {
    u32x4 kf[2][KS], vf[8];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int j = 0; j < KS; ++j)
        kf[tt][j] = attn_lds128(base + (uint32_t)((tt * 16 + lm) * 256) + (((uint32_t)(j * 4 + lq) ^ (uint32_t)lm) * 16u));
#pragma unroll
    for (int s = 0; s < 8; ++s)
      vf[s] = attn_lds128(base + 8192u + (uint32_t)((s < 4 ? 4 * lq + s : 12 + 4 * lq + s) * 256) + (uint32_t)lm * 16u);
    const u32x4 t0 = attn_lds128(base + 16384u + (uint32_t)(4 * lq) * 4u);
    const u32x4 t1 = attn_lds128(base + 16384u + (uint32_t)(16 + 4 * lq) * 4u);
    int tk[8];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      tk[s] = (int)t0[s];
      tk[4 + s] = (int)t1[s];
    }
    // (pad mode: a key counts when its id differs from pad_id, the same test for every tile)
    bool idok[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) idok[s] = (tk[s] == a.pad_id) == id_equal;
    const bool ids_all = !id_equal && __builtin_amdgcn_ballot_w64(idok[0] && idok[1] && idok[2] && idok[3] && idok[4] &&
                                                                  idok[5] && idok[6] && idok[7]) == ~0ull;
    u32x4 pa[QW];
    auto tile_step = [&](int w, auto inside_c) {
      constexpr bool INSIDE = decltype(inside_c)::value;
      bool kvalid[8];
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        const int key = kb + (s < 4 ? 4 * lq + s : 16 + 4 * lq + (s - 4));
        kvalid[s] = INSIDE || (qvalid[w] && key >= max(k_lo, lo_n[w]) && key <= min(k_hi, c_n[w]) &&
                               ((tk[s] == id_ref[w]) == id_equal));
      }
      f32x4 st[2];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        st[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < KS; ++j) st[tt] = mfma16(kf[tt][j], qf[w][j], st[tt]);
      }
      float sv[8];
      float bmax = kNegBig;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        float x = rbf(st[s >> 2][s & 3]);
        if (a.scale_bf != 0.f) x = rbf(x * a.scale_bf);
        sv[s] = x;
        if (kvalid[s]) bmax = fmaxf(bmax, x);
      }
      bmax = fmaxf(bmax, __shfl_xor(bmax, 16, 64));
      bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
      const float m_new = fmaxf(m_run[w], bmax);
      const float alpha = __expf(m_run[w] - m_new);
      m_run[w] = m_new;
      float p[8], psum = 0.f;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        p[s] = kvalid[s] ? __expf(sv[s] - m_new) : 0.f;
        psum += p[s];
      }
      l_run[w] = l_run[w] * alpha + psum;
      pa[w][0] = pack2bf(p[0], p[1]);
      pa[w][1] = pack2bf(p[2], p[3]);
      pa[w][2] = pack2bf(p[4], p[5]);
      pa[w][3] = pack2bf(p[6], p[7]);
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
        float ar[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) ar[i] = __shfl(alpha, 4 * lq + i, 64);
#pragma unroll
        for (int jj = 0; jj < 8; ++jj)
#pragma unroll
          for (int i = 0; i < 4; ++i) O[w][jj][i] *= ar[i];
      }
    };
#pragma unroll
    for (int w = 0; w < QW; ++w) {
      if (ids_all && kb >= lo_max[w] && kb + 31 <= hi_min[w]) tile_step(w, std::true_type{});
      else tile_step(w, std::false_type{});
    }
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
      const uint32_t sel = (jj & 1) ? 0x07060302u : 0x05040100u;
      u32x4 bfrag;
#pragma unroll
      for (int r = 0; r < 4; ++r) bfrag[r] = __builtin_amdgcn_perm(vf[2 * r + 1][jj >> 1], vf[2 * r][jj >> 1], sel);
#pragma unroll
      for (int w = 0; w < QW; ++w) O[w][jj] = mfma16(pa[w], bfrag, O[w][jj]);
    }
  };
#pragma unroll
  for (int u = 0; u < kWgStages - 1; ++u)
    if (u < nblk_wg) request_block(u);
  for (int i = 0; i < nblk_wg; ++i) {
    // this wave's share of block i has landed (behind it: the requests of blocks i + 1 ..
    // i + stages - 2, five each; near the end, where fewer follow, everything is waited for) ...
    if (i + kWgStages - 2 < nblk_wg) tnx_wait_vm(5 * (kWgStages - 2));
    else tnx_wait_vm(0);
    __syncthreads();    // ... and everyone's; every wave is also done reading block i - 1, whose stage is refilled
    if (i + kWgStages - 1 < nblk_wg) request_block(i + kWgStages - 1);
    const int kb = kb0_wg + 32 * i;
    if (any && kb >= kb0 && kb <= kb_last) compute_block(kb, lds0 + (uint32_t)(i % kWgStages) * kWgStageBytes);
  }
#pragma unroll
  for (int w = 0; w < QW; ++w) {
    float lr = l_run[w];
    lr += __shfl_xor(lr, 16, 64);
    lr += __shfl_xor(lr, 32, 64);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = 4 * lq + i;
      const float l = __shfl(lr, n, 64);
      const int gi = n & (a.Gp - 1), ti = (qt0 + w) * PT + (n >> a.gp_shift);
      if (!(gi < a.G && ti < a.T)) continue;
      const float inv = l > 0.f ? 1.0f / l : 0.f;
      uint16_t* o = a.out + ((b * a.T + ti) * a.Hq + hkv * a.G + gi) * DH;
      u32x4 wv;
#pragma unroll
      for (int r = 0; r < 4; ++r) wv[r] = pack2bf(O[w][2 * r][i] * inv, O[w][2 * r + 1][i] * inv);
      *reinterpret_cast<u32x4*>(o + 8 * lm) = wv;
    }
  }
}

// out[qv, d] = bf16( sum_c e^{m_c - M} O_c[d] / sum_c e^{m_c - M} l_c )
// The (m, l) pairs of all chunks are fetched at once into LDS (one round trip instead of one
// dependent load per chunk and pass); every thread then forms M, the weights and the sums in
// chunk order, with its chunk outputs fetched eight at a time.  (Chunks without a key have
// l = 0 and an O nobody wrote: selected away, never multiplied.)
__global__ void attn_combine_kernel(const float* ws, int64_t n_qvec, int dh, int n_chunks,
                                    uint16_t* out) {
  extern __shared__ float ml[];   // [n_chunks][2]
  const int64_t qv = blockIdx.x;
  const int d = threadIdx.x;
  const float* p = ws + qv * n_chunks * (dh + 2);
  for (int i = d; i < 2 * n_chunks; i += blockDim.x) ml[i] = p[(i >> 1) * (dh + 2) + (i & 1)];
  __syncthreads();
  if (d >= dh) return;
  float M = kNegBig;
  for (int c = 0; c < n_chunks; ++c)
    if (ml[2 * c + 1] > 0.f) M = fmaxf(M, ml[2 * c]);
  float L = 0.f, o = 0.f;
  for (int c0 = 0; c0 < n_chunks; c0 += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = p[min(c0 + u, n_chunks - 1) * (dh + 2) + 2 + d];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = c0 + u;
      if (c < n_chunks) {
        const float l = ml[2 * c + 1];
        if (l > 0.f) {
          const float w = __expf(ml[2 * c] - M);
          L += w * l;
          o += w * v[u];
        }
      }
    }
  }
  out[qv * dh + d] = f2bf(L > 0.f ? o / L : 0.f);
}

int next_pow2(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}

}  // namespace

extern "C" size_t tnx_attn_ws_bytes(int64_t B, int64_t T, int64_t S, int Hq, int dh,
                                    int kv_chunk) {
  if (kv_chunk <= 0) return 0;
  const int64_t n_chunks = cdiv(S, kv_chunk);
  return (size_t)(B * T * Hq * n_chunks * (dh + 2)) * sizeof(float);
}

extern "C" int tnx_gqa_attn(void* stream, const tnx_attn_desc* d) {
  TNX_REQUIRE(d, "attn: null descriptor");
  TNX_REQUIRE(d->B > 0 && d->T > 0 && d->S > 0, "attn: B,T,S must be positive");
  TNX_REQUIRE(d->dh == 64 || d->dh == 128 || d->dh == 256, "attn: head_dim %d not in {64,128,256}", d->dh);
  TNX_REQUIRE(d->Hkv > 0 && d->Hq % d->Hkv == 0, "attn: Hq=%d not a multiple of Hkv=%d", d->Hq, d->Hkv);
  const int G = d->Hq / d->Hkv;
  TNX_REQUIRE(G <= 16, "attn: group size %d > 16 not supported", G);
  TNX_REQUIRE(d->kcache && d->vcache && (d->tokens || d->segment_ids) && d->col_ptr && d->out, "attn: null pointer");
  TNX_REQUIRE(d->kv_chunk >= 0 && d->kv_chunk % 32 == 0, "attn: kv_chunk must be a multiple of 32");
  TNX_REQUIRE(d->tok_ld > 0, "attn: tok_ld=%lld must be positive", (long long)d->tok_ld);
  AttnArgs a;
  a.B = d->B; a.T = d->T; a.S = d->S; a.Hq = d->Hq; a.Hkv = d->Hkv; a.dh = d->dh;
  a.G = G; a.Gp = next_pow2(G);
  a.gp_shift = 0;
  while ((1 << a.gp_shift) < a.Gp) ++a.gp_shift;
  a.QT = (unsigned)cdiv(d->T, 16 / a.Gp);
  a.QTG = 1;
  // bf16(scale), as a weak-typed python float multiplied into a bf16 array
  if (d->scale != 0.f) {
    uint32_t u; float f = d->scale; memcpy(&u, &f, 4);
    u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
    memcpy(&a.scale_bf, &u, 4);
  } else {
    a.scale_bf = 0.f;
  }
  a.window = d->window; a.pad_id = d->pad_id;
  a.q = d->q; a.k = d->kcache; a.v = d->vcache; a.tokens = d->segment_ids ? d->segment_ids : d->tokens; a.tok_ld = d->tok_ld;
  a.seg_mode = d->segment_ids ? 1 : 0;
  a.col_ptr = d->col_ptr; a.kv_chunk = d->kv_chunk;
  a.n_chunks = d->kv_chunk > 0 ? (int)cdiv(d->S, d->kv_chunk) : 1;
  a.ws = d->ws; a.out = d->out;
  a.qkv_ws = nullptr; a.qkv = nullptr; a.qkv_split = 0; a.rope_sin = nullptr; a.rope_cos = nullptr;
  if (d->rope_sin) {
    TNX_REQUIRE(d->T == 1 && d->dh == 128, "attn: the fused RoPE / cache write needs T == 1 and head_dim 128");
    TNX_REQUIRE(d->rope_cos && (d->qkv || d->qkv_ws), "attn: fused RoPE needs the sine / cosine table and the qkv output");
    if (d->qkv_ws) TNX_REQUIRE(d->qkv_split >= 1 && d->qkv_split <= 64, "attn: qkv_split=%d out of range", d->qkv_split);
    a.qkv_ws = d->qkv_ws; a.qkv = d->qkv; a.qkv_split = d->qkv_split;
    a.rope_sin = d->rope_sin; a.rope_cos = d->rope_cos;
  } else {
    TNX_REQUIRE(d->q, "attn: null pointer");
  }
  if (a.n_chunks > 1) TNX_REQUIRE(d->ws, "attn: split key range needs a workspace");
  // (the combine keeps the chunks' (max, sum) pairs in LDS: 8 bytes per chunk)
  TNX_REQUIRE(a.n_chunks <= 4096, "attn: %d key chunks (S / kv_chunk), at most 4096", a.n_chunks);
  const int PT = 16 / a.Gp;
  const int64_t QT = cdiv(d->T, PT);
  TNX_REQUIRE(d->B * QT <= 65535 * 32, "attn: too many query tiles");
  dim3 grid((unsigned)a.n_chunks, (unsigned)d->Hkv, (unsigned)(d->B * QT));
  hipStream_t st = as_stream(stream);
  const bool tv = (d->tok_ld % 4 == 0) && ((reinterpret_cast<uintptr_t>(a.tokens) & 15) == 0) && d->S % 4 == 0;
#define TNX_ATTN_LAUNCH(DH, FUSE)                                                                \
  do {                                                                                           \
    if (tv) hipLaunchKernelGGL((attn_kernel<DH, FUSE, true>), grid, dim3(64), 0, st, a);         \
    else hipLaunchKernelGGL((attn_kernel<DH, FUSE, false>), grid, dim3(64), 0, st, a);           \
  } while (0)
  // many query positions at head_dim 128, no key split, no fused rotation: keys and values through
  // LDS, eight query tiles per work-group
  constexpr int kWgTilesPerWave = 2;
  if (!a.rope_sin && a.n_chunks == 1 && d->dh == 128 && tv && QT >= 2 * 4 * kWgTilesPerWave &&
      (uint64_t)d->S * 256u < (1ull << 32) && d->B * cdiv(QT, 4 * kWgTilesPerWave) <= 65535) {
    a.QTG = (unsigned)cdiv(QT, 4 * kWgTilesPerWave);
    dim3 wgrid(1u, (unsigned)d->Hkv, (unsigned)(d->B * a.QTG));
    static std::once_flag wg_once;
    static hipError_t wg_rc = hipSuccess;
    std::call_once(wg_once, [] {
      wg_rc = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_wg_kernel<kWgTilesPerWave>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kWgStages * kWgStageBytes));
    });
    TNX_REQUIRE(wg_rc == hipSuccess, "attn: cannot raise the dynamic LDS limit");
    hipLaunchKernelGGL((attn_wg_kernel<kWgTilesPerWave>), wgrid, dim3(256), kWgStages * kWgStageBytes, st, a);
    TNX_CHECK_LAUNCH("gqa_attn (work-group tiles)");
    return TNX_OK;
  }
  // many query positions, no key split, no fused rotation: two query tiles per wave
  constexpr int kTilesPerWave = 2;
  if (!a.rope_sin && a.n_chunks == 1 && d->dh <= 128 && QT >= 2 * kTilesPerWave) {
    a.QTG = (unsigned)cdiv(QT, kTilesPerWave);
    dim3 tgrid(1u, (unsigned)d->Hkv, (unsigned)(d->B * a.QTG));
    if (d->dh == 64) {
      if (tv) hipLaunchKernelGGL((attn_tiles_kernel<64, true, kTilesPerWave>), tgrid, dim3(64), 0, st, a);
      else hipLaunchKernelGGL((attn_tiles_kernel<64, false, kTilesPerWave>), tgrid, dim3(64), 0, st, a);
    } else {
      if (tv) hipLaunchKernelGGL((attn_tiles_kernel<128, true, kTilesPerWave>), tgrid, dim3(64), 0, st, a);
      else hipLaunchKernelGGL((attn_tiles_kernel<128, false, kTilesPerWave>), tgrid, dim3(64), 0, st, a);
    }
    TNX_CHECK_LAUNCH("gqa_attn (tiles)");
    return TNX_OK;
  }
  switch (d->dh) {
    case 64: TNX_ATTN_LAUNCH(64, 0); break;
    case 128:
      if (a.rope_sin && a.qkv_ws && a.qkv_split <= 8 && G <= 4) TNX_ATTN_LAUNCH(128, 2);
      else if (a.rope_sin) TNX_ATTN_LAUNCH(128, 1);
      else TNX_ATTN_LAUNCH(128, 0);
      break;
    default: TNX_ATTN_LAUNCH(256, 0); break;
  }
#undef TNX_ATTN_LAUNCH
  TNX_CHECK_LAUNCH("gqa_attn");
  if (a.n_chunks > 1) {
    const int64_t nq = d->B * d->T * d->Hq;
    hipLaunchKernelGGL(attn_combine_kernel, dim3((unsigned)nq), dim3(d->dh), (size_t)a.n_chunks * 2 * sizeof(float), st,
                       a.ws, nq, d->dh, a.n_chunks, a.out);
    TNX_CHECK_LAUNCH("gqa_attn_combine");
  }
  return TNX_OK;
}
