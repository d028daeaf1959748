// Grouped GEMM over routed tokens for decode-sized expert batches: at most 16 rows per row block,
// i.e. a weight stream with almost no arithmetic per byte.  What such a launch costs is (a) the
// bytes in flight towards HBM and (b) the dequantisation (two VALU instructions per weight), so
// the kernel is built as 8 * (compute units) independent waves that each stream their share of
// the packed weights without ever meeting another wave after the prologue:
//
//   * one persistent work-group of eight waves per compute unit copies the expert offsets and the
//     sorted routes to LDS (the only dependent global round trip of the prologue), builds the
//     code-book table (the f16 level pairs of qgemm128.h: one v_perm_b32 per look-up address, one
//     v_fma_mix_f32 per weight, one v_cvt_pk_bf16_f32 per pair) and a list of the non-empty
//     (expert, 16-row block) pairs;
//   * the work items are (block, pair of adjacent 16-column tiles) in memory order; a wave takes
//     a contiguous run of them, so its codes are one contiguous stream (the k-tiles of a column
//     tile follow each other, and so do the tiles of an expert), which it requests kMoeRing
//     k-tiles ahead, across item boundaries, through a register ring; the codes are read once:
//     non-temporal loads;
//   * a run never spans more than two blocks (the host only picks this kernel when there are at
//     most as many blocks as waves), so the routes of a wave's rows -- the gather of the
//     activation fragments and the scatter of the outputs -- are looked up once, up front;
//   * activation fragments come straight from global memory in MFMA layout (the eight waves of a
//     work-group work on the same expert's rows, the requests meet in L1); rows the block does
//     not have are out-of-range buffer offsets, which read zeros and move no data;
//   * the loop has no barrier and no memory instruction behind a branch: the counted waits on
//     the ring are the minimum over the paths that reach them, so a tile stored only in the step
//     that finishes it would make the waits of the steps behind it stricter than the ring needs.
//     Finished tiles are parked in LDS and written out after the loop.  For the same reason the
//     first loads are issued in the order of the loop's (as in qgemm128.h);
//   * a k-tile is eight groups (k-step x column tile) of four look-ups, twelve conversion
//     instructions and one MFMA, software-pipelined by hand: the look-ups run two groups ahead of
//     the MFMA, the conversions one.
//
// Included by qlinear.hip after qgemm128.h.
#pragma once

namespace {

constexpr int kMoeRing = 4;                 // k-tiles in flight per wave
constexpr int kMoeWaves = 8;                // waves per work-group
constexpr int kMoeMaxRun = 8;               // items (tile pairs) a wave takes at most
// LDS behind the table: expert offsets [E + 1], sorted routes [n_routes], the block list
// ([0] = number of blocks, [2 + 2b] = expert, [3 + 2b] = row block), each rounded up to 16
// bytes, then 1 KiB per wave and item of its run for finished tiles.
constexpr size_t moe16_round16(size_t b) { return (b + 15) / 16 * 16; }
constexpr size_t moe16_meta_bytes(int64_t E, int64_t n_routes) {
  return moe16_round16((size_t)(E + 1) * 4) + moe16_round16((size_t)n_routes * 4) +
         moe16_round16((size_t)(2 + 2 * (E + n_routes / 16)) * 4);
}
constexpr size_t moe16_smem_bytes(int64_t E, int64_t n_routes) {
  return kBigLutBytes + moe16_meta_bytes(E, n_routes) + (size_t)kMoeWaves * kMoeMaxRun * 1024;
}

template <int I, int N, class F>
__device__ __forceinline__ void moe_static_for(F&& f) {
  if constexpr (I < N) {
    f(ic<I>{});
    moe_static_for<I + 1, N>(f);
  }
}

// MUL: the SiLU(gate) * up epilogue over interleaved gate / up tiles; SPT: scale slots per k-tile
// INT4: integer codes, converted without the table (Int4Magic in common.h; the level offsets are
// subtracted in the scale multiply-add)
template <bool MUL, int SPT, bool INT4>
__global__ __launch_bounds__(kMoeWaves * 64) void moe_gmm16_kernel(const QLArgs a, const int E) {
  constexpr int R = kMoeRing;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lm = lane & 15, lq = lane >> 4;
  const int n_routes = (int)a.M;
  int* offs = reinterpret_cast<int*>(smem + kBigLutBytes);
  int* routes = reinterpret_cast<int*>(smem + kBigLutBytes + moe16_round16((size_t)(E + 1) * 4));
  int* list = reinterpret_cast<int*>(smem + kBigLutBytes + moe16_round16((size_t)(E + 1) * 4) +
                                     moe16_round16((size_t)n_routes * 4));
  const uint32_t stage_lds =
      (uint32_t)(kBigLutBytes + moe16_meta_bytes(E, n_routes)) + (uint32_t)wv * (uint32_t)(kMoeMaxRun * 1024);
  // offsets and routes -> LDS, requested first; the table is built while they are in flight
  for (int i = tid; i <= E; i += kMoeWaves * 64) offs[i] = a.offsets[i];
  for (int i = tid; i < n_routes; i += kMoeWaves * 64) routes[i] = a.sorted_route[i];
  static_assert(kMoeWaves == 8, "the table is written by 512 threads");
  if constexpr (!INT4) {  // table entry e = f16 pair (level[e & 15], level[e >> 4]), 64 copies rotated over the banks
    const float lvl0 = rbf(code_level_imm(a.qtype, tid & 15)), lvl1 = rbf(code_level_imm(a.qtype, (tid >> 4) & 15));
    uint32_t* lut = reinterpret_cast<uint32_t*>(smem);
    const h16x2 h = {(_Float16)lvl0, (_Float16)lvl1};
    const uint32_t v = __builtin_bit_cast(uint32_t, h);
    const int e = tid & 255, c0 = (tid >> 8) * 32;
#pragma unroll
    for (int c = 0; c < 32; ++c) lut[e * 64 + ((c0 + c + lane) & 63)] = v;
  }
  __syncthreads();
  if (wv == 0) {  // non-empty (expert, row block) pairs in expert order: a running sum over the experts
    int carry = 0;
    for (int base = 0; base < E; base += 64) {
      const int e = base + lane;
      int nb = 0;
      if (e < E) nb = (offs[e + 1] - offs[e] + 15) >> 4;
      int incl = nb;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int t = __shfl_up(incl, o, 64);
        if (lane >= o) incl += t;
      }
      const int first = carry + incl - nb;
      for (int rb = 0; rb < nb; ++rb) {
        list[2 + 2 * (first + rb)] = e;
        list[3 + 2 * (first + rb)] = rb;
      }
      carry += __shfl(incl, 63, 64);
    }
    if (lane == 0) list[0] = carry;
  }
  __syncthreads();

  const int ktiles = (int)(a.K / KTILE), tp = (int)(a.N / 32);
  const int nblocks = __builtin_amdgcn_readfirstlane(list[0]);
  const int total = nblocks * tp;
  const int nw = (int)gridDim.x * kMoeWaves;
  const int per = (total + nw - 1) / nw;
  const int i0 = ((int)blockIdx.x * kMoeWaves + wv) * per, i1 = min(i0 + per, total);
  if (i0 >= i1) return;   // (no barrier below)

  // the one or two blocks of this wave's run
  const int bA = i0 / tp, bB = min(bA + 1, nblocks - 1);
  const int iA = bA * tp, iB = iA + tp;   // first items of the two blocks
  const int eA = __builtin_amdgcn_readfirstlane(list[2 + 2 * bA]), rbA = __builtin_amdgcn_readfirstlane(list[3 + 2 * bA]);
  const int eB = __builtin_amdgcn_readfirstlane(list[2 + 2 * bB]), rbB = __builtin_amdgcn_readfirstlane(list[3 + 2 * bB]);
  const int begA = __builtin_amdgcn_readfirstlane(offs[eA]) + rbA * 16;
  const int rowsA = min(16, __builtin_amdgcn_readfirstlane(offs[eA + 1]) - begA);
  const int begB = __builtin_amdgcn_readfirstlane(offs[eB]) + rbB * 16;
  const int rowsB = min(16, __builtin_amdgcn_readfirstlane(offs[eB + 1]) - begB);
  // lane lm gathers row lm of the block (activation fragments)
  const int gA = lm < rowsA ? routes[begA + lm] : -1;
  const int gB = lm < rowsB ? routes[begB + lm] : -1;
  const uint32_t xoffA = gA >= 0 ? ((uint32_t)(gA / a.x_div) * (uint32_t)a.K + (uint32_t)lq * 8u) * 2u : 0xfffffff0u;
  const uint32_t xoffB = gB >= 0 ? ((uint32_t)(gB / a.x_div) * (uint32_t)a.K + (uint32_t)lq * 8u) * 2u : 0xfffffff0u;
  // the route (= output row) of block row lane / 4: the row this lane writes when the tiles leave
  const int rfA = (lane >> 2) < rowsA ? routes[begA + (lane >> 2)] : -1;
  const int rfB = (lane >> 2) < rowsB ? routes[begB + (lane >> 2)] : -1;

  const rsrc_t rx = make_rsrc(a.x, (uint64_t)(a.M / a.x_div) * a.K * 2);
  const rsrc_t rc = make_rsrc(a.codes, (uint64_t)E * a.codes_stride * 4);
  const rsrc_t rs = make_rsrc(a.scales, (uint64_t)E * a.scales_stride * 2);
  const uint32_t lane_off = (uint32_t)lane * 4u;
  Int4Magic magic;
  if constexpr (INT4) magic.pin<false>();
  const uint32_t cvoff = (uint32_t)lane * 16u;
  const uint32_t svoff = (uint32_t)lm * (uint32_t)(SPT * 2);
  const uint32_t ctile = (uint32_t)ktiles * 1024u, stile = (uint32_t)ktiles * (uint32_t)(16 * SPT * 2);
  const uint32_t cexp = (uint32_t)(a.codes_stride * 4), sexp = (uint32_t)(a.scales_stride * 2);

  u32x4 ring_c[R][2], ring_x[R][4];
  // (a lane's scales: one 4-byte word for two slots, one 8-byte word for four; never a register
  // the lane does not use, which the allocator would hand to something else while the load that
  // writes it is still in flight -- a wait for everything outstanding)
  uint32_t ring_s[R][2][SPT / 2];
  f32x4 acc[2];
  zero_acc(acc[0]);
  zero_acc(acc[1]);

  // the request side walks (item, k-tile) R steps ahead of the multiply side; past the run's
  // end it keeps re-requesting the last k-tile (multiplied into accumulators nobody stores)
  int q_i = i0, q_kt = 0;
  auto issue = [&](auto Dc) {
    constexpr int D = decltype(Dc)::value;
    const bool inB = q_i >= iB;
    const int e = inB ? eB : eA;
    const int p = q_i - (inB ? iB : iA);
    const uint32_t cs = (uint32_t)e * cexp + (uint32_t)(2 * p) * ctile + (uint32_t)q_kt * 1024u;
    const uint32_t ss = (uint32_t)e * sexp + (uint32_t)(2 * p) * stile + (uint32_t)q_kt * (uint32_t)(16 * SPT * 2);
    const uint32_t xo = inB ? xoffB : xoffA;
    __builtin_amdgcn_sched_barrier(0);   // the loads of a step stay in this order, here and before the loop
#pragma unroll
    for (int j = 0; j < 4; ++j)
      ring_x[D][j] = __builtin_amdgcn_raw_buffer_load_b128(rx, xo, q_kt * (KTILE * 2) + j * 64, 0);
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      ring_c[D][nt] = __builtin_amdgcn_raw_buffer_load_b128(rc, cvoff, cs + (uint32_t)nt * ctile, kStreamOnce);
      if constexpr (SPT == 2) {
        ring_s[D][nt][0] = __builtin_amdgcn_raw_buffer_load_b32(rs, svoff, ss + (uint32_t)nt * stile, 0);
      } else {
        const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rs, svoff, ss + (uint32_t)nt * stile, 0);
        ring_s[D][nt][0] = v[0];
        ring_s[D][nt][1] = v[1];
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // advance, stopping at the run's last k-tile
    const bool last = q_i == i1 - 1 && q_kt == ktiles - 1;
    const bool wrap = q_kt == ktiles - 1 && !last;
    q_kt = last ? q_kt : (wrap ? 0 : q_kt + 1);
    q_i += wrap ? 1 : 0;
  };

  int c_i = i0, c_kt = 0;
  auto consume = [&](auto Dc) {
    constexpr int D = decltype(Dc)::value;
    // group g = (k-step g / 2, column tile g % 2): scale, code word, look-ups, conversion, MFMA
    auto scale_of = [&](int g) {
      const int j = g >> 1;
      if constexpr (SPT == 2) {
        const uint32_t w = ring_s[D][g & 1][0];
        return (j >> 1) ? bfhi(w) : bflo(w);
      } else {
        const uint32_t w = ring_s[D][g & 1][j >> 1];
        return (j & 1) ? bfhi(w) : bflo(w);
      }
    };
    uint32_t lp[3][4];
    u32x4 bw[2];
    auto look = [&](int g) {
      const uint32_t w = ring_c[D][g & 1][g >> 1];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if constexpr (INT4) {
          uint32_t e = int4_entry_offset(magic, w, k);
          asm volatile("" : "+v"(e));   // (stays where the look-up it replaces would be issued)
          lp[g % 3][k] = e;
        } else {
          lp[g % 3][k] = lds_ld32(__builtin_amdgcn_perm(w, lane_off, 0x0c0c0400u + ((uint32_t)k << 8)));
        }
      }
    };
    auto conv = [&](int g) {
      const float s = scale_of(g);
      const float b0 = INT4 ? s * -1032.0f : 0.0f, b1 = INT4 ? s * -72.0f : 0.0f;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        _Float16 l0, l1;
        level_pair<INT4>(lp[g % 3], k, l0, l1);
        bw[g & 1][k] = cvt_pk_bf16(__builtin_fmaf((float)l0, s, b0), __builtin_fmaf((float)l1, s, b1));
      }
    };
    look(0);
    look(1);
    __builtin_amdgcn_sched_barrier(0);
    conv(0);
    look(2);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      acc[g & 1] = mfma16(ring_x[D][g >> 1], bw[g & 1], acc[g & 1]);
      if (g + 1 < 8) conv(g + 1);
      if (g + 3 < 8) look(g + 3);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (c_kt == ktiles - 1 && c_i < i1) {   // the item's tile pair is complete (no global access in here)
      uint16_t* stage = reinterpret_cast<uint16_t*>(smem + stage_lds + (uint32_t)(c_i - i0) * 1024u);
      if constexpr (MUL) {   // even tile = gate, odd tile = up: one tile of act = f(gate) * up
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float g = rbf(acc[0][i]), u = rbf(acc[1][i]);
          stage[(lq * 4 + i) * 16 + lm] = f2bf(rbf(silu_bf16(g)) * u);
        }
      } else {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int i = 0; i < 4; ++i) stage[(lq * 4 + i) * 32 + nt * 16 + lm] = f2bf(acc[nt][i]);
      }
      zero_acc(acc[0]);
      zero_acc(acc[1]);
    }
    const bool wrap = c_kt == ktiles - 1;
    c_kt = wrap ? 0 : c_kt + 1;
    c_i += wrap ? 1 : 0;
  };

  moe_static_for<0, R>([&](auto d) { issue(d); });
  // whole turns of the ring, the steps past the run's end included: no branch around a load or a wait
  const int steps = (i1 - i0) * ktiles;
  for (int s = 0; s < steps; s += R) {
    moe_static_for<0, R>([&](auto d) {
      consume(d);
      issue(d);
    });
  }
  // write the run's tiles out: lane = (row, quarter of the row) of a 16-row tile
  asm volatile("" ::: "memory");   // (the reads below are of another type than the writes above; LDS keeps a wave's order)
  const int64_t ldy = MUL ? a.N / 2 : a.N;
  const rsrc_t ry = make_rsrc(a.y, (uint64_t)a.M * (uint64_t)ldy * 2);
  const int frow = lane >> 2, fch = lane & 3;
  for (int i = i0; i < i1; ++i) {
    const bool inB = i >= iB;
    const int p = i - (inB ? iB : iA);
    const int rt = inB ? rfB : rfA;
    const uint32_t src = stage_lds + (uint32_t)(i - i0) * 1024u;
    if constexpr (MUL) {
      const u32x2 v = *reinterpret_cast<const __attribute__((address_space(3))) u32x2*>(
          static_cast<uintptr_t>(src + (uint32_t)(frow * 32 + fch * 8)));
      const uint32_t off = rt >= 0 ? ((uint32_t)rt * (uint32_t)ldy + (uint32_t)(p * 16 + fch * 4)) * 2u : 0xfffffff0u;
      __builtin_amdgcn_raw_buffer_store_b64(v, ry, off, 0, 0);
    } else {
      const u32x4 v = lds_ld128(src + (uint32_t)(frow * 64 + fch * 16));
      const uint32_t off = rt >= 0 ? ((uint32_t)rt * (uint32_t)ldy + (uint32_t)(p * 32 + fch * 8)) * 2u : 0xfffffff0u;
      __builtin_amdgcn_raw_buffer_store_b128(v, ry, off, 0, 0);
    }
  }
}

}  // namespace
