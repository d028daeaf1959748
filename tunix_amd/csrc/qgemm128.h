// The quantised GEMM (rollout batch, prefill, per-token logps): one work-group = 8 waves = two
// per SIMD, output tile 16 * MT rows x (64 * NT) columns (MT = 8: 128 rows; 1, 2, 4 for decode
// batches of up to 16, 32, 64 rows); a wave covers all rows x (16 * NT) columns over one half
// of every k-tile.  At 128 rows the op sits past the MFMA/HBM ridge of the machine (2 * 128 flop
// per 0.53 B of weights), so the loop is built around keeping the matrix pipe fed:
//
//   * a k-tile (128 k) is four k-steps of 8 * NT MFMAs (16x16x32 bf16).  While the MFMAs of step
//     g run, the same wave converts the weights of step g+1 (two v_fma_mix_f32 + one
//     v_cvt_pk_bf16_f32 per code pair), issues the table look-ups of step g+2 and reads the
//     activation fragments of step g+1 -- a three-deep software pipeline that runs across
//     k-tile boundaries.  A step is written as units in issue order (one MFMA with its share
//     of that work each) behind scheduling barriers: left to the scheduler, the conversions
//     bunch up and pull look-ups that have not returned yet into waits;
//   * the code book is an LDS table of f16 level pairs indexed by a code byte, replicated 64
//     times with a 256-byte entry stride, so that the LDS address of a look-up is one
//     v_perm_b32: 0x10000 | (byte << 8) | (lane << 2); every bf16-rounded level is exact in
//     f16, and v_fma_mix_f32 multiplies the f16 half it selects with the fp32 scale in one
//     instruction;
//   * activations are double-buffered in LDS (one barrier per k-tile) and go there straight
//     from memory (16 bytes per lane, unpadded rows with XOR-swizzled chunks); packed codes and
//     scales come through a three-deep register ring filled by buffer loads whose per-k-tile
//     offset is a scalar, so the loop has no per-load address arithmetic.
//
// Included by qlinear.hip after QLArgs / store_tile.
#pragma once

namespace {

typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) uint32_t lds_u32;
typedef __attribute__((address_space(3))) u32x4 lds_u32x4;

constexpr int kBigLutBytes = 256 * 256;
// LDS: two activation tiles of max(32, rows) rows x 128 k (256-byte rows whose 16-byte chunks
// are XOR-swizzled by row) from address 0, the table at 64 KiB, adapter fragments (2 KiB per
// column tile) behind it
constexpr uint32_t kBigLutBase = 0x10000, kBigAdapterBase = kBigLutBase + kBigLutBytes;
constexpr size_t big_abytes(int mt) { return (size_t)(mt < 2 ? 32 : 16 * mt) * KTILE * 2; }
constexpr size_t big_smem_bytes(int nt, int mt) { return kBigAdapterBase + 4 * (size_t)nt * 2048; }
static_assert(2 * big_abytes(8) <= kBigLutBase, "the activation tiles end where the table starts");

// LDS accesses by absolute LDS byte address (the dynamic LDS block of these kernels starts at
// address 0: they declare no static LDS).
__device__ __forceinline__ uint32_t lds_ld32(uint32_t addr) {
  return *reinterpret_cast<const lds_u32*>(static_cast<uintptr_t>(addr));
}
__device__ __forceinline__ u32x4 lds_ld128(uint32_t addr) {
  return *reinterpret_cast<const lds_u32x4*>(static_cast<uintptr_t>(addr));
}
__device__ __forceinline__ void lds_st128(uint32_t addr, u32x4 v) {
  *reinterpret_cast<lds_u32x4*>(static_cast<uintptr_t>(addr)) = v;
}

template <int V>
using ic = std::integral_constant<int, V>;

// Optional phase time stamps of work-group (0,0,0) for kernel tuning (off in the product build).
#ifdef TNX_TIMING
__device__ unsigned long long tnx_stamps[8];
#define TNX_STAMP(i)                                                                     \
  do {                                                                                   \
    if (threadIdx.x == 0 && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0)       \
      tnx_stamps[i] = __builtin_amdgcn_s_memrealtime();                                      \
  } while (0)
#else
#define TNX_STAMP(i) do {} while (0)
#endif

// 512 threads: waves 0-3 and 4-7 share the four column groups and split every k-tile between
// them (k-steps 0,1 | 2,3), which puts two waves on each SIMD at 256 registers each.
// MT = row tiles of 16 (8 for 65+ rows; 1, 2, 4 for decode batches of up to 16, 32, 64 rows: the
// weight stream and its dequantisation are the same, the MFMA, fragment and activation work
// shrink with the rows).
// INT4: integer codes, converted without the table (Int4Magic in common.h).
template <int NT, int SPT, int MT, bool INT4 = false>
__global__ __launch_bounds__(512)
void qgemm128_kernel(const QLArgs a) {
  constexpr int HM = (MT + 1) / 2, PF = 3;   // HM: row tiles a wave finishes after the k halves meet
  constexpr int ROWS = 16 * MT;
  constexpr int AP = (ROWS + 31) / 32;       // passes of the activation copy (512 threads x 16 B = 32 rows)
  constexpr int SW = SPT / 2;  // scales of one wave's two k-steps
  constexpr uint32_t ABYTES = (uint32_t)big_abytes(MT);
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6), wn = wv & 3, kh = wv >> 2;  // wave-uniform
  const int lm = lane & 15, lq = lane >> 4;
  TNX_STAMP(0);
  // LDS is addressed absolutely below (table at 0): the dynamic block starts at LDS address 0
  // because this kernel declares no static LDS, which the host checks before the first launch.
  // Pull the whole argument block into SGPRs with one batch of scalar loads: left alone, the
  // compiler sinks each field's load next to its first use, and the prologue pays one scalar
  // memory round trip after the other.
  asm volatile("" ::"s"(a.M), "s"(a.K), "s"(a.N), "s"(a.qtype), "s"(a.x), "s"(a.codes), "s"(a.scales),
               "s"(a.lora_rank), "s"(a.lora_nseg), "s"(a.lora_seg_end[0]), "s"(a.lora_seg_end[1]),
               "s"(a.lora_seg_end[2]), "s"(a.lora_seg_toff[0]), "s"(a.lora_seg_toff[1]),
               "s"(a.lora_seg_toff[2]), "s"(a.lora_seg_toff[3]));
  asm volatile("" ::"s"(a.t_ld), "s"(a.t), "s"(a.lora_b), "s"(a.lora_scale), "s"(a.epilogue), "s"(a.y),
               "s"(a.split_k), "s"(a.ws), "s"(a.ktiles_per_split), "s"(a.next_a_t), "s"(a.next_rank),
               "s"(a.next_tpart));
  // the two code-book levels of this thread's table entry, from literals: nothing at the start
  // of the kernel waits on memory except the loads of the first tiles
  const float lvl0 = rbf(code_level_imm(a.qtype, tid & 15)), lvl1 = rbf(code_level_imm(a.qtype, (tid >> 4) & 15));
  const uint32_t lane_off = (uint32_t)lane * 4u | kBigLutBase;   // byte 2 = 1: the table's base
  Int4Magic magic;
  if constexpr (INT4) magic.pin<true>();
  // entry j of a k-step's code dword: Int4Magic's, or the table's entry for byte j
  auto level_entry = [&](uint32_t w, int j) -> uint32_t {
    if constexpr (INT4) {
      // (tied to its place in the unit order like the look-up it replaces: an instruction without
      // side effects is otherwise free to move across the scheduling barriers)
      uint32_t e = int4_entry(magic, w, j);
      asm volatile("" : "+v"(e));
      return e;
    } else {
      return lds_ld32(__builtin_amdgcn_perm(w, lane_off, 0x0c020400u + ((uint32_t)j << 8)));
    }
  };
  const int64_t m0 = (int64_t)blockIdx.x * ROWS;
  const int64_t ntile0 = ((int64_t)blockIdx.y * 4 + wn) * NT;
  const int64_t ntiles = a.N / 16;
  const int ktiles = (int)(a.K / KTILE);
  const int kt_begin = blockIdx.z * a.ktiles_per_split;
  const int kt_end = min(ktiles, kt_begin + a.ktiles_per_split);

  const u32x4 rx = raw_rsrc(a.x, (uint64_t)a.M * a.K * 2);
  const uint64_t ntk = (uint64_t)ntiles * ktiles;
  const rsrc_t rc = make_rsrc(a.codes, ntk * 1024);
  const rsrc_t rs = make_rsrc(a.scales, ntk * 16 * SPT * 2 + 16);
  // Per-thread offsets (32 bit: the host checks the 4 GiB limits); the k-tile enters as the
  // scalar offset of the load.  Rows past M and column tiles past N start beyond the buffer
  // and read zeros.  A lane's 16 bytes of codes are four k-steps: this wave takes its half.
  uint32_t coff[NT], soff[NT];
  // Activation tiles go from memory straight into LDS, 16 bytes per lane: a wave's 64 lanes fill
  // 1 KB = four consecutive 256-byte rows, the 512 threads 32 rows per pass.  Thread t fills
  // chunk t % 16 of rows t / 16 + 32 c and fetches for it the k-chunk (t % 16) ^ (row % 16):
  // the 16 lanes that read one k-chunk of 16 consecutive rows for an MFMA fragment then hit 16
  // different bank groups.
  const uint32_t chs = (uint32_t)((tid & 15) ^ ((tid >> 4) & 15));
  const uint32_t xbase = ((uint32_t)(m0 + (tid >> 4)) * (uint32_t)a.K + chs * 8u) * 2u;
  // (dma16 of gemm_tile.h: the compiler does not count these loads, the waits for them are
  // written by hand)
  const uint32_t dma_wave = (uint32_t)wv * 1024u;      // this wave's four rows within a 32-row pass
  const uint32_t xstride = 32u * (uint32_t)a.K * 2u;  // 32 rows further per chunk
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const uint32_t tile0 = (uint32_t)(ntile0 + nt) * (uint32_t)ktiles;
    coff[nt] = tile0 * 1024u + (uint32_t)lane * 16u + (uint32_t)kh * 8u;
    soff[nt] = (tile0 * 16u + (uint32_t)lm) * (uint32_t)(SPT * 2) + (SPT == 4 ? (uint32_t)kh * 4u : 0u);
  }

  TNX_STAMP(6);
  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) zero_acc(acc[mt][nt]);

  u32x2 ring_c[PF][NT];
  uint32_t ring_s[PF][NT];
  float sc[PF][NT][SW];   // the scales of a ring stage as fp32
  u32x4 af[2][MT];        // activation fragments of this wave's two k-steps
  u32x4 bfr[2][NT];       // weight fragments of the two k-steps
  uint32_t lp[2][NT][4];  // table entries (f16 level pairs): [s] is read by the steps of parity s, written by the others

  auto load_w = [&](auto Dc, int kt) {
    constexpr int D = decltype(Dc)::value;
    const int ktc = min(kt, ktiles - 1);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      ring_c[D][nt] = __builtin_amdgcn_raw_buffer_load_b64(rc, coff[nt], ktc * 1024, 0);
      ring_s[D][nt] = __builtin_amdgcn_raw_buffer_load_b32(rs, soff[nt], ktc * (16 * SPT * 2), 0);
    }
  };
  // What the first k-tile needs is requested here, ahead of the adapter bookkeeping below (a
  // few hundred scalar and vector instructions that touch no memory).
  if (kt_begin < kt_end) {
#pragma unroll
    for (int c = 0; c < AP; ++c)
      dma16(dma_wave + (uint32_t)c * 8192u, rx, xbase + (uint32_t)c * xstride, kt_begin * (KTILE * 2));
    load_w(ic<0>{}, kt_begin);
  }
  __builtin_amdgcn_sched_barrier(0);

  // LoRA delta through the activation pipeline: the "k-tile" after the last real one is the
  // 128-row block of t = bf16(x . A), columns [toff_a, +64) | [toff_b, +64) (the one or two
  // adapter segments this work-group's columns belong to), so that it is in LDS when the main
  // loop ends; the B^T fragments of this wave's columns are fetched at kernel start.
  int toff[NT];
  int toff_a = 0, toff_b = 0;
  bool lora_fast = a.lora_rank > 0 && a.lora_rank <= 64 && blockIdx.z == 0;
  if (a.lora_rank > 0) {
    if (a.lora_nseg < 0) {  // interleaved gate / up pair: even tiles segment 0, odd tiles segment 1
      toff_a = 0;
      toff_b = a.lora_rank;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) toff[nt] = (int)((ntile0 + nt) & 1) * a.lora_rank;
    } else {
      // segments are contiguous column ranges: index and offset by straight selects (no
      // branches, the argument arrays stay in SGPRs); N < 2^31, the host checks the 4 GiB limits
      int e0 = (int)a.lora_seg_end[0], e1 = (int)a.lora_seg_end[1], e2 = (int)a.lora_seg_end[2];
      int t0 = a.lora_seg_toff[0], t1 = a.lora_seg_toff[1], t2 = a.lora_seg_toff[2], t3 = a.lora_seg_toff[3];
      // opaque copies: otherwise the selects below are folded back into indexed loads from the
      // argument block, one more scalar memory round trip each
      asm volatile("" : "+s"(e0), "+s"(e1), "+s"(e2), "+s"(t0), "+s"(t1), "+s"(t2), "+s"(t3));
      auto seg_idx = [&](int ntile) {
        const int col = ntile * 16;
        return (int)(a.lora_nseg > 1 && col >= e0) + (int)(a.lora_nseg > 2 && col >= e1) +
               (int)(a.lora_nseg > 3 && col >= e2);
      };
      auto idx_toff = [&](int i) {
        // bit selects (a chain of ?: over an index becomes a table in private memory)
        auto pick = [](int cur, int cand, bool c) { return cur ^ ((cur ^ cand) & (0 - (int)c)); };
        return pick(pick(pick(t0, t1, i == 1), t2, i == 2), t3, i == 3);
      };
      const int last = (int)ntiles - 1;
      const int wg_nt0 = (int)blockIdx.y * 4 * NT;
      const int ia = seg_idx(wg_nt0), ib = seg_idx(min(wg_nt0 + 4 * NT - 1, last));
      toff_a = idx_toff(ia);
      toff_b = idx_toff(ib);
      // the tile is shared by all waves: a work-group spanning three segments falls back to
      // fragments from global memory (decided identically in every thread, no LDS involved)
      lora_fast = lora_fast && ib - ia <= 1;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) toff[nt] = idx_toff(seg_idx(min((int)ntile0 + nt, last)));
    }
  }
  // B^T fragments of the adapter for this column group: fetched now, parked in the group's
  // 4 KiB of LDS behind the activation buffers until the epilogue (both waves of the group
  // write the same values; the barriers of the main loop order them before the reads)
  const uint32_t lb_lds = kBigAdapterBase + (uint32_t)wn * (uint32_t)(NT * 2048) + (uint32_t)lane * 16u;
  uint32_t tbase = 0;
  u32x4 lbv[NT][2];  // live only until the main loop starts
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int j = 0; j < 2; ++j) lbv[nt][j] = u32x4{0, 0, 0, 0};
  // (issued behind the first weight and activation loads: at kernel start every buffer is a
  // fresh page, address translation misses are served in order, and these are needed last)
  auto load_adapter_b = [&]() {
    const rsrc_t rb = make_rsrc(a.lora_b, (uint64_t)a.N * a.lora_rank * 2);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        if (j * 32 < a.lora_rank)
          lbv[nt][j] = buf_load128(rb, (((uint32_t)(ntile0 + nt) * 16u + (uint32_t)lm) * (uint32_t)a.lora_rank +
                                        (uint32_t)(j * 32 + lq * 8)) * 2u);
  };
  if (lora_fast) {
    const int ch = (int)chs;
    const int col = ((ch < 8) ? toff_a : toff_b) + min((ch & 7) * 8, a.lora_rank - 8);
    tbase = (uint32_t)((m0 + (tid >> 4)) * a.t_ld + col) * 2u;
  }
  const u32x4 rt = raw_rsrc(lora_fast ? (const void*)a.t : (const void*)a.x,
                            lora_fast ? (uint64_t)a.M * a.t_ld * 2 : (uint64_t)a.M * a.K * 2);
  auto sel_rsrc = [&](bool ut) -> u32x4 {
    const uint32_t m = 0u - (uint32_t)ut;
    return u32x4{rx[0] ^ ((rx[0] ^ rt[0]) & m), rx[1] ^ ((rx[1] ^ rt[1]) & m), rx[2] ^ ((rx[2] ^ rt[2]) & m), rx[3]};
  };
  const uint32_t tstride = (uint32_t)(32 * a.t_ld * 2);

  // k-tiles past the last one are clamped: their data is fetched but never multiplied
  auto load_a = [&](int kt, uint32_t buf) {
    const bool ut = lora_fast && kt >= kt_end;
    const int s = ut ? 0 : min(kt, ktiles - 1) * (KTILE * 2);
    const u32x4 r = sel_rsrc(ut);
    // bit selects (not ?:, which the compiler turns into a private-memory table)
    const uint32_t m = 0u - (uint32_t)ut;
    const uint32_t base = xbase ^ ((xbase ^ tbase) & m), stride = xstride ^ ((xstride ^ tstride) & m);
#pragma unroll
    for (int c = 0; c < AP; ++c) dma16(buf + dma_wave + (uint32_t)c * 8192u, r, base + (uint32_t)c * stride, s);
  };
  // scales of ring stage D -> fp32; a k-tile past the end gets zero scales, which turns its
  // weights into zeros
  auto expand_scales = [&](auto Dc, bool active) {
    constexpr int D = decltype(Dc)::value;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const uint32_t w = ring_s[D][nt];
      if constexpr (SPT == 2) {  // one group per two k-steps: this wave's half of the pair
        const uint32_t bits = kh ? (w & 0xffff0000u) : (w << 16);
        sc[D][nt][0] = active ? __builtin_bit_cast(float, bits) : 0.f;
      } else {
        sc[D][nt][0] = active ? bflo(w) : 0.f;
        sc[D][nt][1] = active ? bfhi(w) : 0.f;
      }
    }
  };
  // table look-ups of this wave's k-step J (0 | 1) of ring stage D; the raw f16 pairs land in dst
  auto lut_issue = [&](auto Dc, auto Jc, uint32_t (&dst)[NT][4]) {
    constexpr int D = decltype(Dc)::value, J = decltype(Jc)::value;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const uint32_t w = ring_c[D][nt][J];
      // table address bytes: [0] = lane * 4, [1] = code byte b of w, [2] = 1 (the table's base), [3] = 0
#pragma unroll
      for (int j = 0; j < 4; ++j) dst[nt][j] = level_entry(w, j);
    }
  };
  // f16 level pair x fp32 scale -> bf16 pair
  auto convert = [&](auto Dc, auto Jc, u32x4 (&dst)[NT], const uint32_t (&src)[NT][4]) {
    constexpr int D = decltype(Dc)::value, J = decltype(Jc)::value;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const float s = sc[D][nt][SPT == 2 ? 0 : J];
      u32x4 r;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        _Float16 l0, l1;
        level_pair<INT4>(src[nt], b, l0, l1);
        r[b] = cvt_pk_bf16(__builtin_fmaf((float)l0, s, 0.0f), __builtin_fmaf((float)l1, s, 0.0f));
      }
      dst[nt] = r;
    }
  };
  // LDS byte addresses of this lane's fragments: row l % 16 (+ 16 per row tile, an immediate),
  // k-chunk 8 kh + 4 J + l / 16 of the wave's k-step J, swizzled by the row; the other step of
  // the same tile is 64 bytes away under XOR.  a_cur1: step 1 of the current tile, a_nxt0: step 0
  // of the next one (the two the loop reads); they trade places, and steps, after every k-tile.
  // (With fewer than 32 rows a pass still moves 32: the extra rows are zeros or rows of nobody's
  // tile, and land in LDS rows no fragment reads.)
  uint32_t a_cur1 = (uint32_t)lm * 256u + (((uint32_t)(kh * 8 + 4 + lq) ^ (uint32_t)lm) * 16u);
  uint32_t a_nxt0 = (a_cur1 ^ 64u) + ABYTES;
  uint32_t dma_buf = 0;     // the tile buffer the second step of the current k-tile refills
  // One of this wave's two k-steps, written as NT * 8 units in the order they should issue: two
  // units per code pair of the step.  The MT * NT MFMAs are spread evenly over the units
  // (column tile-major: the first MT use the column tile whose conversion finished first).  An
  // even unit forms the two f16 x scale products of its pair of the NEXT step's weights, the odd
  // unit packs them to bf16.  The first half of the units also carries the LDS reads: one table
  // look-up each (pair u of the step AFTER the next, into the other half of lp) and the
  // activation fragments of the next step; the second half the requests to memory: the weights of
  // k-tile kt + PF into this tile's ring stage (ST, first step, ahead of the barrier), or the
  // activations of k-tile kt + 2 into this tile's LDS buffer (LD, second step: behind the
  // barrier, when no wave reads that buffer any more).
  // A scheduling barrier behind every unit keeps that order.
  auto kstep = [&](auto CURc, auto Dcc, auto Jcc, auto Dlc, auto Jlc, uint32_t rd_base, auto Jrc, auto STc,
                   auto LDc, auto EXc, int kt, bool ex_active) {
    constexpr int CUR = decltype(CURc)::value, NXT = CUR ^ 1;
    constexpr int DC = decltype(Dcc)::value, JC = decltype(Jcc)::value;
    constexpr int DL = decltype(Dlc)::value, JL = decltype(Jlc)::value;
    (void)sizeof(Jrc);   // (the k-step of the fragments to read is part of rd_base)
    constexpr bool ST = decltype(STc)::value != 0, LD = decltype(LDc)::value != 0;
    constexpr int EX = decltype(EXc)::value;   // -1, or the ring stage whose scales to expand
    constexpr int UNITS = NT * 8, MPS = MT * NT;
    static_assert(UNITS % MPS == 0 && 4 + 2 * NT <= UNITS / 2 && AP <= 4, "unit layout");
    float f0 = 0.f, f1 = 0.f;
    const bool ut = lora_fast && kt >= kt_end;      // LD: the activation tile to fetch is the adapter block
    // (INT4: left alone, the compiler keeps this wave-uniform offset in a vector register in that
    // instantiation and hands it to the load's scalar operand as it is)
    const int xs_ = ut ? 0 : min(kt, ktiles - 1) * (KTILE * 2);
    const int xs = INT4 ? __builtin_amdgcn_readfirstlane(xs_) : xs_;
    const u32x4 xr = sel_rsrc(ut);
    const uint32_t um = 0u - (uint32_t)ut;
    const uint32_t xo = xbase ^ ((xbase ^ tbase) & um), xst = xstride ^ ((xstride ^ tstride) & um);
    const int wkt = min(kt + (PF - 2), ktiles - 1);   // LD: weights of k-tile (this + PF)
#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
      const int p = u >> 1, pnt = p >> 2, pb = p & 3;
      if ((u * MPS) % UNITS == 0) {
        const int mi = u * MPS / UNITS, nt = mi / MT, m = mi % MT;
        acc[m][nt] = mfma16(af[CUR][m], bfr[CUR][nt], acc[m][nt]);
      }
      if ((u & 1) == 0) {
        _Float16 l0, l1;
        level_pair<INT4>(lp[CUR][pnt], pb, l0, l1);
        const float sv = sc[DC][pnt][SPT == 2 ? 0 : JC];
        f0 = __builtin_fmaf((float)l0, sv, 0.0f);
        f1 = __builtin_fmaf((float)l1, sv, 0.0f);
      } else {
        bfr[NXT][pnt][pb] = cvt_pk_bf16(f0, f1);
      }
      if (u < UNITS / 2) {   // all LDS reads in the first half: nothing of them is in flight at the barrier
        lp[NXT][u >> 2][u & 3] = level_entry(ring_c[DL][u >> 2][JL], u & 3);
        if (u < MT) af[NXT][u] = lds_ld128(rd_base + (uint32_t)(u * 16 * 256));
      } else {
        const int q = u - UNITS / 2;
        if (LD && q >= 1 && q <= AP)   // (after the barrier: every wave has read this tile's fragments)
          dma16(dma_buf + dma_wave + (uint32_t)(q - 1) * 8192u, xr, xo + (uint32_t)(q - 1) * xst, xs);
        if (ST) {
          constexpr int DW = DC;   // the ring stage of this k-tile: all its codes have been looked up
          if (q >= 4 && q < 4 + NT) {
            ring_c[DW][q - 4] = __builtin_amdgcn_raw_buffer_load_b64(rc, coff[q - 4], wkt * 1024, 0);
          } else if (q >= 4 + NT && q < 4 + 2 * NT) {
            ring_s[DW][q - 4 - NT] = __builtin_amdgcn_raw_buffer_load_b32(rs, soff[q - 4 - NT], wkt * (16 * SPT * 2), 0);
          }
        }
      }
      if (EX >= 0 && u < NT * SW) {
        constexpr int E = EX < 0 ? 0 : EX;
        const int ent = u / SW, ej = u % SW;
        const uint32_t w = ring_s[E][ent];
        if constexpr (SPT == 2) {
          const uint32_t bits = kh ? (w & 0xffff0000u) : (w << 16);
          sc[E][ent][0] = ex_active ? __builtin_bit_cast(float, bits) : 0.f;
        } else {
          sc[E][ent][ej] = ex_active ? (ej ? bfhi(w) : bflo(w)) : 0.f;
        }
      }
      __builtin_amdgcn_sched_barrier(0);   // units issue in the order written
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // One k-tile of ring stage D = this wave's two k-steps.  On entry af[0] holds the activation
  // fragments of the first step, bfr[0] its weights and lp the table entries of the second.
  // The one barrier of the k-tile sits between the steps: every wave has finished reading this
  // tile, and the next tile, requested by the second step of the tile before, has landed in LDS
  // (the only younger loads are the 2 NT weight / scale loads the first step has just issued).
  auto tile = [&](auto Dc, int kt) {
    constexpr int d = decltype(Dc)::value, dn = (d + 1) % PF;
    const bool next_active = kt + 1 < kt_end;
    __builtin_amdgcn_sched_barrier(0);
    kstep(ic<0>{}, Dc, ic<1>{}, ic<dn>{}, ic<0>{}, a_cur1, ic<1>{}, ic<1>{}, ic<0>{}, ic<dn>{}, kt + 2, next_active);
    tnx_wait_vm(2 * NT);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    kstep(ic<1>{}, ic<dn>{}, ic<0>{}, ic<dn>{}, ic<1>{}, a_nxt0, ic<0>{}, ic<0>{}, ic<1>{}, ic<-1>{}, kt + 2, false);
    const uint32_t r = a_cur1;
    a_cur1 = a_nxt0 ^ 64u;
    a_nxt0 = r ^ 64u;
    dma_buf ^= ABYTES;
  };

  if (kt_begin < kt_end) {
    // Order of the first loads: each is followed by at least as many later loads as it will be
    // in the steady state of the loop, so the counted waits of the loop body need not fall back
    // to "everything outstanding" for the sake of the path that enters from here.
    TNX_STAMP(7);
    if constexpr (!INT4) {
       // table entry e = f16 pair (level[e & 15], level[e >> 4]); copies rotated over banks,
       // half of them per thread; built while the first loads are in flight
      uint32_t* lut = reinterpret_cast<uint32_t*>(smem + kBigLutBase);
      const h16x2 h = {(_Float16)lvl0, (_Float16)lvl1};
      const uint32_t v = __builtin_bit_cast(uint32_t, h);
      const int e = tid & 255, c0 = (tid >> 8) * 32;
#pragma unroll
      for (int c = 0; c < 32; ++c) lut[e * 64 + ((c0 + c + lane) & 63)] = v;
    }
    // The rest of the first loads go out behind the table: what the first k-tile needs (its
    // activations and weights, requested above by every wave) is then at the head of the unit's
    // memory queue, and the first tile is multiplied while the second one's data arrives.
    __builtin_amdgcn_sched_barrier(0);
    load_w(ic<1>{}, kt_begin + 1);
    load_a(kt_begin + 1, ABYTES);
    load_w(ic<2>{}, kt_begin + 2);
    if (lora_fast) load_adapter_b();
    __builtin_amdgcn_sched_barrier(0);
    TNX_STAMP(1);
    expand_scales(ic<0>{}, true);
    // the first tile's AP loads are the oldest in flight; at least 3 x 2 NT weight / scale loads
    // and the second tile's AP follow them
    tnx_wait_vm(6 * NT + AP);
    __syncthreads();  // table and first activation tile
    lut_issue(ic<0>{}, ic<0>{}, lp[1]);
#pragma unroll
    for (int m = 0; m < MT; ++m) af[0][m] = lds_ld128((a_cur1 ^ 64u) + (uint32_t)(m * 16 * 256));
    convert(ic<0>{}, ic<0>{}, bfr[0], lp[1]);
    lut_issue(ic<0>{}, ic<1>{}, lp[0]);
    if (lora_fast) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int j = 0; j < 2; ++j) lds_st128(lb_lds + (uint32_t)((nt * 2 + j) * 1024), lbv[nt][j]);
    }
    TNX_STAMP(2);
    // whole turns of the ring (three k-tiles) without a branch inside -- a conditional tile
    // would make the waits of the tile after it assume that its loads never happened -- then
    // the one or two tiles left
    int kt = kt_begin;
    for (; kt + PF <= kt_end; kt += PF) {
      tile(ic<0>{}, kt);
      tile(ic<1>{}, kt + 1);
      tile(ic<2>{}, kt + 2);
    }
    if (kt < kt_end) {
      tile(ic<0>{}, kt);
      if (kt + 1 < kt_end) tile(ic<1>{}, kt + 1);
    }
  }
  TNX_STAMP(3);

  const bool has_rows = MT > 1 || kh == 0;
  const int64_t m0w = m0 + kh * (HM * 16);   // first row of the tile this wave finishes
  const uint32_t row_lds = (uint32_t)(kh * (HM * 16) * 256);
  // every load into LDS has landed (the last k-tile requested one more tile): the epilogue
  // reuses the buffers
  tnx_wait_vm(0);
  const uint32_t n_tiles = (uint32_t)max(kt_end - kt_begin, 0);
  const uint32_t t_buf = (n_tiles & 1u) * ABYTES;   // the adapter block is "k-tile" n_tiles of this split

  // The adapter's share of the rows this wave will finish, before the k halves meet: it needs
  // nothing from the partner (the t block sits in LDS as the k-tile after the last, the B^T
  // fragments since the prologue), so it runs while slower waves are still in their last k-tile.
  f32x4 part[HM][NT];
#pragma unroll
  for (int mt = 0; mt < HM; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) zero_acc(part[mt][nt]);
  if (lora_fast && has_rows) {
    const uint32_t tb = t_buf + row_lds + (uint32_t)lm * 256u;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const uint32_t half = toff[nt] == toff_a ? 0u : 8u;   // first 16-byte chunk of the segment's 64 columns
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (j * 32 < a.lora_rank) {
          const u32x4 lbf = lds_ld128(lb_lds + (uint32_t)((nt * 2 + j) * 1024));
#pragma unroll
          for (int mt = 0; mt < HM; ++mt)
            part[mt][nt] = mfma16(lds_ld128(tb + (uint32_t)(mt * 16 * 256) +
                                            (((half + (uint32_t)(j * 4 + lq)) ^ (uint32_t)lm) * 16u)), lbf, part[mt][nt]);
        }
      }
    }
  }

  // The two k halves meet: each wave keeps the row half kh of its column group (row tiles
  // [kh * HM, ...); with a single row tile the first wave keeps it and the second keeps none),
  // hands the other tiles to its partner through the (now idle) table area and adds what the
  // partner hands over.
  f32x4 out[HM][NT];
  {
    __syncthreads();  // every wave is done with the table
    const uint32_t xw = kBigLutBase + (uint32_t)wv * 8192u + (uint32_t)lane * 16u;
    const uint32_t xr = kBigLutBase + (uint32_t)(wv ^ 4) * 8192u + (uint32_t)lane * 16u;
#pragma unroll
    for (int m = 0; m < HM; ++m)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const f32x4 v = kh ? acc[m][nt] : acc[HM + m < MT ? HM + m : 0][nt];
        lds_st128(xw + (uint32_t)((m * NT + nt) * 1024), __builtin_bit_cast(u32x4, v));
      }
    __syncthreads();
#pragma unroll
    for (int m = 0; m < HM; ++m)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const f32x4 own = kh ? acc[HM + m < MT ? HM + m : 0][nt] : acc[m][nt];
        const f32x4 got = __builtin_bit_cast(f32x4, lds_ld128(xr + (uint32_t)((m * NT + nt) * 1024)));
        out[m][nt] = own + got;
      }
  }
  if (lora_fast && has_rows) {
#pragma unroll
    for (int mt = 0; mt < HM; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) out[mt][nt][i] += a.lora_scale * part[mt][nt][i];
  } else if (a.lora_rank > 0 && blockIdx.z == 0 && !lora_fast && has_rows) {
    TileSrc s;
    s.M = a.M; s.K = a.K; s.x = a.x; s.row_index = nullptr; s.row_div = 1; s.x_rows = a.M;
    s.w_bf16 = nullptr; s.codes = a.codes; s.scales = a.scales; s.group = a.group; s.qtype = a.qtype;
    s.ntiles = ntiles; s.lora_rank = a.lora_rank; s.t = a.t; s.t_ld = a.t_ld; s.lora_b = a.lora_b;
    s.lora_scale = a.lora_scale;
    tile_lora<HM, NT>(s, m0w, ntile0, toff, out);
  }
  TNX_STAMP(4);
  const bool mul = a.epilogue == TNX_EPI_SILU_MUL || a.epilogue == TNX_EPI_GELU_MUL;
  if (NT == 2 && mul && a.split_k <= 1) {
    // act = f(gate) * up goes through LDS (the activation buffer the adapter block is not in):
    // rows leave the work-group as 128-byte runs instead of 2-byte scatters, and, when asked,
    // the tile is multiplied with the NEXT linear's adapter A (its LoRA down-projection, whose
    // K axis is this kernel's output axis), one fp32 fragment plane per work-group.
    constexpr int ACT_LD = 72;  // 64 act columns + 8 pad (bf16 elements)
    const uint32_t act_lds = t_buf ^ ABYTES;
    const int64_t ldy = a.N / 2;
    const int64_t wgcol0 = (int64_t)blockIdx.y * 64;      // first act column of the work-group
    const bool fuse_next = a.next_tpart != nullptr;
    u32x4 bn[4][2];
    if (fuse_next) {
      const rsrc_t rn = make_rsrc(a.next_a_t, (uint64_t)a.next_rank * ldy * 2);
#pragma unroll
      for (int n = 0; n < 4; ++n)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int64_t k = wgcol0 + j * 32 + lq * 8;
          const bool ok = n * 16 < a.next_rank && k + 8 <= ldy;
          bn[n][j] = buf_load128(rn, ok ? (uint32_t)(((int64_t)(n * 16 + lm) * ldy + k) * 2) : 0xfffffff0u);
        }
    }
    uint16_t* act_s = reinterpret_cast<uint16_t*>(smem + act_lds);
    if (has_rows) {
#pragma unroll
      for (int mt = 0; mt < HM; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float g = rbf(out[mt][0][i]);
          const float u = rbf(out[mt][1][i]);
          const float act = a.epilogue == TNX_EPI_SILU_MUL ? silu_bf16(g) : gelu_tanh_bf16(g);
          act_s[(kh * (HM * 16) + mt * 16 + lq * 4 + i) * ACT_LD + wn * 16 + lm] = f2bf(rbf(act) * u);
        }
    }
    __syncthreads();
    uint16_t* y = reinterpret_cast<uint16_t*>(a.y);
#pragma unroll
    for (int c = 0; c < (ROWS * 8 + 511) / 512; ++c) {
      const int idx = tid + 512 * c, row = idx >> 3, ch = idx & 7;
      if (row >= ROWS) break;
      const u32x4 v = lds_ld128(act_lds + (uint32_t)((row * ACT_LD + ch * 8) * 2));
      if (m0 + row < a.M && wgcol0 + ch * 8 + 8 <= ldy)
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(y + (m0 + row) * ldy + wgcol0 + ch * 8));
    }
    if (fuse_next && wv < MT) {   // one row tile per wave; fewer rows leave plane slots unwritten
      float* plane = a.next_tpart + ((int64_t)blockIdx.x * gridDim.y + blockIdx.y) * 8192;
      {
        const int mt = wv;
        u32x4 af2[2];
#pragma unroll
        for (int j = 0; j < 2; ++j)
          af2[j] = lds_ld128(act_lds + (uint32_t)(((mt * 16 + lm) * ACT_LD + j * 32 + lq * 8) * 2));
#pragma unroll
        for (int n = 0; n < 4; ++n) {
          f32x4 pacc = f32x4{0.f, 0.f, 0.f, 0.f};
          pacc = mfma16(af2[0], bn[n][0], pacc);
          pacc = mfma16(af2[1], bn[n][1], pacc);
          __builtin_nontemporal_store(pacc, reinterpret_cast<f32x4*>(plane + ((mt * 4 + n) * 64 + lane) * 4));
        }
      }
    }
  } else if (NT == 2 && MT >= 4 && a.split_k > 1 && has_rows && ntile0 + NT <= ntiles &&
             (uint64_t)a.M * (uint64_t)a.N * 4 < (1ull << 32)) {
    // fp32 partial plane of this k split.  A lane's accumulators are four rows of one column;
    // stored as they are, a wave would issue 32 four-byte stores of 64-byte runs.  Each 16 x 32
    // row tile goes through a wave-private corner of the activation buffers instead (idle since
    // the barriers of the exchange above) and leaves as two 16-byte stores per lane, 128-byte
    // runs (rows past M fall outside the plane's buffer and are dropped).  The planes are written
    // once and read once, by another kernel on other XCDs: stored with the non-temporal policy
    // (decode step 6.51 -> 6.42 ms; the same policy on the outputs of the norm and of attention,
    // which many work-groups re-read, measured neutral and is not used there).
    constexpr int T_LD = 36;   // floats per LDS row: 32 + 4, conflict-free for both passes
    const uint32_t scr = (uint32_t)wv * (16u * T_LD * 4u);
    static_assert(MT < 4 || 8 * 16 * T_LD * 4 <= 2 * (int)ABYTES, "transposition scratch fits the activation buffers");
    const rsrc_t rp = make_rsrc(a.ws + (int64_t)blockIdx.z * a.M * a.N, (uint64_t)a.M * a.N * 4);
    const uint32_t col0 = (uint32_t)ntile0 * 16u;
#pragma unroll
    for (int mt = 0; mt < HM; ++mt) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float v = out[mt][nt][i];   // (a bit cast applied to the vector element itself reads element 0)
          *reinterpret_cast<lds_u32*>(static_cast<uintptr_t>(scr + (uint32_t)(((lq * 4 + i) * T_LD + nt * 16 + lm) * 4))) =
              __float_as_uint(v);
        }
      // (the reads below are of another type than the writes above: keep the compiler from
      // moving them across; LDS itself executes a wave's accesses in order)
      asm volatile("" ::: "memory");
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int r = (lane >> 3) + 8 * j, c4 = (lane & 7) * 4;
        const u32x4 v = lds_ld128(scr + (uint32_t)((r * T_LD + c4) * 4));
        const uint32_t off = ((uint32_t)(m0w + mt * 16 + r) * (uint32_t)a.N + col0 + (uint32_t)c4) * 4u;
        __builtin_amdgcn_raw_buffer_store_b128(v, rp, off, 0, kStreamOnce);
      }
      asm volatile("" ::: "memory");
    }
  } else {
    if (has_rows) store_tile<HM, NT>(a, m0w, a.M, ntile0, ntiles, out, [](int64_t r) { return r; });
  }
  TNX_STAMP(5);
}

}  // namespace
