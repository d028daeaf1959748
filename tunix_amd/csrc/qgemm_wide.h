// The quantised GEMM for many rows (prefill, per-token logps): output tile 128 rows x 256
// columns per work-group of four waves, one per SIMD (the 128 accumulator registers of a wave's
// 128 x 64 block next to the operand pipeline).  Same weight
// format, table look-up and conversion as qgemm128_kernel; what differs follows from what a
// wave that has its SIMD to itself can issue:
//
//   * 32x32x16 MFMAs.  One wave issues independent 16x16x32 MFMAs at half the rate of the
//     matrix pipe and serialises every vector instruction behind them; a 32x32x16 MFMA keeps
//     the pipe busy for 32 clocks and leaves room for the four conversion instructions, the
//     look-up and the fragment read that go with it.  The packed weight tiles (16 columns x
//     128 k, built for the 16x16x32 operand layout) are read with another lane -> chunk map for
//     that: lane l takes column l % 32 of a 32-column group and, per k-tile, the two 16-byte
//     chunks that hold its k-groups 8 (l / 32) + 16 u of that column.
//   * every wave walks all eight 16-deep slabs of a k-tile (no k split inside the work-group,
//     no exchange of accumulators); products are formed transposed (weights as the MFMA's A
//     operand), so that a lane owns runs of four consecutive output columns of one row and the
//     tile leaves through LDS as whole 16-byte row chunks.
//   * a slab is written as eight slots in issue order, one MFMA each with its share of the
//     work for the following slabs; a scheduling barrier behind every slot keeps that order.
//
// Work-groups are numbered in groups of 64 row blocks per column tile (consecutive work-group
// ids go to consecutive XCDs): the eight row blocks an XCD works on at a time want the same
// column tile's weights, which its L2 then holds for all of them.
//
// From the expanded copy of the weights (kWidePre) a wave needs half the register file, and
// two work-groups share a compute unit, two waves a SIMD.
//
// Included by qlinear.hip after qgemm128.h.
#pragma once

namespace {

constexpr int kWideRows = 128, kWideCols = 256;
// LDS: two activation tiles of 128 rows x 128 k (256-byte rows, 16-byte chunks XOR-swizzled by
// row) at 0 and 32 KB, the table behind them.
constexpr uint32_t kWideTileBytes = kWideRows * KTILE * 2, kWideLutBase = 2 * kWideTileBytes;
constexpr size_t kWideSmemBytes = kWideLutBase + kBigLutBytes;
static_assert(kWideLutBase == 0x10000, "the table look-up forms its address with byte 2 = 1");

typedef float f32x16 __attribute__((ext_vector_type(16)));
__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
  // D[32x32] += A[32x16] * B[16x32]; lane l holds A row l%32 / B column l%32, k = 8*(l/32)..+7;
  // D: column l%32, rows 8*(r/4) + 4*(l/32) + r%4 for register r.
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// GROUPED: the grouped GEMM over routed tokens at many rows per expert.  A work-group takes one
// 128-row block of one expert's routes (in expert-sorted order) and one column tile; block b ->
// (expert, row block) is found from the expert offsets by a running sum; activation rows are
// gathered through sorted_route (row = route / x_div), output rows are routes.  No adapter, no
// lm_head statistics in this mode.
// MODE: where the bf16 weight fragments come from.  kWideTable: codes through the LDS table;
// kWideInt4: integer codes converted without the table (Int4Magic in common.h); kWidePre: a copy
// of the weights that was converted once, bf16(bf16(level) * scale), and laid out as the
// fragments themselves (tnx_qw_expand: [column tile][k-tile][wave][column group][slab][lane] x
// 16 bytes), so that a lane's fragment of a slab is one 16-byte load and the loop has neither
// conversion instructions nor look-ups.  The frozen base weights of a model fit HBM a second time
// in that form; rows in the hundreds of thousands per weight byte make its four times larger
// stream irrelevant.  Same MFMA sequence on the same operand bits: results are bit-identical.
constexpr int kWideTable = 0, kWideInt4 = 1, kWidePre = 2;
// kWidePre keeps so little besides its accumulators in registers that two of its waves fit one
// SIMD (128 accumulator registers + 128 others each) and two of its work-groups one compute unit
// (68 KB of LDS each: the two activation tiles, later the output stage): each covers the other's
// barriers, first loads and epilogue.
constexpr int kWidePreStages = 6;   // slabs of weight fragments in flight per wave
constexpr size_t kWidePreSmemBytes = 68 * 1024;
static_assert(kWidePreSmemBytes >= 2 * kWideTileBytes && kWidePreSmemBytes >= kWideRows * (kWideCols + 8) * 2,
              "the activation tiles and the output stage fit");
static_assert(24 % kWidePreStages == 0, "a stage keeps its slot over the three unrolled k-tiles");
template <int SPT, bool GROUPED = false, int MODE = kWideTable>
__global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(MODE == kWidePre ? 2 : 1, MODE == kWidePre ? 2 : 1)))
void qgemm_wide_kernel(const QLArgs a, const WideHead h) {
  constexpr bool INT4 = MODE == kWideInt4, PRE = MODE == kWidePre;
  static_assert(!(PRE && GROUPED), "the grouped form reads packed codes");
  constexpr int RT = 4, CG = 2, PF = 3, AP = 8;   // 32-row tiles, 32-column groups per wave
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wn = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lh = lane >> 5;
  // LDS is addressed absolutely (table at 0): no static LDS in this kernel, checked by the host
  asm volatile("" ::"s"(a.M), "s"(a.K), "s"(a.N), "s"(a.qtype), "s"(a.x), "s"(a.codes), "s"(a.scales),
               "s"(a.lora_rank), "s"(a.lora_nseg), "s"(a.lora_seg_end[0]), "s"(a.lora_seg_end[1]),
               "s"(a.lora_seg_end[2]), "s"(a.lora_seg_toff[0]), "s"(a.lora_seg_toff[1]),
               "s"(a.lora_seg_toff[2]), "s"(a.lora_seg_toff[3]));
  asm volatile("" ::"s"(a.t_ld), "s"(a.t), "s"(a.lora_b), "s"(a.lora_scale), "s"(a.epilogue), "s"(a.y),
               "s"(a.residual));
  const float lvl0 = rbf(code_level_imm(a.qtype, tid & 15)), lvl1 = rbf(code_level_imm(a.qtype, (tid >> 4) & 15));
  const uint32_t lane_off = (uint32_t)lane * 4u | kWideLutBase;   // byte 2 = 1: the table's base

  // work-group id -> (row block, column tile): groups of 64 row blocks, the column tile moves
  // every 64 ids (ids go round-robin to the eight XCDs: the eight row blocks an XCD holds at a
  // time share the column tile's weights in its L2)
  const int tiles_m = (int)((a.M + kWideRows - 1) / kWideRows), tiles_n = (int)((a.N + kWideCols - 1) / kWideCols);
  int mtile, ntile;
  int expert = 0, m_end = 0;   // GROUPED: the block's expert and the end of its routes in sorted order
  if constexpr (GROUPED) {
    // column tiles of one row block sit next to each other; every wave finds the block's expert
    // itself (same result in all of them: nothing is shared, no barrier)
    const int b = (int)blockIdx.x / tiles_n;
    ntile = (int)blockIdx.x % tiles_n;
    int carry = 0, found_e = -1, found_rb = 0;
    for (int base = 0; base < a.n_experts; base += 64) {
      const int e = base + lane;
      int nb = 0;
      if (e < a.n_experts) nb = (a.offsets[e + 1] - a.offsets[e] + kWideRows - 1) / kWideRows;
      int incl = nb;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int t = __shfl_up(incl, o, 64);
        if (lane >= o) incl += t;
      }
      const int first = carry + incl - nb;
      const uint64_t hit = __ballot(nb > 0 && b >= first && b < first + nb);
      if (hit) {
        const int l = __ffsll((long long)hit) - 1;
        found_e = base + l;
        found_rb = b - __shfl(first, l, 64);
      }
      carry += __shfl(incl, 63, 64);
    }
    if (found_e < 0) return;   // past the last block (the grid covers an upper bound)
    expert = __builtin_amdgcn_readfirstlane(found_e);
    mtile = __builtin_amdgcn_readfirstlane(found_rb);
    m_end = a.offsets[expert + 1];
  } else {
    constexpr int GR = 64;
    const int per_group = GR * tiles_n;
    const int g = (int)blockIdx.x / per_group, r = (int)blockIdx.x % per_group;
    const int gm = min(GR, tiles_m - g * GR);
    mtile = g * GR + r % gm;
    ntile = r / gm;
  }
  // first row of the tile (GROUPED: first position in the sorted route list)
  const int64_t m0 = GROUPED ? (int64_t)a.offsets[expert] + (int64_t)mtile * kWideRows : (int64_t)mtile * kWideRows;
  const int64_t ntile0 = ((int64_t)ntile * 4 + wn) * 4;   // first packed 16-column tile of this wave
  const int64_t ntiles = a.N / 16;
  const int ktiles = (int)(a.K / KTILE);
  const int rows_here = (int)min((int64_t)kWideRows, (GROUPED ? (int64_t)m_end : a.M) - m0);

  // the activation resource starts at this work-group's first row: offsets stay small whatever
  // M is, and rows past M lie beyond the resource and read zeros (GROUPED: the whole buffer,
  // rows are gathered)
  const u32x4 rx = GROUPED ? raw_rsrc(a.x, (uint64_t)(a.M / a.x_div) * a.K * 2)
                           : raw_rsrc(a.x + m0 * a.K, (uint64_t)rows_here * a.K * 2);
  const uint64_t ntk = (uint64_t)ntiles * ktiles;
  const rsrc_t rc = make_rsrc(a.codes + (GROUPED ? (int64_t)expert * a.codes_stride : 0), ntk * 1024);
  const rsrc_t rs = make_rsrc(a.scales + (GROUPED ? (int64_t)expert * a.scales_stride : 0), ntk * 16 * SPT * 2 + 16);
  // Lane l: column l % 32 of a group = column (l % 16) of packed tile 2 cg + (l % 32) / 16.  A
  // packed tile holds, at chunk 16 q + c, the k-groups 8 q + 32 j (dword j) of its column c;
  // slab u of the MFMA wants k-group 2 u + l / 32 from this lane: chunk q = l / 32 gives the
  // even slabs (dword u / 2), chunk q = 2 + l / 32 the odd ones.  Column tiles past N start
  // beyond the buffer and read zeros.
  uint32_t coff[CG], soff[CG];
  // Activation tiles go from memory straight into LDS, 16 bytes per lane, a wave's 64 lanes
  // into 1 KB = four consecutive 256-byte rows.  Thread t fills chunk t % 16 of rows t / 16 + 16 c
  // (c = 0..7) and fetches for it the k-chunk (t % 16) ^ (row % 16): with the chunks of a row
  // permuted like that, the 16 lanes that read one k-chunk of 16 consecutive rows for an MFMA
  // fragment hit 16 different bank groups.
  const uint32_t chs = (uint32_t)((tid & 15) ^ ((tid >> 4) & 15));
  const uint32_t xbase = ((uint32_t)(tid >> 4) * (uint32_t)a.K + chs * 8u) * 2u;
  const uint32_t xstride = 16u * (uint32_t)a.K * 2u;  // 16 rows further per pass
  // GROUPED: the byte offset of each of this thread's eight rows (rows the block does not have:
  // beyond the buffer, which reads zeros)
  uint32_t xrow[GROUPED ? 8 : 1];
  if constexpr (GROUPED) {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int r = (tid >> 4) + 16 * c;
      const int route = r < rows_here ? a.sorted_route[m0 + r] : -1;
      xrow[c] = route >= 0 ? ((uint32_t)(route / a.x_div) * (uint32_t)a.K + chs * 8u) * 2u : 0xfffff000u;
    }
  }
  auto xoff = [&](int c, uint32_t base, uint32_t stride) -> uint32_t {
    if constexpr (GROUPED) return xrow[c];
    return base + (uint32_t)c * stride;
  };
#pragma unroll
  for (int cg = 0; cg < CG; ++cg) {
    const uint32_t tile0 = (uint32_t)(ntile0 + 2 * cg + (l32 >> 4)) * (uint32_t)ktiles;
    coff[cg] = tile0 * 1024u + (uint32_t)(16 * lh + (l32 & 15)) * 16u;
    soff[cg] = (tile0 * 16u + (uint32_t)(l32 & 15)) * (uint32_t)(SPT * 2);
  }

  f32x16 acc[RT][CG];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[rt][cg][i] = 0.f;

  u32x4 ring_c[PF][CG][2];   // [.][.][0]: even slabs, [1]: odd slabs
  u32x2 ring_s[PF][CG];
  float sc[PF][CG][SPT];
  // INT4: the entries keep their offsets (1024 + n | 64 + n), and the products subtract them
  // again as -1032 s | -72 s in the multiply-add
  float sb[INT4 ? PF : 1][CG][SPT][2];
  auto set_scale = [&](int d, int cg, int j, float v) {
    sc[d][cg][j] = v;
    if constexpr (INT4) {
      sb[d][cg][j][0] = v * -1032.0f;
      sb[d][cg][j][1] = v * -72.0f;
    }
  };
  u32x4 xf[2][RT];           // activation fragments of the current / next slab
  u32x4 wf[2][CG];           // weight fragments of the current / next slab
  // PRE: the fragments of the next kWidePreStages slabs, loaded as they are; stage = slab % stages
  u32x4 wr[PRE ? kWidePreStages : 1][CG];
  const rsrc_t re = make_rsrc(PRE ? (const void*)a.w_pre : (const void*)a.x,
                              PRE ? (uint64_t)tiles_n * (uint64_t)ktiles * 65536u : 0u);
  uint32_t evoff[CG];
#pragma unroll
  for (int cg = 0; cg < CG; ++cg) evoff[cg] = (uint32_t)(((wn * CG + cg) * 8 * 64 + lane) * 16);
  // slab `sl` (counted from this work-group's first k-tile) of column group cg -> its stage
  auto load_pre = [&](int sl, int u, int cg) {
    const int kt_ = min(sl >> 3, ktiles - 1);
    wr[PRE ? sl % kWidePreStages : 0][cg] =
        __builtin_amdgcn_raw_buffer_load_b128(re, evoff[cg] + (uint32_t)u * 1024u, (ntile * ktiles + kt_) * 65536, 0);
  };
  // f16 level pairs of the slab after the next (table path: entry b = the pair of byte b, looked
  // up into the place of the entry just consumed; INT4: entries as described above, the slab's
  // parity picks the set, since a set is read until its slab has been converted)
  uint32_t lp[INT4 ? 2 : 1][CG][4];
  float cf0 = 0.f, cf1 = 0.f;  // products of the pair whose pack is still to come

  // LoRA: the k-tile after the last one is the 128-row block of t = bf16(x . A), columns
  // [toff_a, +64) | [toff_b, +64) (the host sends only shapes whose work-groups span at most
  // two adapter segments here); the B^T fragments of this lane's columns stay in registers.
  const bool lora = a.lora_rank > 0;
  int toff[4];
  int toff_a = 0, toff_b = 0;
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) toff[nt] = 0;
  if (lora) {
    if (a.lora_nseg < 0) {
      toff_b = a.lora_rank;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) toff[nt] = (int)((ntile0 + nt) & 1) * a.lora_rank;
    } else {
      int e0 = (int)a.lora_seg_end[0], e1 = (int)a.lora_seg_end[1], e2 = (int)a.lora_seg_end[2];
      int t0 = a.lora_seg_toff[0], t1 = a.lora_seg_toff[1], t2 = a.lora_seg_toff[2], t3 = a.lora_seg_toff[3];
      asm volatile("" : "+s"(e0), "+s"(e1), "+s"(e2), "+s"(t0), "+s"(t1), "+s"(t2), "+s"(t3));
      auto seg_idx = [&](int nt16) {
        const int col = nt16 * 16;
        return (int)(a.lora_nseg > 1 && col >= e0) + (int)(a.lora_nseg > 2 && col >= e1) +
               (int)(a.lora_nseg > 3 && col >= e2);
      };
      auto idx_toff = [&](int i) {
        auto pick = [](int cur, int cand, bool c) { return cur ^ ((cur ^ cand) & (0 - (int)c)); };
        return pick(pick(pick(t0, t1, i == 1), t2, i == 2), t3, i == 3);
      };
      const int last = (int)ntiles - 1;
      const int wg_nt0 = ntile * 16;
      toff_a = idx_toff(seg_idx(min(wg_nt0, last)));
      toff_b = idx_toff(seg_idx(min(wg_nt0 + 15, last)));
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) toff[nt] = idx_toff(seg_idx(min((int)ntile0 + nt, last)));
    }
  }
  u32x4 lbv[CG][4];          // B^T of the adapter: this lane's column, ranks 16 u + 8 (l / 32) ..+7
#pragma unroll
  for (int cg = 0; cg < CG; ++cg)
#pragma unroll
    for (int u = 0; u < 4; ++u) lbv[cg][u] = u32x4{0, 0, 0, 0};
  uint32_t tbase = 0;
  if (lora) {
    const int ch = (int)chs;
    const int col = ((ch < 8) ? toff_a : toff_b) + min((ch & 7) * 8, a.lora_rank - 8);
    tbase = (uint32_t)((tid >> 4) * a.t_ld + col) * 2u;
  }
  const u32x4 rt_ = lora ? raw_rsrc(a.t + m0 * a.t_ld, (uint64_t)rows_here * a.t_ld * 2) : rx;
  const uint32_t tstride = (uint32_t)(16 * a.t_ld * 2);

  // (dma16 of gemm_tile.h: the compiler does not count these loads, the waits for them are
  // written by hand)
  const uint32_t dma_wave = (uint32_t)wn * 1024u;      // this wave's four rows within a 16-row pass
  auto sel_rsrc = [&](bool ut) -> u32x4 {
    const uint32_t m = 0u - (uint32_t)ut;
    return u32x4{rx[0] ^ ((rx[0] ^ rt_[0]) & m), rx[1] ^ ((rx[1] ^ rt_[1]) & m), rx[2] ^ ((rx[2] ^ rt_[2]) & m), rx[3]};
  };
  auto load_a = [&](int kt, uint32_t buf) {
    const bool ut = lora && kt >= ktiles;
    const int s = ut ? 0 : min(kt, ktiles - 1) * (KTILE * 2);
    const u32x4 r = sel_rsrc(ut);
    const uint32_t m = 0u - (uint32_t)ut;
    const uint32_t base = xbase ^ ((xbase ^ tbase) & m), stride = xstride ^ ((xstride ^ tstride) & m);
#pragma unroll
    for (int c = 0; c < AP; ++c) dma16(buf + dma_wave + (uint32_t)c * 4096u, r, xoff(c, base, stride), s);
  };
  auto load_scale = [&](auto Dc, int cg, int ktc) {
    constexpr int D = decltype(Dc)::value;
    if constexpr (SPT == 2) {
      ring_s[D][cg][0] = __builtin_amdgcn_raw_buffer_load_b32(rs, soff[cg], ktc * (16 * SPT * 2), 0);
    } else {
      ring_s[D][cg] = __builtin_amdgcn_raw_buffer_load_b64(rs, soff[cg], ktc * (16 * SPT * 2), 0);
    }
  };
  auto load_w = [&](auto Dc, int kt) {
    constexpr int D = decltype(Dc)::value;
    const int ktc = min(kt, ktiles - 1);
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
      ring_c[D][cg][0] = __builtin_amdgcn_raw_buffer_load_b128(rc, coff[cg], ktc * 1024, 0);
      ring_c[D][cg][1] = __builtin_amdgcn_raw_buffer_load_b128(rc, coff[cg] + 512u, ktc * 1024, 0);
      load_scale(Dc, cg, ktc);
    }
  };
  auto expand_scales = [&](auto Dc, bool active) {
    constexpr int D = decltype(Dc)::value;
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
#pragma unroll
      for (int j = 0; j < SPT; ++j) {
        const uint32_t w = ring_s[D][cg][j >> 1];
        set_scale(D, cg, j, active ? ((j & 1) ? bfhi(w) : bflo(w)) : 0.f);
      }
    }
  };
  // Fragment addresses: slab u wants k-chunk 2 u + l / 32 of row l % 32 (+ 32 per row tile, an
  // immediate).  xaddr[u] points into the tile slab u is read from next and flips to the other
  // tile after each use; slab 0 is read one tile ahead (by slab 7 of the tile before).
  Int4Magic magic;
  if constexpr (INT4) magic.pin<false>();
  // entry j of the dword w of one slab: Int4Magic's (offsets on), or the table's entry for byte j of w
  auto level_entry = [&](uint32_t w, int j) -> uint32_t {
    if constexpr (INT4) return int4_entry_offset(magic, w, j);
    else return lds_ld32(__builtin_amdgcn_perm(w, lane_off, 0x0c020400u + ((uint32_t)j << 8)));
  };
  // the two levels of byte b of a slab's dword times scale j of ring stage d, from that slab's entries
  auto pair_products = [&](const uint32_t (&e)[4], int b, int d, int cg, int j, float& p0, float& p1) {
    _Float16 l0, l1;
    level_pair<INT4>(e, b, l0, l1);
    const float sv = sc[d][cg][j];
    p0 = __builtin_fmaf((float)l0, sv, INT4 ? sb[INT4 ? d : 0][cg][j][0] : 0.0f);
    p1 = __builtin_fmaf((float)l1, sv, INT4 ? sb[INT4 ? d : 0][cg][j][1] : 0.0f);
  };
  uint32_t xaddr[8];
#pragma unroll
  for (int u = 0; u < 8; ++u)
    xaddr[u] = (uint32_t)l32 * 256u + (((uint32_t)(2 * u + lh) ^ (uint32_t)(l32 & 15)) * 16u) + (u == 0 ? kWideTileBytes : 0u);
  uint32_t dma_buf = 0;     // the tile buffer that slab 7 of the current k-tile refills

  // One slab (16 k) = eight slots, one MFMA each (column group i / 4, row tile i % 4), written
  // in the order they should issue.  Slot i also carries, for code pair (group i / 4, byte i % 4):
  // the two f16 x scale products and the bf16 pack of that pair of the NEXT slab's weights, the
  // table look-up (address: one v_perm) of the same pair of the slab AFTER the next, which
  // overwrites the entry just consumed, and in even slots an activation fragment read for the
  // next slab.  Slab 5 expands the next k-tile's scales; slab 6 requests the weights of k-tile
  // kt + PF into the ring stage this tile has finished with; the barrier sits between slabs 6
  // and 7 (the fragments slab 7 reads are the next tile's, requested by slab 7 of the tile
  // before); slab 7 requests the activations of k-tile kt + 2 into the tile buffer this k-tile
  // has been read from (every wave's fragment reads of it completed before the barrier).
  auto slab = [&](auto Uc, auto Dc, int kt, bool next_active) {
    constexpr int U = decltype(Uc)::value, D = decltype(Dc)::value, DN = (D + 1) % PF;
    constexpr int CUR = U & 1, NXT = CUR ^ 1;
    constexpr int UC = (U + 1) & 7, DC = U < 7 ? D : DN;   // slab whose weights are converted here
    constexpr int UL = (U + 2) & 7, DL = U < 6 ? D : DN;   // slab whose table entries are fetched here
    constexpr bool LW = U == 6, LD = U == 7, EX = U == 5;
    const bool ut = lora && kt + 2 >= ktiles;      // LD: the activation tile to fetch is the adapter block
    const int xs = ut ? 0 : min(kt + 2, ktiles - 1) * (KTILE * 2);
    const u32x4 xr = LD ? sel_rsrc(ut) : rx;
    const uint32_t um = 0u - (uint32_t)ut;
    const uint32_t xo = xbase ^ ((xbase ^ tbase) & um), xst = xstride ^ ((xstride ^ tstride) & um);
    const int wkt = min(kt + PF, ktiles - 1);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int cg = i >> 2, rt = i & 3;
      if constexpr (PRE) {
        // the fragment as loaded; once a column group's four MFMAs have read it, its stage takes
        // the same group's fragment of the slab kWidePreStages further on
        constexpr int SL = D * 8 + U;
        acc[rt][cg] = mfma32(wr[SL % kWidePreStages][cg], xf[CUR][rt], acc[rt][cg]);
        if (rt == 3) {
          const int sl = kt * 8 + U + kWidePreStages;   // (kt counts from this work-group's first k-tile: no k split here)
          const int kt_ = min(sl >> 3, ktiles - 1);
          wr[SL % kWidePreStages][cg] = __builtin_amdgcn_raw_buffer_load_b128(
              re, evoff[cg] + (uint32_t)((U + kWidePreStages) & 7) * 1024u, (ntile * ktiles + kt_) * 65536, 0);
        }
      } else {
      acc[rt][cg] = mfma32(wf[CUR][cg], xf[CUR][rt], acc[rt][cg]);
      {
        // the pack of the pair before this one (a slot behind its products: packed in the same
        // slot it would wait on them); slot 0 packs the last pair of the slab before, which
        // belongs to the fragment the MFMAs of slots 4-7 of THIS slab multiply
        if (i == 0) wf[CUR][CG - 1][3] = cvt_pk_bf16(cf0, cf1);
        else wf[NXT][(i - 1) >> 2][(i - 1) & 3] = cvt_pk_bf16(cf0, cf1);
        pair_products(lp[INT4 ? (UC & 1) : 0][cg], rt, DC, cg, SPT == 2 ? (UC >> 2) : (UC >> 1), cf0, cf1);
        lp[INT4 ? (UL & 1) : 0][cg][rt] = level_entry(ring_c[DL][cg][UL & 1][UL >> 1], rt);
      }
      }
      if ((i & 1) == 0) xf[NXT][i >> 1] = lds_ld128(xaddr[UC] + (uint32_t)((i >> 1) * 32 * 256));
      if (i == 7) xaddr[UC] ^= kWideTileBytes;
      if (LD) dma16(dma_buf + dma_wave + (uint32_t)i * 4096u, xr, xoff(i, xo, xst), xs);
      if (LW && !PRE) {
        if (i < 4) ring_c[D][i >> 1][i & 1] = __builtin_amdgcn_raw_buffer_load_b128(rc, coff[i >> 1] + (uint32_t)(i & 1) * 512u, wkt * 1024, 0);
        else if (i < 6) load_scale(Dc, i - 4, wkt);
      }
      if (EX && !PRE && i < CG * SPT) {
        const uint32_t w = ring_s[DN][i / SPT][(i % SPT) >> 1];
        set_scale(DN, i / SPT, i % SPT, next_active ? (((i % SPT) & 1) ? bfhi(w) : bflo(w)) : 0.f);
      }
      __builtin_amdgcn_sched_barrier(0);   // slots issue in the order written
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto tile = [&](auto Dc, int kt) {
    const bool next_active = kt + 1 < ktiles;
    __builtin_amdgcn_sched_barrier(0);
    slab(ic<0>{}, Dc, kt, next_active);
    slab(ic<1>{}, Dc, kt, next_active);
    slab(ic<2>{}, Dc, kt, next_active);
    slab(ic<3>{}, Dc, kt, next_active);
    slab(ic<4>{}, Dc, kt, next_active);
    slab(ic<5>{}, Dc, kt, next_active);
    slab(ic<6>{}, Dc, kt, next_active);
    // the next tile's activations, requested by slab 7 of the tile before, have landed in LDS:
    // the only younger loads are the six weight / scale loads slab 6 has just issued (PRE: the
    // second fragment load of that slab 7 and the two of each slab since, fifteen)
    tnx_wait_vm(PRE ? 14 : 6);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    slab(ic<7>{}, Dc, kt, next_active);
    dma_buf ^= kWideTileBytes;
  };

  // (order of the first loads: each is followed by at least as many later loads as it will be
  // in the steady state of the loop, so the counted waits of the loop body never have to fall
  // back to "everything outstanding" for the sake of the path that enters from here)
  load_a(0, 0u);
  if constexpr (PRE) {
#pragma unroll
    for (int sl = 0; sl < kWidePreStages; ++sl)
#pragma unroll
      for (int cg = 0; cg < CG; ++cg) load_pre(sl, sl & 7, cg);
  } else {
    load_w(ic<0>{}, 0);
  }
  if constexpr (MODE == kWideTable) {  // table entry e = f16 pair (level[e & 15], level[e >> 4]), 64 copies rotated over the banks
    uint32_t* lut = reinterpret_cast<uint32_t*>(smem + kWideLutBase);
    const h16x2 h = {(_Float16)lvl0, (_Float16)lvl1};
    const uint32_t v = __builtin_bit_cast(uint32_t, h);
#pragma unroll
    for (int c = 0; c < 64; ++c) lut[tid * 64 + ((c + lane) & 63)] = v;
  }
  load_a(1, kWideTileBytes);
  if constexpr (!PRE) {
    load_w(ic<1>{}, 1);
    load_w(ic<2>{}, 2);
  }
  // the adapter's B^T fragments: up front, or (two work-groups per unit: no registers to park
  // them in) behind the loop, where the other work-group covers their round trip
  auto load_adapter_b = [&]() {
    const rsrc_t rb = make_rsrc(a.lora_b, (uint64_t)a.N * a.lora_rank * 2);
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (u * 16 < a.lora_rank)
          lbv[cg][u] = buf_load128(rb, (((uint32_t)(ntile0 + 2 * cg) * 16u + (uint32_t)l32) * (uint32_t)a.lora_rank +
                                        (uint32_t)(u * 16 + lh * 8)) * 2u);
  };
  constexpr bool LATE_B = PRE;
  if (lora && !LATE_B) load_adapter_b();
  if constexpr (!PRE) expand_scales(ic<0>{}, true);
  // the first tile is in LDS: its eight loads are the oldest, and at least 26 follow them (three
  // ring stages of six, the second tile's eight); vmcnt(20) also covers the first ring stage
  // (PRE: 24 fragment loads and the second tile's eight follow them)
  tnx_wait_vm(PRE ? 2 * kWidePreStages + 8 : 20);
  __syncthreads();
  // slab 0: table entries, conversion, fragments; then the table entries of slab 1
  if constexpr (!PRE) {
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
      for (int b = 0; b < 4; ++b) lp[0][cg][b] = level_entry(ring_c[0][cg][0][0], b);
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) xf[0][rt] = lds_ld128((xaddr[0] ^ kWideTileBytes) + (uint32_t)(rt * 32 * 256));
  if constexpr (!PRE) {
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        pair_products(lp[0][cg], b, 0, cg, 0, cf0, cf1);
        if (cg < CG - 1 || b < 3) wf[0][cg][b] = cvt_pk_bf16(cf0, cf1);   // the last pair: slot 0 of the loop
      }
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
      for (int b = 0; b < 4; ++b) lp[INT4 ? 1 : 0][cg][b] = level_entry(ring_c[0][cg][1][0], b);
  }
  // whole turns of the ring without a branch inside (a conditional tile would make the waits
  // of the tile after it assume that its loads never happened), then the one or two tiles left
  int kt = 0;
  for (; kt + PF <= ktiles; kt += PF) {
    tile(ic<0>{}, kt);
    tile(ic<1>{}, kt + 1);
    tile(ic<2>{}, kt + 2);
  }
  if (kt < ktiles) {
    tile(ic<0>{}, kt);
    if (kt + 1 < ktiles) tile(ic<1>{}, kt + 1);
  }

  if (lora) {
    if constexpr (LATE_B) load_adapter_b();
    // The t block is k-tile number ktiles: it sits in tile buffer ktiles % 2.  The
    // two 16-column halves of a group may belong to different adapters (always so for a
    // gate | up pair): one pass per half then, the other half's lanes contributing zeros.
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
      const bool same = toff[2 * cg] == toff[2 * cg + 1];
      f32x16 part[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 16; ++i) part[rt][i] = 0.f;
      for (int p = 0; p < (same ? 1 : 2); ++p) {
        const uint32_t half = toff[2 * cg + p] == toff_a ? 0u : 8u;   // first 16-byte chunk of the segment's 64 columns
        const uint32_t base = (uint32_t)(ktiles & 1) * kWideTileBytes + (uint32_t)l32 * 256u;
        const bool mine = same || (l32 >> 4) == p;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (u * 16 < a.lora_rank) {
            const u32x4 lb = mine ? lbv[cg][u] : u32x4{0, 0, 0, 0};
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
              part[rt] = mfma32(lb, lds_ld128(base + (uint32_t)(rt * 32 * 256) +
                                              (((half + (uint32_t)(2 * u + lh)) ^ (uint32_t)(l32 & 15)) * 16u)), part[rt]);
          }
        }
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[rt][cg][i] += a.lora_scale * part[rt][i];
    }
  }
  tnx_wait_vm(0);   // no load into LDS is still on its way
  __syncthreads();  // every wave is done with the activation buffers: they become the output stage

  // The bf16 tile goes through LDS (row stride cols + 8 elements) and leaves as 16-byte chunks
  // of whole rows.  A lane holds, for row rt * 32 + l % 32 and group cg, the columns
  // 8 b + 4 (l / 32) + e of the group in register 4 b + e.
  const bool mul = a.epilogue == TNX_EPI_SILU_MUL || a.epilogue == TNX_EPI_GELU_MUL;
  const int cols = mul ? kWideCols / 2 : kWideCols;      // output columns of the work-group
  const int sld = cols + 8;
  const uint32_t stage = 0;   // 128 rows x (256 + 8) columns: over both tiles and into the table, all dead now
  if (mul) {
    // a group is [16 gate columns | 16 up columns]: registers 4 b + e (b < 2) and 4 (b + 2) + e
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float g = rbf(acc[rt][cg][4 * b + e]);
            const float u = rbf(acc[rt][cg][4 * (b + 2) + e]);
            const float act = a.epilogue == TNX_EPI_SILU_MUL ? silu_bf16(g) : gelu_tanh_bf16(g);
            v[e] = rbf(act) * u;
          }
          const u32x2 pk = {pack2bf(v[0], v[1]), pack2bf(v[2], v[3])};
          const uint32_t at = stage + (uint32_t)(((rt * 32 + l32) * sld + wn * 32 + cg * 16 + 8 * b + 4 * lh) * 2);
          *reinterpret_cast<__attribute__((address_space(3))) u32x2*>(static_cast<uintptr_t>(at)) = pk;
        }
  } else {
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const u32x2 pk = {pack2bf(acc[rt][cg][4 * b], acc[rt][cg][4 * b + 1]),
                            pack2bf(acc[rt][cg][4 * b + 2], acc[rt][cg][4 * b + 3])};
          const uint32_t at = stage + (uint32_t)(((rt * 32 + l32) * sld + wn * 64 + cg * 32 + 8 * b + 4 * lh) * 2);
          *reinterpret_cast<__attribute__((address_space(3))) u32x2*>(static_cast<uintptr_t>(at)) = pk;
        }
  }
  __syncthreads();
  if (h.part != nullptr && h.logits_out != nullptr) {
    // the raw logits (no temperature) as fp32: a wave writes one row of the tile at a time, a
    // lane four columns (1 KB per row, whole lines)
    const int64_t c0 = (int64_t)ntile * kWideCols + lane * 4;
    for (int row = wn; row < rows_here; row += 4) {
      const u32x2 v = *reinterpret_cast<const __attribute__((address_space(3))) u32x2*>(
          static_cast<uintptr_t>(stage + (uint32_t)((row * sld + lane * 4) * 2)));
      float* o = h.logits_out + (m0 + row) * a.N + c0;
      if (c0 + 4 <= a.N) {
        *reinterpret_cast<f32x4*>(o) = f32x4{bflo(v[0]), bfhi(v[0]), bflo(v[1]), bfhi(v[1])};
      } else {
        const float x[4] = {bflo(v[0]), bfhi(v[0]), bflo(v[1]), bfhi(v[1])};
        for (int e = 0; e < 4; ++e)
          if (c0 + e < a.N) o[e] = x[e];
      }
    }
  }
  if (h.part != nullptr) {
    // lm_head: thread (row, half) reduces the row's 128 staged logits of column block
    // 2 * ntile + half to (max, first arg-max, sum of exp(l - max), logit of the row's target)
    const int row = tid & 127, half = tid >> 7;
    const int64_t pb = (int64_t)ntile * 2 + half;
    if (row >= rows_here || pb >= h.nvb) return;
    const int64_t grow = m0 + row, c0 = pb * 128;
    const int tg = h.targets ? h.targets[grow] : -1;
    const uint32_t base = stage + (uint32_t)((row * sld + half * 128) * 2);
    const float ninf = -__builtin_inff();
    float mx = ninf, tgt = ninf, se = 0.f, we = 0.f;
    int idx = (int)c0;
    // The logits are divided by the temperature in fp32, as the reference does.  At temperature 1
    // the division is the identity and is left out: an IEEE division is a dozen instructions, and
    // at two per element it was a seventh of this kernel's time on the log-probability pass.
    auto reduce = [&](auto unit_c) {
      constexpr bool unit = decltype(unit_c)::value;
#pragma unroll 4
      for (int ch = 0; ch < 16; ++ch) {
        const u32x4 v = lds_ld128(base + (uint32_t)(ch * 16));
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          const int64_t col = c0 + ch * 8 + q;
          const float raw = (q & 1) ? bfhi(v[q >> 1]) : bflo(v[q >> 1]);
          const float l = col < a.N ? (unit ? raw : __fdiv_rn(raw, h.temperature)) : ninf;
          if (l > mx) {   // columns ascend: the first maximal index stays
            mx = l;
            idx = (int)col;
          }
          if ((int)col == tg) tgt = l;
        }
      }
      if (mx != ninf) {
#pragma unroll 4
        for (int ch = 0; ch < 16; ++ch) {
          const u32x4 v = lds_ld128(base + (uint32_t)(ch * 16));
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const int64_t col = c0 + ch * 8 + q;
            const float raw = (q & 1) ? bfhi(v[q >> 1]) : bflo(v[q >> 1]);
            if (col < a.N) {
              const float l = unit ? raw : __fdiv_rn(raw, h.temperature);
              const float e = __expf(l - mx);
              se += e;
              we += e * l;
            }
          }
        }
      }
    };
    // A block that lies wholly inside the vocabulary, no entropy term asked for (every block of a
    // log-probability pass over a head whose width is a multiple of 128): the same arithmetic in
    // the same order without the per-element column tests, and the target's logit is read from its
    // place in the staged row instead of being compared for 128 times.
    auto reduce_full = [&](auto unit_c) {
      constexpr bool unit = decltype(unit_c)::value;
      const int c0i = (int)c0;
      if (tg >= c0i && tg < c0i + 128) {
        const uint32_t w = lds_ld32(base + (uint32_t)((tg - c0i) >> 1) * 4u);
        const float raw = ((tg - c0i) & 1) ? bfhi(w) : bflo(w);
        tgt = unit ? raw : __fdiv_rn(raw, h.temperature);
      }
#pragma unroll 4
      for (int ch = 0; ch < 16; ++ch) {
        const u32x4 v = lds_ld128(base + (uint32_t)(ch * 16));
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          const float raw = (q & 1) ? bfhi(v[q >> 1]) : bflo(v[q >> 1]);
          const float l = unit ? raw : __fdiv_rn(raw, h.temperature);
          if (l > mx) {
            mx = l;
            idx = c0i + ch * 8 + q;
          }
        }
      }
      if (mx != ninf) {
#pragma unroll 4
        for (int ch = 0; ch < 16; ++ch) {
          const u32x4 v = lds_ld128(base + (uint32_t)(ch * 16));
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const float raw = (q & 1) ? bfhi(v[q >> 1]) : bflo(v[q >> 1]);
            const float l = unit ? raw : __fdiv_rn(raw, h.temperature);
            se += __expf(l - mx);
          }
        }
      }
    };
    // The whole-vocabulary draw: the statistics of the general form and, per column, the logit
    // plus the Gumbel noise of element row * N + col of rows_total * N; the block's best (first
    // among equals: columns ascend), its id and its logit go to part_draw.
    if (h.part_draw != nullptr) {
      uint32_t ks0 = 0u, ks1 = (uint32_t)(*h.step_ptr);
      threefry2x32(h.key0, h.key1, ks0, ks1);   // fold_in(key, step)
      const uint64_t total = (uint64_t)h.rows_total * (uint64_t)a.N;
      float gv = ninf, gl = ninf;
      int gi = 0x7fffffff;
      for (int ch = 0; ch < 16; ++ch) {
        const u32x4 v = lds_ld128(base + (uint32_t)(ch * 16));
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          const int64_t col = c0 + ch * 8 + q;
          if (col < a.N) {
            const float raw = (q & 1) ? bfhi(v[q >> 1]) : bflo(v[q >> 1]);
            const float l = __fdiv_rn(raw, h.temperature);
            const float n = l + gumbel_from_bits(random_bits(ks0, ks1, (uint64_t)grow * (uint64_t)a.N + (uint64_t)col,
                                                             total, h.variant));
            if (n > gv) {
              gv = n;
              gi = (int)col;
              gl = l;
            }
          }
        }
      }
      float* q3 = h.part_draw + (grow * h.nvb + pb) * 3;
      q3[0] = gv;
      q3[1] = __int_as_float(gi);
      q3[2] = gl;
    }
    const bool plain = c0 + 128 <= a.N && h.part_ent == nullptr;
    if (h.temperature == 1.0f) {
      if (plain) reduce_full(std::true_type{});
      else reduce(std::true_type{});
    } else {
      if (plain) reduce_full(std::false_type{});
      else reduce(std::false_type{});
    }
    float* p = h.part + (grow * h.nvb + pb) * 4;
    p[0] = mx;
    p[1] = __int_as_float(idx);
    p[2] = se;
    p[3] = tgt;
    if (h.part_ent) h.part_ent[grow * h.nvb + pb] = we;
    return;
  }
  {
    const int64_t ldy = mul ? a.N / 2 : a.N;
    const int64_t col0 = (int64_t)ntile * cols;
    const int chunks = cols / 8;                       // 16-byte chunks per row: 16 | 32
    const int ch = tid % chunks, r0 = tid / chunks, rstep = 256 / chunks;
    uint16_t* y = reinterpret_cast<uint16_t*>(a.y);
    const bool col_ok = col0 + ch * 8 + 8 <= ldy;
    for (int row = r0; row < kWideRows; row += rstep) {
      if (row >= rows_here || !col_ok) continue;
      u32x4 v = lds_ld128(stage + (uint32_t)((row * sld + ch * 8) * 2));
      const int64_t orow = GROUPED ? (int64_t)a.sorted_route[m0 + row] : m0 + row;
      const int64_t o = orow * ldy + col0 + ch * 8;
      if (a.epilogue == TNX_EPI_RESIDUAL) {
        const u32x4 res = *reinterpret_cast<const u32x4*>(a.residual + o);
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = pack2bf(bflo(v[q]) + bflo(res[q]), bfhi(v[q]) + bfhi(res[q]));
      }
      *reinterpret_cast<u32x4*>(y + o) = v;
    }
  }
}

}  // namespace
