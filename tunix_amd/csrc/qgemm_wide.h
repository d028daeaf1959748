// The quantised GEMM for many rows (prefill, per-token logps): output tile 128 rows x 256
// columns per work-group of four waves, one per SIMD with the whole register file (the 128
// accumulator registers of a wave's 128 x 64 block next to the operand pipeline).  Past a few
// hundred rows the op is bound by the matrix pipe, and what keeps the pipe waiting is the
// traffic between L2 and the compute unit: a 128 x 256 tile fetches 32 KB of activations and
// 17 KB of packed weights per k-tile for twice the MFMA work a 128 x 128 tile gets from
// 32 + 8.5 KB.  Same weight format, table look-up, conversion and software pipeline as
// qgemm128_kernel, but every wave walks all four k-steps of a k-tile (no k split inside the
// work-group, so no exchange of accumulators) and the products are formed transposed
// (weights as the MFMA's A operand): a lane then owns four consecutive output columns of one
// row, and the tile leaves through LDS as whole 16-byte row chunks.
//
// Work-groups are numbered so that the eight XCDs (consecutive work-group ids go to
// consecutive XCDs) each walk one 128-row block across the column tiles: a block's activations
// stay in that XCD's L2 while the weights of a column tile, wanted by all eight at about the
// same time, come out of the memory-side cache.
//
// Included by qlinear.hip after qgemm128.h.
#pragma once

namespace {

constexpr int kWideRows = 128, kWideCols = 256;
constexpr size_t kWideSmemBytes = kBigLutBytes + 2 * (size_t)kWideRows * A_LD * 2;

template <int SPT>
__global__ __launch_bounds__(256)
void qgemm_wide_kernel(const QLArgs a) {
  constexpr int NT = 4, MT = 8, PF = 3, AP = 8;
  constexpr uint32_t ABYTES = kWideRows * A_LD * 2;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wn = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lm = lane & 15, lq = lane >> 4;
  // LDS is addressed absolutely (table at 0)
  if ((uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem != 0u) return;
  asm volatile("" ::"s"(a.M), "s"(a.K), "s"(a.N), "s"(a.qtype), "s"(a.x), "s"(a.codes), "s"(a.scales),
               "s"(a.lora_rank), "s"(a.lora_nseg), "s"(a.lora_seg_end[0]), "s"(a.lora_seg_end[1]),
               "s"(a.lora_seg_end[2]), "s"(a.lora_seg_toff[0]), "s"(a.lora_seg_toff[1]),
               "s"(a.lora_seg_toff[2]), "s"(a.lora_seg_toff[3]));
  asm volatile("" ::"s"(a.t_ld), "s"(a.t), "s"(a.lora_b), "s"(a.lora_scale), "s"(a.epilogue), "s"(a.y),
               "s"(a.residual));
  const float lvl0 = rbf(code_level_imm(a.qtype, tid & 15)), lvl1 = rbf(code_level_imm(a.qtype, (tid >> 4) & 15));
  const uint32_t lane_off = (uint32_t)lane * 4u;

  // work-group id -> (row block, column tile): groups of eight row blocks, the column tile
  // moves every eight ids
  const int tiles_m = (int)((a.M + kWideRows - 1) / kWideRows), tiles_n = (int)((a.N + kWideCols - 1) / kWideCols);
  int mtile, ntile;
  {
    const int per_group = 8 * tiles_n;
    const int g = (int)blockIdx.x / per_group, r = (int)blockIdx.x % per_group;
    const int gm = min(8, tiles_m - g * 8);
    mtile = g * 8 + r % gm;
    ntile = r / gm;
  }
  const int64_t m0 = (int64_t)mtile * kWideRows;
  const int64_t ntile0 = ((int64_t)ntile * 4 + wn) * NT;
  const int64_t ntiles = a.N / 16;
  const int ktiles = (int)(a.K / KTILE);
  const int rows_here = (int)min((int64_t)kWideRows, a.M - m0);

  // the activation resource starts at this work-group's first row: offsets stay small whatever
  // M is, and rows past M lie beyond the resource and read zeros
  const rsrc_t rx = make_rsrc(a.x + m0 * a.K, (uint64_t)rows_here * a.K * 2);
  const uint64_t ntk = (uint64_t)ntiles * ktiles;
  const rsrc_t rc = make_rsrc(a.codes, ntk * 1024);
  const rsrc_t rs = make_rsrc(a.scales, ntk * 16 * SPT * 2 + 16);
  uint32_t coff[NT], soff[NT];
  const uint32_t xbase = ((uint32_t)(tid >> 4) * (uint32_t)a.K + (uint32_t)(tid & 15) * 8u) * 2u;
  const uint32_t xstride = 16u * (uint32_t)a.K * 2u;  // 16 rows further per pass
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const uint32_t tile0 = (uint32_t)(ntile0 + nt) * (uint32_t)ktiles;
    coff[nt] = tile0 * 1024u + (uint32_t)lane * 16u;
    soff[nt] = (tile0 * 16u + (uint32_t)lm) * (uint32_t)(SPT * 2);
  }

  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) zero_acc(acc[mt][nt]);

  u32x4 a_next[AP];
  u32x4 ring_c[PF][NT];
  u32x2 ring_s[PF][NT];
  float sc[PF][NT][SPT];
  u32x4 af[2][MT];
  u32x4 bfr[2][NT];
  uint32_t lp[NT][4];

  // LoRA: the k-tile after the last one is the 128-row block of t = bf16(x . A), columns
  // [toff_a, +64) | [toff_b, +64) (the host sends only shapes whose work-groups span at most
  // two adapter segments here); the B^T fragments of this wave's columns stay in registers.
  const bool lora = a.lora_rank > 0;
  int toff[NT];
  int toff_a = 0, toff_b = 0;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) toff[nt] = 0;
  if (lora) {
    if (a.lora_nseg < 0) {
      toff_b = a.lora_rank;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) toff[nt] = (int)((ntile0 + nt) & 1) * a.lora_rank;
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
      const int wg_nt0 = ntile * 4 * NT;
      toff_a = idx_toff(seg_idx(min(wg_nt0, last)));
      toff_b = idx_toff(seg_idx(min(wg_nt0 + 4 * NT - 1, last)));
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) toff[nt] = idx_toff(seg_idx(min((int)ntile0 + nt, last)));
    }
  }
  u32x4 lbv[NT][2];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int j = 0; j < 2; ++j) lbv[nt][j] = u32x4{0, 0, 0, 0};
  uint32_t tbase = 0;
  if (lora) {
    const int ch = tid & 15;
    const int col = ((ch < 8) ? toff_a : toff_b) + min((ch & 7) * 8, a.lora_rank - 8);
    tbase = (uint32_t)((tid >> 4) * a.t_ld + col) * 2u;
  }
  const rsrc_t rt = lora ? make_rsrc(a.t + m0 * a.t_ld, (uint64_t)rows_here * a.t_ld * 2) : rx;
  const uint32_t tstride = (uint32_t)(16 * a.t_ld * 2);

  auto load_a = [&](int kt) {
    const bool ut = lora && kt >= ktiles;
    const int s = ut ? 0 : min(kt, ktiles - 1) * (KTILE * 2);
    const rsrc_t r = ut ? rt : rx;
    const uint32_t m = 0u - (uint32_t)ut;
    const uint32_t base = xbase ^ ((xbase ^ tbase) & m), stride = xstride ^ ((xstride ^ tstride) & m);
#pragma unroll
    for (int c = 0; c < AP; ++c)
      a_next[c] = __builtin_amdgcn_raw_buffer_load_b128(r, base + (uint32_t)c * stride, s, 0);
  };
  auto load_w = [&](auto Dc, int kt) {
    constexpr int D = decltype(Dc)::value;
    const int ktc = min(kt, ktiles - 1);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      ring_c[D][nt] = __builtin_amdgcn_raw_buffer_load_b128(rc, coff[nt], ktc * 1024, 0);
      if constexpr (SPT == 2) {
        ring_s[D][nt][0] = __builtin_amdgcn_raw_buffer_load_b32(rs, soff[nt], ktc * (16 * SPT * 2), 0);
      } else {
        ring_s[D][nt] = __builtin_amdgcn_raw_buffer_load_b64(rs, soff[nt], ktc * (16 * SPT * 2), 0);
      }
    }
  };
  auto expand_scales = [&](auto Dc, bool active) {
    constexpr int D = decltype(Dc)::value;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int j = 0; j < SPT; ++j) {
        const uint32_t w = ring_s[D][nt][j >> 1];
        sc[D][nt][j] = active ? ((j & 1) ? bfhi(w) : bflo(w)) : 0.f;
      }
    }
  };
  auto lut_issue = [&](auto Dc, auto Jc, uint32_t (&dst)[NT][4]) {
    constexpr int D = decltype(Dc)::value, J = decltype(Jc)::value;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const uint32_t w = ring_c[D][nt][J];
      dst[nt][0] = lds_ld32(__builtin_amdgcn_perm(w, lane_off, 0x0c0c0400u));
      dst[nt][1] = lds_ld32(__builtin_amdgcn_perm(w, lane_off, 0x0c0c0500u));
      dst[nt][2] = lds_ld32(__builtin_amdgcn_perm(w, lane_off, 0x0c0c0600u));
      dst[nt][3] = lds_ld32(__builtin_amdgcn_perm(w, lane_off, 0x0c0c0700u));
    }
  };
  auto convert = [&](auto Dc, auto Jc, u32x4 (&dst)[NT], const uint32_t (&src)[NT][4]) {
    constexpr int D = decltype(Dc)::value, J = decltype(Jc)::value;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const float s = sc[D][nt][SPT == 2 ? (J >> 1) : J];
      u32x4 r;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const h16x2 h = __builtin_bit_cast(h16x2, src[nt][b]);
        r[b] = cvt_pk_bf16(__builtin_fmaf((float)h[0], s, 0.0f), __builtin_fmaf((float)h[1], s, 0.0f));
      }
      dst[nt] = r;
    }
  };
  uint32_t a_rd = kBigLutBytes + (uint32_t)(lm * A_LD + lq * 8) * 2u;
  uint32_t a_rd_nxt = a_rd + ABYTES;
  uint32_t a_wr = kBigLutBytes + (uint32_t)((tid >> 4) * A_LD + (tid & 15) * 8) * 2u;
  uint32_t a_wr_nxt = a_wr + ABYTES;
  auto read_a = [&](u32x4 (&dst)[MT], uint32_t base, auto Jc) {
    constexpr int J = decltype(Jc)::value;
#pragma unroll
    for (int m = 0; m < MT; ++m) dst[m] = lds_ld128(base + (uint32_t)((m * 16 * A_LD + J * 32) * 2));
  };
  auto store_a = [&](uint32_t base) {
#pragma unroll
    for (int c = 0; c < AP; ++c) lds_st128(base + (uint32_t)(c * 16 * A_LD * 2), a_next[c]);
  };
  // (the products are formed transposed: D[weight column][row] += W^T . x^T)
  // One k-step = 32 slots, one matrix instruction each, written in the order they should issue
  // (a wave that has its SIMD to itself hides nothing behind another wave: whatever does not
  // issue in the shadow of a matrix instruction adds to the loop).  Slot i multiplies
  // accumulator (row tile i % 8, column tile i / 8), and carries two vector instructions and at
  // most two memory instructions:
  //   even slots  the two f16 x scale products of code pair i / 2 of the NEXT step's weights,
  //               an activation fragment read for the next step (i < 16), an LDS write of the
  //               next activation tile (ST, i >= 16), a global load (LD);
  //   odd slots   the bf16 pack of that pair, and the table look-up (address: one v_perm) of
  //               the same pair of the step AFTER the next, which overwrites the entry the
  //               even slot just consumed.
  // Column tile nt of the next step's weights is complete after slot 8 nt + 7, and the next
  // step uses it from its slot 8 nt on.  The group barriers restate the slot contents for the
  // machine scheduler.
  auto step = [&](auto CURc, auto Dcc, auto Jcc, auto Dlc, auto Jlc, uint32_t rd_base, auto Jrc, auto STc,
                  auto LDc, auto EXc, int kt, bool ex_active) {
    constexpr int CUR = decltype(CURc)::value, NXT = CUR ^ 1;
    constexpr int DC = decltype(Dcc)::value, JC = decltype(Jcc)::value;
    constexpr int DL = decltype(Dlc)::value, JL = decltype(Jlc)::value, JR = decltype(Jrc)::value;
    constexpr bool ST = decltype(STc)::value != 0, LD = decltype(LDc)::value != 0;
    constexpr int EX = decltype(EXc)::value;   // -1, or the ring stage whose scales to expand
    float f0 = 0.f, f1 = 0.f;
    const bool ut = lora && kt >= ktiles;      // LD: the tile to fetch is the adapter block
    const int xs = ut ? 0 : min(kt, ktiles - 1) * (KTILE * 2);
    const rsrc_t xr = ut ? rt : rx;
    const uint32_t um = 0u - (uint32_t)ut;
    const uint32_t xb = xbase ^ ((xbase ^ tbase) & um), xst = xstride ^ ((xstride ^ tstride) & um);
    const int wkt = min(kt + (PF - 2), ktiles - 1);   // LD: weights of k-tile (this + PF)
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      const int nt = i >> 3, m = i & 7, pr = i >> 1, pnt = pr >> 2, pb = pr & 3;
      acc[m][nt] = mfma16(bfr[CUR][nt], af[CUR][m], acc[m][nt]);
      if ((i & 1) == 0) {
        const h16x2 h = __builtin_bit_cast(h16x2, lp[pnt][pb]);
        const float sv = sc[DC][pnt][SPT == 2 ? (JC >> 1) : JC];
        f0 = __builtin_fmaf((float)h[0], sv, 0.0f);
        f1 = __builtin_fmaf((float)h[1], sv, 0.0f);
        if (i < 16) af[NXT][i >> 1] = lds_ld128(rd_base + (uint32_t)(((i >> 1) * 16 * A_LD + JR * 32) * 2));
        if (ST && i >= 16) lds_st128(a_wr_nxt + (uint32_t)(((i - 16) >> 1) * 16 * A_LD * 2), a_next[(i - 16) >> 1]);
        if (LD) {
          const int q = i >> 1;
          if (q < 8) {
            a_next[q] = __builtin_amdgcn_raw_buffer_load_b128(xr, xb + (uint32_t)q * xst, xs, 0);
          } else if (q < 12) {
            ring_c[DL == 0 ? PF - 1 : DL - 1][q - 8] = __builtin_amdgcn_raw_buffer_load_b128(rc, coff[q - 8], wkt * 1024, 0);
          } else if constexpr (SPT == 2) {
            ring_s[DL == 0 ? PF - 1 : DL - 1][q - 12][0] =
                __builtin_amdgcn_raw_buffer_load_b32(rs, soff[q - 12], wkt * (16 * SPT * 2), 0);
          } else {
            ring_s[DL == 0 ? PF - 1 : DL - 1][q - 12] =
                __builtin_amdgcn_raw_buffer_load_b64(rs, soff[q - 12], wkt * (16 * SPT * 2), 0);
          }
        }
      } else {
        bfr[NXT][pnt][pb] = cvt_pk_bf16(f0, f1);
        lp[pnt][pb] = lds_ld32(__builtin_amdgcn_perm(ring_c[DL][pnt][JL], lane_off, 0x0c0c0400u + ((uint32_t)pb << 8)));
      }
      if (EX >= 0 && i < NT * SPT) {
        const int ent = i / SPT, ej = i % SPT;
        const uint32_t w = ring_s[EX < 0 ? 0 : EX][ent][ej >> 1];
        sc[EX < 0 ? 0 : EX][ent][ej] = ex_active ? ((ej & 1) ? bfhi(w) : bflo(w)) : 0.f;
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
      if (EX >= 0 && i < NT * SPT) __builtin_amdgcn_sched_group_barrier(0x002, 1, 0);
      if ((i & 1) == 1 || i < 16) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if (ST && (i & 1) == 0 && i >= 16) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
      if (LD && (i & 1) == 0) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // One k-tile of ring stage D.  On entry af[0] / bfr[0] hold the fragments of k-step 0 and lp
  // the table entries of k-step 1.  Step 2 stores the next activation tile (fetched by step 3 of
  // the tile before), the barrier sits before step 3 (whose fragment reads are the first of the
  // next tile), and step 3 issues the global loads: activations of k-tile kt + 2, weights of
  // k-tile kt + PF into the ring stage this tile has just finished with.
  auto tile = [&](auto Dc, int kt) {
    constexpr int d = decltype(Dc)::value, dn = (d + 1) % PF;
    const bool next_active = kt + 1 < ktiles;
    __builtin_amdgcn_sched_barrier(0);
    step(ic<0>{}, Dc, ic<1>{}, Dc, ic<2>{}, a_rd, ic<1>{}, ic<0>{}, ic<0>{}, ic<-1>{}, 0, false);
    step(ic<1>{}, Dc, ic<2>{}, Dc, ic<3>{}, a_rd, ic<2>{}, ic<0>{}, ic<0>{}, ic<-1>{}, 0, false);
    step(ic<0>{}, Dc, ic<3>{}, ic<dn>{}, ic<0>{}, a_rd, ic<3>{}, ic<1>{}, ic<0>{}, ic<dn>{}, 0, next_active);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    step(ic<1>{}, ic<dn>{}, ic<0>{}, ic<dn>{}, ic<1>{}, a_rd_nxt, ic<0>{}, ic<0>{}, ic<1>{}, ic<-1>{}, kt + 2, false);
    const uint32_t r = a_rd; a_rd = a_rd_nxt; a_rd_nxt = r;
    const uint32_t w = a_wr; a_wr = a_wr_nxt; a_wr_nxt = w;
  };

  // (order of the first loads: each is followed by at least as many later loads as it will be
  // in the steady state of the loop, so the counted waits of the loop body never have to fall
  // back to "everything outstanding" for the sake of the path that enters from here)
  load_a(0);
  load_w(ic<0>{}, 0);
  {  // table entry e = f16 pair (level[e & 15], level[e >> 4]), 64 copies rotated over the banks
    uint32_t* lut = reinterpret_cast<uint32_t*>(smem);
    const h16x2 h = {(_Float16)lvl0, (_Float16)lvl1};
    const uint32_t v = __builtin_bit_cast(uint32_t, h);
#pragma unroll
    for (int c = 0; c < 64; ++c) lut[tid * 64 + ((c + lane) & 63)] = v;
  }
  store_a(a_wr);
  load_a(1);
  load_w(ic<1>{}, 1);
  load_w(ic<2>{}, 2);
  if (lora) {
    const rsrc_t rb = make_rsrc(a.lora_b, (uint64_t)a.N * a.lora_rank * 2);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        if (j * 32 < a.lora_rank)
          lbv[nt][j] = buf_load128(rb, (((uint32_t)(ntile0 + nt) * 16u + (uint32_t)lm) * (uint32_t)a.lora_rank +
                                        (uint32_t)(j * 32 + lq * 8)) * 2u);
  }
  expand_scales(ic<0>{}, true);
  __syncthreads();
  lut_issue(ic<0>{}, ic<0>{}, lp);
  read_a(af[0], a_rd, ic<0>{});
  convert(ic<0>{}, ic<0>{}, bfr[0], lp);
  lut_issue(ic<0>{}, ic<1>{}, lp);
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
    // the t block sits in the activation buffer the last k-tile left as "next" (now a_rd)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const uint32_t base = a_rd + (uint32_t)((toff[nt] == toff_a ? 0 : 64) * 2);
      f32x4 part[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) zero_acc(part[mt]);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (j * 32 < a.lora_rank) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            part[mt] = mfma16(lbv[nt][j], lds_ld128(base + (uint32_t)((mt * 16 * A_LD + j * 32) * 2)), part[mt]);
        }
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[mt][nt][i] += a.lora_scale * part[mt][i];
    }
  }
  __syncthreads();  // every wave is done with the activation buffers: they become the output stage

  // The bf16 tile goes through LDS (row stride cols + 8 elements) and leaves as 16-byte chunks
  // of whole rows.  A lane holds, for row mt * 16 + lm, the four columns nt * 16 + lq * 4 + i.
  const bool mul = a.epilogue == TNX_EPI_SILU_MUL || a.epilogue == TNX_EPI_GELU_MUL;
  const int cols = mul ? kWideCols / 2 : kWideCols;      // output columns of the work-group
  const int sld = cols + 8;
  const uint32_t stage = kBigLutBytes;
  if (mul) {
#pragma unroll
    for (int p = 0; p < NT / 2; ++p)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float g = rbf(acc[mt][2 * p][i]);
          const float u = rbf(acc[mt][2 * p + 1][i]);
          const float act = a.epilogue == TNX_EPI_SILU_MUL ? silu_bf16(g) : gelu_tanh_bf16(g);
          v[i] = rbf(act) * u;
        }
        const u32x2 pk = {pack2bf(v[0], v[1]), pack2bf(v[2], v[3])};
        const uint32_t at = stage + (uint32_t)(((mt * 16 + lm) * sld + wn * 32 + p * 16 + lq * 4) * 2);
        *reinterpret_cast<__attribute__((address_space(3))) u32x2*>(static_cast<uintptr_t>(at)) = pk;
      }
  } else {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const u32x2 pk = {pack2bf(acc[mt][nt][0], acc[mt][nt][1]), pack2bf(acc[mt][nt][2], acc[mt][nt][3])};
        const uint32_t at = stage + (uint32_t)(((mt * 16 + lm) * sld + wn * 64 + nt * 16 + lq * 4) * 2);
        *reinterpret_cast<__attribute__((address_space(3))) u32x2*>(static_cast<uintptr_t>(at)) = pk;
      }
  }
  __syncthreads();
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
      const int64_t o = (m0 + row) * ldy + col0 + ch * 8;
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
