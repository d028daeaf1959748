// Shared main loop of the skinny GEMMs (quantized linears, MoE grouped GEMM, lm_head).
//
// A work-group of 4 waves owns 16*MT activation rows (MT = 8: a rollout batch of 128) and
// 64*NT output columns; wave w owns NT column tiles of 16.  The activation tile [16*MT x 128k]
// is loaded straight into LDS once per k-tile (double buffered, 256-byte rows whose 16-byte
// chunks are XOR-swizzled by row) and read as MFMA A fragments; weights go
// HBM -> registers (one 128-bit buffer load per lane and k-tile for QW codes), are expanded to
// bf16 through a bank-replicated LDS table and multiplied by their group scale in registers:
// the MFMA B operand is bf16(bf16(level) * scale), i.e. the weight "dequantised to bf16", and
// the fp32 accumulators are touched by nothing but MFMA until the epilogue.
//
// Latency: a work-group runs alone on its CU (one wave per SIMD), so HBM latency is covered
// by a register ring of PF weight k-tiles in flight per wave and the L2 latency of the
// activations by requesting a tile one k-tile ahead of its use.  All loads are raw buffer
// loads: out-of-range rows / tiles read zeros without branches.
#pragma once
#include "common.h"

constexpr int KTILE = 128;
constexpr int A_LD = KTILE;      // bf16 elements per LDS row (256 B, no padding: the chunks are swizzled)
constexpr size_t tile_smem_bytes(int mt) {
  return 2 * (size_t)mt * 16 * A_LD * sizeof(uint16_t) + TNX_LUT_WORDS * sizeof(uint32_t);
}
// LDS layout: [2][16*MT][A_LD] bf16 activation buffers, then the code-book table.
__device__ __forceinline__ uint32_t* tile_lut(unsigned char* smem, int mt) {
  return reinterpret_cast<uint32_t*>(smem + 2 * (size_t)mt * 16 * A_LD * sizeof(uint16_t));
}

struct TileSrc {
  int64_t M, K;
  const uint16_t* x;         // bf16 [M,K] (or gathered through row_index)
  const int32_t* row_index;  // optional: LDS row r reads x row row_index[m0 + r] / row_div
  int row_div;
  int64_t x_rows;            // rows of the x allocation (== M unless gathered)
  const uint16_t* w_bf16;    // dense bf16 [N,K] (DENSE) ...
  const uint32_t* codes;     // ... or QW codes / scales
  const uint16_t* scales;
  int group, qtype;
  int64_t ntiles;            // N / 16
  int lora_rank;
  const uint16_t* t;
  int64_t t_ld;
  const uint16_t* lora_b;
  float lora_scale;
};

__device__ __forceinline__ void zero_acc(f32x4& v) { v = f32x4{0.f, 0.f, 0.f, 0.f}; }

// A buffer descriptor in scalar registers, for loads written in assembly.
__device__ __forceinline__ u32x4 raw_rsrc(const void* p, uint64_t bytes) {
  const uint64_t q = (uint64_t)p;
  const uint32_t n = (uint32_t)(bytes > 0xffffffffull ? 0xffffffffull : bytes);
  return u32x4{(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)q),
               (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)(q >> 32) & 0xffffu)),
               (uint32_t)__builtin_amdgcn_readfirstlane((int)n), 0x00020000u};
}
// One 16-byte-per-lane load from a buffer straight into LDS, at byte address `lds` + 16 * lane
// (M0 carries the wave-uniform base; lanes past the buffer write zeros).  The compiler does not
// count these loads: its own waits for other loads can only turn out longer than needed (loads
// complete in order), and the waits for these are written by hand (tnx_wait_vm).
// (The s_nop covers what the compiler's hazard handling cannot see inside the assembly: M0 written
// just before its use, and a descriptor or offset register written by a vector instruction --
// v_readfirstlane -- within the five slots before a memory instruction reads it.)
__device__ __forceinline__ void dma16(uint32_t lds, const u32x4& r, uint32_t voff, int soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :: "s"(lds), "v"(voff), "s"(r), "s"(soff) : "memory", "m0");
}
// s_waitcnt vmcnt(N) alone (the other counters at their maximum)
#define tnx_wait_vm(N) __builtin_amdgcn_s_waitcnt(0x0f70 | ((N) & 15) | (((N) >> 4) << 14))

// Rows [m0, m0+16*MT) x k-tile kt of x -> the LDS tile at byte address `lds`.  Thread t fills
// chunk t % 16 of rows t / 16 + 16 c (a wave: 1 KB = four consecutive rows) and fetches for it
// the k-chunk (t % 16) ^ (row % 16): the 16 lanes that read one k-chunk of 16 consecutive rows
// as an MFMA fragment then hit 16 different bank groups.  Rows beyond M read zeros (buffer
// bounds) or a clamped row (gather).
template <int MT>
__device__ __forceinline__ void load_a(const TileSrc& s, const u32x4& rx, int64_t m0, int kt, int tid,
                                       uint32_t lds) {
  const uint32_t wave_lds = lds + (uint32_t)__builtin_amdgcn_readfirstlane(tid >> 6) * 1024u;
  const uint32_t ch = (uint32_t)((tid & 15) ^ ((tid >> 4) & 15));
#pragma unroll
  for (int c = 0; c < MT; ++c) {
    int64_t src = m0 + (tid >> 4) + 16 * c;
    if (s.row_index) src = s.row_index[src < s.M ? src : s.M - 1] / s.row_div;
    // 32-bit offset: the host checks (rows + 128) * K * 2 < 4 GiB
    dma16(wave_lds + (uint32_t)c * 4096u, rx, ((uint32_t)src * (uint32_t)s.K + (uint32_t)kt * KTILE + ch * 8u) * 2u, 0);
  }
}
// LDS byte address of a __shared__ object
__device__ __forceinline__ uint32_t lds_addr(const void* p) { return (uint32_t)(uintptr_t)p; }

template <int MT, int NT, bool DENSE>
__device__ __forceinline__ void tile_mainloop(const TileSrc& s, int64_t m0, int64_t ntile0,
                                              int kt_begin, int kt_end, uint16_t* sA,
                                              const uint32_t* lut_lane, f32x4 (&acc)[MT][NT]) {
  const int tid = threadIdx.x, lane = tid & 63, lm = lane & 15, lq = lane >> 4;
  const int ktiles = (int)(s.K / KTILE);
  constexpr int kBufElems = MT * 16 * A_LD;
  constexpr uint32_t kBufBytes = kBufElems * 2;
  const u32x4 rx = raw_rsrc(s.x, (uint64_t)s.x_rows * s.K * 2);
  const uint32_t lds_a = lds_addr(sA);
  // this lane's fragment of row tile mt, k-step j: row l % 16, k-chunk 4 j + l / 16, swizzled
  auto frag = [&](const uint16_t* buf, int mt, int j) -> u32x4 {
    return *reinterpret_cast<const u32x4*>(reinterpret_cast<const unsigned char*>(buf) + mt * 4096 + lm * 256 +
                                           (((j * 4 + lq) ^ lm) * 16));
  };

  if constexpr (DENSE) {
    constexpr int PF = 2;  // weight k-tiles in flight
    const rsrc_t rw = make_rsrc(s.w_bf16, (uint64_t)s.ntiles * 16 * s.K * 2);
    u32x4 ring[PF][NT][4];
    auto load_w = [&](u32x4 (&dst)[NT][4], int kt) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        // tiles past the last column tile are redirected to offset ~0u: the buffer reads zeros
        const bool ok = (ntile0 + nt) < s.ntiles;
        const uint32_t row = (uint32_t)((ntile0 + nt) * 16 + lm);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          dst[nt][j] = buf_load128(
              rw, ok ? (row * (uint32_t)s.K + (uint32_t)(kt * KTILE + j * 32 + lq * 8)) * 2u : 0xfffffff0u);
      }
    };
    load_a<MT>(s, rx, m0, kt_begin, tid, lds_a);
#pragma unroll
    for (int d = 0; d < PF; ++d) load_w(ring[d], kt_begin + d);
    for (int kt0 = kt_begin; kt0 < kt_end; kt0 += PF) {
#pragma unroll
      for (int d = 0; d < PF; ++d) {
        const int kt = kt0 + d;
        const bool active = kt < kt_end;
        {
          const uint32_t par = (uint32_t)((kt - kt_begin) & 1);
          const uint16_t* buf = sA + par * kBufElems;
          u32x4 wf[NT][4];
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int j = 0; j < 4; ++j) wf[nt][j] = ring[d][nt][j];
          // this k-tile's activations have landed (the only younger loads: one ring stage of
          // weights); every wave is past its reads of the other buffer, which the next tile takes
          tnx_wait_vm(NT * 4);
          __syncthreads();
          load_a<MT>(s, rx, m0, kt + 1, tid, lds_a + (par ^ 1u) * kBufBytes);
          load_w(ring[d], kt + PF);
          if (active)
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              const u32x4 af = frag(buf, mt, j);
#pragma unroll
              for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = mfma16(af, wf[nt][j], acc[mt][nt]);
            }
        }
      }
    }
    tnx_wait_vm(0);   // the tile requested last is not used, but must not land in LDS the caller reuses
  } else {
    constexpr int PF = 2;  // weight k-tiles in flight
    const int spt = scales_per_tile(s.group);  // scale slots per tile and column (2 or 4)
    const uint64_t ntk = (uint64_t)s.ntiles * ktiles;
    const rsrc_t rc = make_rsrc(s.codes, ntk * 1024);
    const rsrc_t rs = make_rsrc(s.scales, ntk * 16 * spt * 2 + 16);
    u32x4 ring_c[PF][NT];
    u32x2 ring_s[PF][NT];  // up to four bf16 scales of this lane's column
    auto load_w = [&](u32x4 (&c)[NT], u32x2 (&sc)[NT], int kt) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        // 32-bit offsets: the host checks that codes and scales are below 4 GiB
        const uint32_t tile = (uint32_t)(ntile0 + nt) * (uint32_t)ktiles + (uint32_t)kt;
        c[nt] = buf_load128(rc, tile * 1024u + (uint32_t)lane * 16u);
        // always 8 bytes (the upper half is the next column when there are two slots): no
        // control flow around loads, so that the waits on them can be counted exactly
        sc[nt] = __builtin_amdgcn_raw_buffer_load_b64(rs, (tile * 16u + (uint32_t)lm) * (uint32_t)spt * 2u, 0, 0);
      }
    };
    if constexpr (MT == 1) {
      // One 16-row tile (a decode batch, the few rows an expert gets): every wave fetches the
      // activation fragments of its MFMAs itself, straight from global memory in fragment
      // layout (16 rows x 64 bytes per load, the four waves' requests meet in L1) -- no LDS
      // staging, no barrier in the loop, the waves drift apart and hide each other's waits.
      constexpr int PX = 3;
      const rsrc_t rx1 = make_rsrc(s.x, (uint64_t)s.x_rows * s.K * 2);
      int64_t src = m0 + lm;
      if (s.row_index) src = s.row_index[src < s.M ? src : s.M - 1] / s.row_div;   // gather; rows past M: a clamped row, never stored
      const uint32_t xoff = ((uint32_t)src * (uint32_t)s.K + (uint32_t)(lq * 8)) * 2u;   // rows past M (no gather) lie beyond the resource: zeros
      u32x4 xr[PX][4], rc3[PX][NT];
      u32x2 rs3[PX][NT];
      auto load_x = [&](u32x4 (&dst)[4], int kt) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          dst[j] = __builtin_amdgcn_raw_buffer_load_b128(rx1, xoff, (kt * KTILE + j * 32) * 2, 0);
      };
      const int kt_last = ktiles - 1;
#pragma unroll
      for (int d = 0; d < PX; ++d) {
        load_x(xr[d], min(kt_begin + d, kt_last));
        load_w(rc3[d], rs3[d], min(kt_begin + d, kt_last));
      }
      __syncthreads();  // the code-book table (built by the caller just before) is complete
      for (int kt0 = kt_begin; kt0 < kt_end; kt0 += PX) {
#pragma unroll
        for (int d = 0; d < PX; ++d) {
          const int kt = kt0 + d;
          const bool active = kt < kt_end;
          u32x4 cw[NT], xf[4];
          float sc[NT][4];
#pragma unroll
          for (int j = 0; j < 4; ++j) xf[j] = xr[d][j];
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            cw[nt] = rc3[d][nt];
            const u32x2 p = rs3[d][nt];
            float f[4] = {bflo(p[0]), bfhi(p[0]), bflo(p[1]), bfhi(p[1])};
#pragma unroll
            for (int j = 0; j < 4; ++j) sc[nt][j] = spt == 2 ? f[j >> 1] : f[j];
          }
          load_x(xr[d], min(kt + PX, kt_last));
          load_w(rc3[d], rs3[d], min(kt + PX, kt_last));
          if (active)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
              for (int nt = 0; nt < NT; ++nt)
                acc[0][nt] = mfma16(xf[j], dequant8_scaled(cw[nt][j], lut_lane, sc[nt][j]), acc[0][nt]);
            }
        }
      }
      return;
    }
    // Loads are never predicated (k-tiles past the end read unused neighbouring or zero data)
    // and the trip count is padded to a multiple of PF, so every wait is counted exactly.
    load_a<MT>(s, rx, m0, kt_begin, tid, lds_a);
#pragma unroll
    for (int d = 0; d < PF; ++d) load_w(ring_c[d], ring_s[d], kt_begin + d);
    for (int kt0 = kt_begin; kt0 < kt_end; kt0 += PF) {
#pragma unroll
      for (int d = 0; d < PF; ++d) {
        const int kt = kt0 + d;
        const bool active = kt < kt_end;
        {
          const uint32_t par = (uint32_t)((kt - kt_begin) & 1);
          const uint16_t* buf = sA + par * kBufElems;
          u32x4 cw[NT];
          float sc[NT][4];
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            cw[nt] = ring_c[d][nt];
            const u32x2 p = ring_s[d][nt];
            // scale of k-step j is scale number (j * spt) / 4 of the tile
            float f[4] = {bflo(p[0]), bfhi(p[0]), bflo(p[1]), bfhi(p[1])};
#pragma unroll
            for (int j = 0; j < 4; ++j) sc[nt][j] = spt == 2 ? f[j >> 1] : f[j];
          }
          // this k-tile's activations have landed (the only younger loads: one ring stage of
          // codes and scales); every wave is past its reads of the other buffer
          tnx_wait_vm(NT * 2);
          __syncthreads();
          // activations first, then the weights PF tiles ahead
          load_a<MT>(s, rx, m0, kt + 1, tid, lds_a + (par ^ 1u) * kBufBytes);
          load_w(ring_c[d], ring_s[d], kt + PF);
          if (active)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            u32x4 bf[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) bf[nt] = dequant8_scaled(cw[nt][j], lut_lane, sc[nt][j]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              const u32x4 af = frag(buf, mt, j);
#pragma unroll
              for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = mfma16(af, bf[nt], acc[mt][nt]);
            }
          }
        }
      }
    }
    tnx_wait_vm(0);   // the tile requested last is not used, but must not land in LDS the caller reuses
  }
}

// acc += lora_scale * t[:, toff[nt] : toff[nt]+r] . B ;  A fragments straight from global
// (t is a few tens of KiB and L2 resident).
template <int MT, int NT>
__device__ __forceinline__ void tile_lora(const TileSrc& s, int64_t m0, int64_t ntile0,
                                          const int (&toff)[NT], f32x4 (&acc)[MT][NT]) {
  const int lane = threadIdx.x & 63, lm = lane & 15, lq = lane >> 4;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    if (ntile0 + nt >= s.ntiles) continue;
    const int64_t col0 = (ntile0 + nt) * 16;
    f32x4 part[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) zero_acc(part[mt]);
    for (int j = 0; j < s.lora_rank / 32; ++j) {
      const u32x4 bfrag = *reinterpret_cast<const u32x4*>(s.lora_b + (col0 + lm) * s.lora_rank +
                                                          j * 32 + lq * 8);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int64_t row = m0 + mt * 16 + lm;
        u32x4 af = u32x4{0, 0, 0, 0};
        if (row < s.M)
          af = *reinterpret_cast<const u32x4*>(s.t + row * s.t_ld + toff[nt] + j * 32 + lq * 8);
        part[mt] = mfma16(af, bfrag, part[mt]);
      }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[mt][nt][i] += s.lora_scale * part[mt][i];
  }
}
