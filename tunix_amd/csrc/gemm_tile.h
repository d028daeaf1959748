// Shared main loop of the skinny GEMMs (quantized linears, MoE grouped GEMM, lm_head).
//
// A work-group of 4 waves owns 16*MT activation rows (MT = 8: a rollout batch of 128) and 64*NT output columns; wave w owns
// NT column tiles of 16.  The activation tile [16*MT x 128k] is staged in LDS once per k-tile
// and read as MFMA A fragments; weights go HBM -> registers (one 128-bit load per lane and
// k-tile for QW codes) and are expanded to bf16 through a bank-replicated LDS table.  Group
// scales multiply the fp32 partial sum of each group, so the bf16 MFMA operands are exact
// code-book values.
#pragma once
#include "common.h"

constexpr int KTILE = 128;
constexpr int A_LD = KTILE + 8;  // bf16 elements per LDS row (272 B)
constexpr size_t tile_smem_bytes(int mt) {
  return (size_t)mt * 16 * A_LD * sizeof(uint16_t) + TNX_LUT_WORDS * sizeof(uint32_t);
}

struct TileSrc {
  int64_t M, K;
  const uint16_t* x;         // bf16 [M,K] (or gathered through row_index)
  const int32_t* row_index;  // optional: LDS row r reads x row row_index[m0 + r] / row_div
  int row_div;
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

// Stage rows [m0, m0+16*MT) x k-tile kt of x into LDS (zero rows beyond M).
template <int MT>
__device__ __forceinline__ void stage_a(const TileSrc& s, int64_t m0, int kt, uint16_t* sA, int tid) {
#pragma unroll
  for (int c = 0; c < MT; ++c) {
    const int idx = tid + 256 * c;
    const int row = idx >> 4, ch = idx & 15;
    u32x4 v = u32x4{0, 0, 0, 0};
    if (m0 + row < s.M) {
      int64_t src = m0 + row;
      if (s.row_index) src = s.row_index[src] / s.row_div;
      v = *reinterpret_cast<const u32x4*>(s.x + src * s.K + (int64_t)kt * KTILE + ch * 8);
    }
    *reinterpret_cast<u32x4*>(sA + row * A_LD + ch * 8) = v;
  }
}

template <int MT, int NT, bool DENSE>
__device__ __forceinline__ void tile_mainloop(const TileSrc& s, int64_t m0, int64_t ntile0,
                                              int kt_begin, int kt_end, uint16_t* sA,
                                              const uint32_t* lut_lane, f32x4 (&acc)[MT][NT]) {
  const int tid = threadIdx.x, lane = tid & 63, lm = lane & 15, lq = lane >> 4;
  const int ktiles = (int)(s.K / KTILE);
  bool tile_ok[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) tile_ok[nt] = (ntile0 + nt) < s.ntiles;

  if constexpr (DENSE) {
    for (int kt = kt_begin; kt < kt_end; ++kt) {
      u32x4 wf[NT][4];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          wf[nt][j] = u32x4{0, 0, 0, 0};
          if (tile_ok[nt])
            wf[nt][j] = *reinterpret_cast<const u32x4*>(s.w_bf16 + ((ntile0 + nt) * 16 + lm) * s.K +
                                                        (int64_t)kt * KTILE + j * 32 + lq * 8);
        }
      __syncthreads();
      stage_a<MT>(s, m0, kt, sA, tid);
      __syncthreads();
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const u32x4 af =
              *reinterpret_cast<const u32x4*>(sA + (mt * 16 + lm) * A_LD + j * 32 + lq * 8);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = mfma16(af, wf[nt][j], acc[mt][nt]);
        }
    }
  } else {
    const int spt = s.group >= KTILE ? 1 : KTILE / s.group;  // scales per tile and column
    const int steps_per_scale = 4 / spt;                     // k-steps of 32 sharing a scale
    f32x4 part[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) zero_acc(part[mt][nt]);
    for (int kt = kt_begin; kt < kt_end; ++kt) {
      u32x4 cw[NT];
      uint16_t sc[NT][4];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        cw[nt] = u32x4{0, 0, 0, 0};
#pragma unroll
        for (int q = 0; q < 4; ++q) sc[nt][q] = 0;
        if (tile_ok[nt]) {
          const int64_t tile = (ntile0 + nt) * ktiles + kt;
          cw[nt] = *reinterpret_cast<const u32x4*>(s.codes + tile * 256 + lane * 4);
          const uint16_t* sp = s.scales + tile * (spt * 16) + lm;
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (q < spt) sc[nt][q] = sp[q * 16];
        }
      }
      __syncthreads();  // previous A tile fully consumed
      stage_a<MT>(s, m0, kt, sA, tid);
      __syncthreads();
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u32x4 bf[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) bf[nt] = dequant8(cw[nt][j], lut_lane);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const u32x4 af =
              *reinterpret_cast<const u32x4*>(sA + (mt * 16 + lm) * A_LD + j * 32 + lq * 8);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) part[mt][nt] = mfma16(af, bf[nt], part[mt][nt]);
        }
        if ((j + 1) % steps_per_scale == 0) {
          const int q = j / steps_per_scale;
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            const float scale = bf2f(sc[nt][q]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
              for (int i = 0; i < 4; ++i) acc[mt][nt][i] += scale * part[mt][nt][i];
              zero_acc(part[mt][nt]);
            }
          }
        }
      }
    }
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
