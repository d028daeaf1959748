// Shared device helpers for the gfx950 kernels of libtunix_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "tunix_hip.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define TNX_WAVE 64

// ---- error plumbing (host) -------------------------------------------------------------
void tnx_set_error(const char* fmt, ...);
#define TNX_REQUIRE(cond, ...)      \
  do {                              \
    if (!(cond)) {                  \
      tnx_set_error(__VA_ARGS__);   \
      return TNX_EINVAL;            \
    }                               \
  } while (0)
#define TNX_CHECK_LAUNCH(name)                                                  \
  do {                                                                          \
    hipError_t e_ = hipGetLastError();                                          \
    if (e_ != hipSuccess) {                                                     \
      tnx_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));      \
      return TNX_ELAUNCH;                                                       \
    }                                                                           \
  } while (0)

// ---- bf16 <-> f32 ----------------------------------------------------------------------
__device__ __forceinline__ float bf2f(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
__device__ __forceinline__ uint16_t f2bf(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);  // round-to-nearest-even (v_cvt_pk_bf16_f32)
}
__device__ __forceinline__ float rbf(float f) { return bf2f(f2bf(f)); }
__device__ __forceinline__ uint32_t pack2bf(float lo, float hi) {
  return (uint32_t)f2bf(lo) | ((uint32_t)f2bf(hi) << 16);
}
__device__ __forceinline__ float bflo(uint32_t p) { return __uint_as_float(p << 16); }
__device__ __forceinline__ float bfhi(uint32_t p) { return __uint_as_float(p & 0xffff0000u); }

__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
  // D[16x16] += A[16x32] * B[32x16]; lane l holds A row l%16 / B column l%16, k = 8*(l/16)..+7;
  // D: column l%16, rows 4*(l/16)..+3.
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                 __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// ---- code books ------------------------------------------------------------------------
// The 16 NF4 levels of QLoRA (Dettmers et al. 2023), fp32.
__device__ __constant__ const float kNf4Levels[16] = {
    -1.0f,        -0.6961928f,  -0.52507305f, -0.39491749f, -0.28444138f, -0.18477343f,
    -0.09105004f, 0.0f,         0.0795803f,   0.1609302f,   0.2461123f,   0.33791524f,
    0.44070983f,  0.562617f,    0.72295684f,  1.0f};

__device__ __forceinline__ float code_level(int qtype, int code) {
  return qtype == TNX_Q_NF4 ? kNf4Levels[code] : (float)(code - 8);
}
// The same value from literals (a select tree over the code's bits): no memory access, for
// kernels whose first instructions would otherwise wait on the table.
__device__ __forceinline__ float code_level_imm(int qtype, int code) {
  const bool b0 = code & 1, b1 = code & 2, b2 = code & 4, b3 = code & 8;
  const float p0 = b0 ? -0.6961928f : -1.0f, p1 = b0 ? -0.39491749f : -0.52507305f;
  const float p2 = b0 ? -0.18477343f : -0.28444138f, p3 = b0 ? 0.0f : -0.09105004f;
  const float p4 = b0 ? 0.1609302f : 0.0795803f, p5 = b0 ? 0.33791524f : 0.2461123f;
  const float p6 = b0 ? 0.562617f : 0.44070983f, p7 = b0 ? 1.0f : 0.72295684f;
  const float q0 = b1 ? p1 : p0, q1 = b1 ? p3 : p2, q2 = b1 ? p5 : p4, q3 = b1 ? p7 : p6;
  const float r0 = b2 ? q1 : q0, r1 = b2 ? q3 : q2;
  const float nf4 = b3 ? r1 : r0;
  return qtype == TNX_Q_NF4 ? nf4 : (float)(code - 8);
}

// Scales stored per (k-tile of 128, column): S = max(2, 128 / group) slots of 128 / S k each
// (a group of 128 or more repeats its scale), so that a lane's scales are one aligned 4- or 8-byte word.
__host__ __device__ inline int scales_per_tile(int group) { return group >= 64 ? 2 : 128 / group; }

// LDS look-up table: byte (two codes) -> two levels as an f16 pair (every bf16-rounded level is
// exact in f16, and v_fma_mix_f32 converts the half it selects and multiplies it with the fp32
// scale in one instruction), replicated so that lane l reads entry [byte][l % 32] and every
// lane of a half-wave hits its own bank.
#define TNX_LUT_COPIES 32
#define TNX_LUT_WORDS (256 * TNX_LUT_COPIES)
__device__ __forceinline__ void build_lut(uint32_t* lut, int qtype, int tid, int nthreads) {
  // thread `byte` looks its two levels up once and writes all copies of its entry
  for (int byte = tid; byte < 256; byte += nthreads) {
    typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
    const f16x2_t hv = {(_Float16)rbf(code_level(qtype, byte & 15)), (_Float16)rbf(code_level(qtype, byte >> 4))};
    const uint32_t v = __builtin_bit_cast(uint32_t, hv);
#pragma unroll
    for (int c = 0; c < TNX_LUT_COPIES; ++c)  // rotated so that the lanes hit different banks
      lut[byte * TNX_LUT_COPIES + ((c + tid) & (TNX_LUT_COPIES - 1))] = v;
  }
}
// The integer code book without a table.  A code byte is (k even | k odd << 4) and a dword holds
// a lane's four code bytes of one k-step.  Masked into the mantissa of an f16 whose exponent makes
// one mantissa step worth exactly one level -- 0x6400 (1024, step 1) for a nibble at bit 0, 0x5400
// (64, step 1/16) for a nibble at bit 4 -- the nibbles of bytes 0 and 2 become an f16 pair
// (1024 + n | 1024 + n) or (64 + n | 64 + n) with one v_and_or_b32, those of bytes 1 and 3 after
// one shift by 8, and one packed f16 add of -1032 or -72 leaves the exact levels n - 8.  Entry j
// of a dword is then: 0 = the even k of bytes 0 | 2, 1 = the odd k of bytes 0 | 2, 2 / 3 = the
// same of bytes 1 | 3; the pair of byte b is half b / 2 of entries 2 (b % 2) and 2 (b % 2) + 1.
// One VALU instruction more per pair than the table path, and no LDS instruction.
struct Int4Magic {
  uint32_t mask_lo = 0x000f000fu, mask_hi = 0x00f000f0u, magic_lo = 0x64006400u, magic_hi = 0x54005400u;
  uint32_t bias_lo = 0xe408e408u, bias_hi = 0xd480d480u;   // f16 pairs (-1032 | -1032), (-72 | -72)
  // Kept in registers as opaque values, so that the compiler forms v_and_or_b32 (which takes no
  // literal and only one scalar operand): the exponents in vector registers; masks and biases in
  // scalar registers, or in vector registers too for a kernel that has no scalar registers left
  // (out of them, the compiler parks loop-carried scalars in vector registers and then hands
  // one to an assembly operand that must be scalar).
  template <bool VEC>
  __device__ __forceinline__ void pin() {
    asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));
    if constexpr (VEC) asm volatile("" : "+v"(mask_lo), "+v"(mask_hi), "+v"(bias_lo), "+v"(bias_hi));
    else asm volatile("" : "+s"(mask_lo), "+s"(mask_hi), "+s"(bias_lo), "+s"(bias_hi));
  }
};
// entry j with the offsets still on: 1024 + n (even j) or 64 + n (odd j) in both halves.  A kernel
// with registers to spare multiplies these with the scale s and adds -1032 s or -72 s in the same
// fused multiply-add (exact: the sum (n - 8) s has at most 12 significant bits) and saves the
// packed add.
__device__ __forceinline__ uint32_t int4_entry_offset(const Int4Magic& m, uint32_t w, int j) {
  const uint32_t src = j < 2 ? w : w >> 8;
  return (j & 1) ? ((src & m.mask_hi) | m.magic_hi) : ((src & m.mask_lo) | m.magic_lo);
}
__device__ __forceinline__ uint32_t int4_entry(const Int4Magic& m, uint32_t w, int j) {
  typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
  const uint32_t v = int4_entry_offset(m, w, j);
  const f16x2_t sum = __builtin_bit_cast(f16x2_t, v) + __builtin_bit_cast(f16x2_t, (j & 1) ? m.bias_hi : m.bias_lo);
  return __builtin_bit_cast(uint32_t, sum);
}
// the two levels of code byte b, as f16: from a dword's four entries above (INT4) or from the
// table's four entries, one per byte
template <bool INT4>
__device__ __forceinline__ void level_pair(const uint32_t (&e)[4], int b, _Float16& l0, _Float16& l1) {
  typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
  if constexpr (INT4) {
    l0 = __builtin_bit_cast(f16x2_t, e[2 * (b & 1)])[b >> 1];
    l1 = __builtin_bit_cast(f16x2_t, e[2 * (b & 1) + 1])[b >> 1];
  } else {
    const f16x2_t h = __builtin_bit_cast(f16x2_t, e[b]);
    l0 = h[0];
    l1 = h[1];
  }
}
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t cvt_pk_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}
// Eight codes -> eight bf16 weights bf16(bf16(level) * scale): the B fragment of one k-step.
__device__ __forceinline__ u32x4 dequant8_scaled(uint32_t w, const uint32_t* lut_lane, float scale) {
  u32x4 r;
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
    const f16x2_t h = __builtin_bit_cast(f16x2_t, lut_lane[((w >> (8 * b)) & 0xffu) * TNX_LUT_COPIES]);
    r[b] = cvt_pk_bf16(__builtin_fmaf((float)h[0], scale, 0.0f), __builtin_fmaf((float)h[1], scale, 0.0f));
  }
  return r;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

static inline hipStream_t as_stream(void* s) { return (hipStream_t)s; }
static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Raw buffer resources: 32-bit byte offsets, and loads whose vector offset (plus the
// immediate) lies past the size return zeros instead of faulting.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* p, uint64_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0,
                                           (uint32_t)(bytes > 0xffffffffull ? 0xffffffffull : bytes),
                                           0x00020000);
}
// Cache policy of buffer accesses whose data is used exactly once and by one wave (the keys and
// values of attention; the fp32 partial planes a split-k GEMM leaves for the next kernel):
// non-temporal.  A flat read of this part runs at 7.1-7.3 TB/s with it against 6.2-6.4 TB/s
// without; attention over cold caches 6.0 against 5.4 TB/s at context 768.  (Measured and not
// adopted for the packed weights of the GEMM, 1 us slower per launch, for the head's weight rows,
// neutral, and for the norm's reads of the partial planes, slower.)
constexpr int kStreamOnce = 2;   // the "nt" bit of the gfx940+ cache-policy operand
__device__ __forceinline__ u32x4 buf_load128(rsrc_t r, uint32_t byte_off) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 0);
}
