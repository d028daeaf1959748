// jax.random's default bit stream on the device: threefry2x32, the two random_bits layouts and
// the Gumbel transform of jax.random.categorical.  Shared by the sampling kernels and the fused
// head's whole-vocabulary draw.
#pragma once
#include <stdint.h>

#include <hip/hip_runtime.h>

namespace {

__device__ __forceinline__ uint32_t rotl(uint32_t x, int r) { return (x << r) | (x >> (32 - r)); }

// Threefry-2x32, 20 rounds (Salmon et al. 2011), as used by jax.random's default PRNG.
__device__ __forceinline__ void threefry2x32(uint32_t k0, uint32_t k1, uint32_t& x0, uint32_t& x1) {
  const uint32_t ks[3] = {k0, k1, k0 ^ k1 ^ 0x1BD11BDAu};
  const int rot[8] = {13, 15, 26, 6, 17, 29, 16, 24};
  x0 += ks[0];
  x1 += ks[1];
#pragma unroll
  for (int g = 0; g < 5; ++g) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      x0 += x1;
      x1 = rotl(x1, rot[(g & 1) * 4 + r]);
      x1 ^= x0;
    }
    x0 += ks[(g + 1) % 3];
    x1 += ks[(g + 2) % 3] + (uint32_t)(g + 1);
  }
}

// 32 random bits of element n of an array of `total` elements.
//   variant 1: counters (0, n), output x0 ^ x1       (jax_threefry_partitionable = True)
//   variant 0: the array of counters is split in two halves (first half -> x0, second -> x1)
__device__ __forceinline__ uint32_t random_bits(uint32_t k0, uint32_t k1, uint64_t n, uint64_t total,
                                                int variant) {
  if (variant == 1) {
    uint32_t x0 = (uint32_t)(n >> 32), x1 = (uint32_t)n;
    threefry2x32(k0, k1, x0, x1);
    return x0 ^ x1;
  }
  const uint64_t half = (total + 1) / 2;
  const uint64_t i = n < half ? n : n - half;
  uint32_t x0 = (uint32_t)i;
  uint32_t x1 = (i + half < total) ? (uint32_t)(i + half) : 0u;
  threefry2x32(k0, k1, x0, x1);
  return n < half ? x0 : x1;
}

// jax.random.gumbel: -log(-log(uniform(minval=tiny, maxval=1)))
__device__ __forceinline__ float gumbel_from_bits(uint32_t bits) {
  const float tiny = 1.17549435e-38f;
  float u = __uint_as_float((bits >> 9) | 0x3f800000u) - 1.0f;
  u = fmaxf(tiny, u * (1.0f - tiny) + tiny);
  return -logf(-logf(u));
}

}  // namespace
