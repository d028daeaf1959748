// Measurement probe of bench.py, built into its own shared object (libtunix_probe.so): it is not
// part of the product library or of its C ABI.
#include "common.h"

namespace {

// Reads `bytes` once with the access pattern of the streaming kernels of this library (buffer
// loads of W = 16 or 8 bytes per lane, eight loads in flight per lane) and folds them into one
// word per work-group: a read of known size to scale hardware fetch counters with.
template <int W>
__global__ __launch_bounds__(256) void stream_read_kernel(const void* src, uint64_t bytes, uint32_t* sink) {
  const uint64_t per_wg = 256ull * W * 8ull;                     // bytes per work-group and turn
  uint32_t acc = 0;
  for (uint64_t base = (uint64_t)blockIdx.x * per_wg; base < bytes; base += (uint64_t)gridDim.x * per_wg) {
    const unsigned char* p = reinterpret_cast<const unsigned char*>(src) + base;
    const rsrc_t r = make_rsrc(p, bytes - base < per_wg ? bytes - base : per_wg);
    if constexpr (W == 16) {
      u32x4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = buf_load128(r, (uint32_t)((u * 256 + threadIdx.x) * 16));
#pragma unroll
      for (int u = 0; u < 8; ++u) acc ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
    } else {
      u32x2 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = __builtin_amdgcn_raw_buffer_load_b64(r, (uint32_t)((u * 256 + threadIdx.x) * 8), 0, 0);
#pragma unroll
      for (int u = 0; u < 8; ++u) acc ^= v[u][0] ^ v[u][1];
    }
  }
  acc ^= __shfl_xor(acc, 32, 64);
  if ((threadIdx.x & 63) == 0) atomicXor(sink + (blockIdx.x & 63), acc);
}

}  // namespace

// Reads `bytes` bytes at `src` exactly once with buffer loads of bytes_per_lane = 16 or 8 bytes per
// lane and xors them into sink64[0..63] (64 device words): a read of known size to run under a
// hardware fetch counter next to the kernels of interest.  Returns 0, or -1 for bad arguments or a
// failed launch.
extern "C" int tnx_probe_stream_read(void* stream, const void* src, uint64_t bytes, int bytes_per_lane,
                                     uint32_t* sink64) {
  if (!src || !sink64 || bytes == 0 || (bytes_per_lane != 16 && bytes_per_lane != 8)) return -1;
  const uint64_t turns = cdiv((int64_t)bytes, 256 * bytes_per_lane * 8);
  const unsigned wgs = (unsigned)(turns < 4096 ? turns : 4096);
  if (bytes_per_lane == 16)
    hipLaunchKernelGGL(stream_read_kernel<16>, dim3(wgs), dim3(256), 0, as_stream(stream), src, bytes, sink64);
  else
    hipLaunchKernelGGL(stream_read_kernel<8>, dim3(wgs), dim3(256), 0, as_stream(stream), src, bytes, sink64);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}
