// Measurement aid: a plain streaming read with no arithmetic to speak of, so that a benchmark
// can quote, from the same process and minutes, what this GPU delivers for the bytes a GEMV
// streams.  Not on the product path and without a counterpart in the reference.
#include "gq_common.hpp"
#include "gq_internal.hpp"

namespace gq {

// 2048 persistent waves.  A range is walked in tiles of 4 rows x 2 KiB: each 16-lane quarter of
// a wave streams its own row, 256 contiguous bytes per instruction, all eight instructions of
// the tile in flight (of the shapes tried, 1 x 1 KiB to 32 x 32 B per instruction, this one
// read fastest).  The xor of everything read is kept alive by a store that practically never
// happens.
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* __restrict__ a, int64_t na,
                                                          const uint4* __restrict__ b, int64_t nb,
                                                          uint32_t* sink) {
  const int lane = threadIdx.x & 63;
  const int64_t gw = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t nw = static_cast<int64_t>(gridDim.x) * 4;
  uint32_t acc = 0;
  for (int pass = 0; pass < 2; ++pass) {
    const uint4* src = pass == 0 ? a : b;
    const int64_t n = pass == 0 ? na : nb;
    const int64_t tiles = n / 512;  // 512 uint4 = 4 rows of 128
    for (int64_t t = gw; t < tiles; t += nw) {
      const uint4* p = src + t * 512 + (lane >> 4) * 128 + (lane & 15);
      uint4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = p[16 * u];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (int64_t i = tiles * 512 + gw * 64 + lane; i < n; i += nw * 64) {  // what is left of the range
      const uint4 v = src[i];
      acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
  }
  if (acc == 0x9e3779b9u && sink != nullptr) sink[0] = acc;
}

hipError_t launch_stream_read(const void* a, int64_t a_bytes, const void* b, int64_t b_bytes,
                              void* sink, hipStream_t s) {
  hipLaunchKernelGGL(stream_read_kernel, dim3(512), dim3(256), 0, s, static_cast<const uint4*>(a),
                     a_bytes / 16, static_cast<const uint4*>(b), b_bytes / 16,
                     static_cast<uint32_t*>(sink));
  return hipGetLastError();
}

}  // namespace gq
