// Pieces shared by the decode GEMV kernels: scheme traits, kernel parameters and the
// per-group fused unpack + dot product.
#pragma once

#include "gq_common.hpp"
#include "gq_internal.hpp"

namespace gq {

template <int BITS>
struct GemvTraits;
template <>
struct GemvTraits<4> {
  static constexpr int G = 32;   // values per group
  static constexpr int CH = 4;   // 16-byte x chunks per group (8 halves each)
};
template <>
struct GemvTraits<3> {
  static constexpr int G = 40;
  static constexpr int CH = 5;
};

struct GemvParams {
  const uint16_t* x;
  const uint32_t* qw;
  const uint16_t* qs;
  const uint16_t* bias;
  void* y;
  const int32_t* expert_ids;
  int64_t x_slot_stride;
  int64_t expert_w_stride;  // N * nw
  int64_t expert_s_stride;  // N * ng
  int N, K, ng, nw;
  int num_experts;
  int gc;  // groups staged per LDS chunk (multiple of 64)
  int out_f32;
};

// sum_k x_k * (field_k - m) for one group, given the 4 storage words and the staged x pairs
template <int BITS>
__device__ __forceinline__ float group_dot(const uint4 w4, const uint32_t* __restrict__ xr,
                                           float corr) {
  const uint32_t w[4] = {w4.x, w4.y, w4.z, w4.w};
  constexpr uint32_t kMagic = 0x64006400u;
  if (BITS == 4) {
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t w8 = w[i] >> 8;
      lo = dot2(and_or(w[i], 0x000f000fu, kMagic), xr[4 * i + 0], lo);
      hi = dot2(and_or(w[i], 0x00f000f0u, kMagic), xr[4 * i + 1], hi);
      lo = dot2(and_or(w8, 0x000f000fu, kMagic), xr[4 * i + 2], lo);
      hi = dot2(and_or(w8, 0x00f000f0u, kMagic), xr[4 * i + 3], hi);
    }
    return fmaf(hi, 0.0625f, lo) - corr;
  } else {
    float a1 = 0.f, a8 = 0.f, a64 = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // low half keeps fields 0-4, high half gets fields 5-9 aligned to bit 16
      const uint32_t t = (w[i] & 0x0000ffffu) | ((w[i] << 1) & 0xffff0000u);
      const uint32_t t9 = t >> 9;
      a1 = dot2(and_or(t, 0x00070007u, kMagic), xr[5 * i + 0], a1);
      a8 = dot2(and_or(t, 0x00380038u, kMagic), xr[5 * i + 1], a8);
      a64 = dot2(and_or(t, 0x01c001c0u, kMagic), xr[5 * i + 2], a64);
      a1 = dot2(and_or(t9, 0x00070007u, kMagic), xr[5 * i + 3], a1);
      a8 = dot2(and_or(t9, 0x00380038u, kMagic), xr[5 * i + 4], a8);
    }
    return fmaf(a64, 0.015625f, fmaf(a8, 0.125f, a1)) - corr;
  }
}


// launchers of the kernel families (each in its own translation unit)
hipError_t launch_gemv_lds(const GemvParams& p, int bits, int nb, int slots, hipStream_t s);
// register-resident x, persistent waves; returns hipErrorNotSupported when the shape does not fit
hipError_t launch_gemv_reg(const GemvParams& p, int bits, int nb, int slots, hipStream_t s);

}  // namespace gq
