// quantize_weight / dequantize / embedding-take kernels (HBM-bound streaming, bit-exact).
//
// Replaces the TE definitions of the reference:
//   python/mlc_llm/quantization/group_quantization.py:235-306 (_quantize), :155-186 (_dequantize)
//   python/mlc_llm/quantization/utils.py:15-48 (convert_uint_to_float), :136-188 (pack_weight)
//   python/mlc_llm/compiler_pass/fuse_dequantize_take.py:14-49 (dequantize fused into take)
//
// One thread owns one uint32 storage word (8 or 10 values); the four threads of a lane quad own
// one quantisation group (both schemes store a group in 4 words), so the group max is two DPP
// steps and all global traffic is coalesced word-by-word.
#include "gq_common.hpp"
#include "gq_internal.hpp"

namespace gq {

template <int BITS>
__global__ __launch_bounds__(256) void quantize_kernel(const uint16_t* __restrict__ w,
                                                       int64_t rows, int64_t K, int64_t nw,
                                                       int64_t ng, int group_size, int half_even,
                                                       uint32_t* __restrict__ qw,
                                                       uint16_t* __restrict__ qs) {
  using S = Scheme<BITS>;
  constexpr int E = S::kElem;
  const int64_t total = rows * nw;
  int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  // quads never straddle rows (nw % 4 == 0); inactive lanes still take part in the shuffles
  const bool live = idx < total;
  if (!live) idx = total - 1;
  const int64_t row = idx / nw;
  const int64_t wd = idx - row * nw;
  const int64_t g = wd >> 2;
  const int64_t k0 = g * group_size + (wd & 3) * E;
  const uint16_t* wr = w + row * K;

  float v[E];
  bool ok[E];
  const bool full = (k0 + E <= K);
  if (BITS == 4 && full && ((K & 7) == 0)) {
    const uint4 raw = *reinterpret_cast<const uint4*>(wr + k0);
    const uint32_t r4[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = h2f(static_cast<uint16_t>(r4[i] & 0xffffu));
      v[2 * i + 1] = h2f(static_cast<uint16_t>(r4[i] >> 16));
      ok[2 * i] = ok[2 * i + 1] = true;
    }
  } else if (BITS == 3 && full && ((K & 1) == 0)) {
    const uint32_t* p = reinterpret_cast<const uint32_t*>(wr + k0);
#pragma unroll
    for (int i = 0; i < E / 2; ++i) {
      const uint32_t r = p[i];
      v[2 * i] = h2f(static_cast<uint16_t>(r & 0xffffu));
      v[2 * i + 1] = h2f(static_cast<uint16_t>(r >> 16));
      ok[2 * i] = ok[2 * i + 1] = true;
    }
  } else {
#pragma unroll
    for (int i = 0; i < E; ++i) {
      ok[i] = (k0 + i) < K;
      v[i] = ok[i] ? h2f(wr[k0 + i]) : 0.0f;
    }
  }

  // group max of |w|; lanes beyond K contribute fp16 lowest, as the reference pads
  float amax = -65504.0f;
#pragma unroll
  for (int i = 0; i < E; ++i) {
    const float a = fabsf(v[i]);
    amax = (ok[i] && a > amax) ? a : amax;
  }
  amax = fmaxf(amax, dpp_f<0xB1>(amax));
  amax = fmaxf(amax, dpp_f<0x4E>(amax));

  const float m = static_cast<float>(S::kMaxInt);
  const uint16_t sh = f2h(amax / m);  // fp16 divide: float divide, one rounding to half
  const float s = h2f(sh);
  // v / s for the E values of this word.  The fp16 quotient of two halves is the float quotient
  // rounded once more; a float quotient within half an ulp (plus a hair) rounds to the same half,
  // because a ratio of two 11-bit significands that is not itself a rounding boundary of fp16
  // stays more than 2^-23 (relative) away from one.  One Newton step on the hardware reciprocal
  // gives that accuracy for a third of the instructions of a correctly rounded divide.  s = 0
  // (an all-zero or denormal-only group) and overflowing quotients keep the first product, which
  // is the NaN / infinity the plain divide yields.
  const float rs = __builtin_amdgcn_rcpf(s);
  uint32_t word = 0;
#pragma unroll
  for (int i = 0; i < E; ++i) {
    const float q0 = v[i] * rs;
    const float q1 = fmaf(fmaf(-q0, s, v[i]), rs, q0);
    const float quo = (s == 0.0f || fabsf(q0) == __builtin_inff()) ? q0 : q1;
    float t = h2f(f2h(quo));  // fp16 divide
    t = h2f(f2h(t + m));           // fp16 add
    float r = half_even ? rintf(t) : roundf(t);
    r = (r > 0.0f) ? r : 0.0f;  // compare+select max: NaN (0/0) becomes 0
    r = (r < 2.0f * m) ? r : 2.0f * m;
    const uint32_t q = ok[i] ? static_cast<uint32_t>(r) : 0u;
    word |= q << (i * BITS);
  }
  if (live) {
    qw[idx] = word;
    if ((wd & 3) == 0) qs[row * ng + g] = sh;
  }
}

// out[orow, k] = (unpack(qw[row, k]) - m) * qs[row, k / G] for k < K; row = ids ? ids[orow] : orow
template <int BITS>
__global__ __launch_bounds__(256) void dequantize_kernel(const int32_t* __restrict__ ids,
                                                         int64_t out_rows,
                                                         const uint32_t* __restrict__ qw,
                                                         const uint16_t* __restrict__ qs,
                                                         int64_t table_rows, int64_t K, int64_t nw,
                                                         int64_t ng, uint16_t* __restrict__ out) {
  using S = Scheme<BITS>;
  constexpr int E = S::kElem;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= out_rows * nw) return;
  const int64_t orow = idx / nw;
  const int64_t wd = idx - orow * nw;
  int64_t row = orow;
  if (ids != nullptr) {
    row = ids[orow];
    row = row < 0 ? 0 : (row >= table_rows ? table_rows - 1 : row);
  }
  const int64_t k0 = wd * E;
  if (k0 >= K) return;
  const uint32_t word = qw[row * nw + wd];
  const float s = h2f(qs[row * ng + (wd >> 2)]);
  uint16_t o[E];
#pragma unroll
  for (int i = 0; i < E; ++i) {
    const int u = static_cast<int>((word >> (i * BITS)) & S::kMask);
    // (u - m) is exact; the product of two halves is exact in float, so this is one rounding
    o[i] = f2h(static_cast<float>(u - S::kMaxInt) * s);
  }
  uint16_t* dst = out + orow * K + k0;
  if (BITS == 4 && k0 + E <= K && ((K & 7) == 0)) {
    uint4 pk;
    pk.x = o[0] | (static_cast<uint32_t>(o[1]) << 16);
    pk.y = o[2] | (static_cast<uint32_t>(o[3]) << 16);
    pk.z = o[4] | (static_cast<uint32_t>(o[5]) << 16);
    pk.w = o[6] | (static_cast<uint32_t>(o[7]) << 16);
    *reinterpret_cast<uint4*>(dst) = pk;
  } else if (BITS == 3 && k0 + E <= K && ((K & 1) == 0)) {
    uint32_t* d32 = reinterpret_cast<uint32_t*>(dst);
#pragma unroll
    for (int i = 0; i < E / 2; ++i) d32[i] = o[2 * i] | (static_cast<uint32_t>(o[2 * i + 1]) << 16);
  } else {
#pragma unroll
    for (int i = 0; i < E; ++i)
      if (k0 + i < K) dst[i] = o[i];
  }
}

hipError_t launch_quantize(const uint16_t* w, int64_t rows, int64_t K, int bits, int group_size,
                           int round_mode, uint32_t* qw, uint16_t* qs, hipStream_t s) {
  const int64_t ng = (K + group_size - 1) / group_size;
  const int64_t nw = 4 * ng;
  const int64_t total = rows * nw;
  if (total == 0) return hipSuccess;
  const dim3 grid(static_cast<unsigned>((total + 255) / 256));
  if (bits == 4)
    hipLaunchKernelGGL(quantize_kernel<4>, grid, dim3(256), 0, s, w, rows, K, nw, ng, group_size,
                       round_mode, qw, qs);
  else
    hipLaunchKernelGGL(quantize_kernel<3>, grid, dim3(256), 0, s, w, rows, K, nw, ng, group_size,
                       round_mode, qw, qs);
  return hipGetLastError();
}

hipError_t launch_dequantize(const int32_t* ids, int64_t out_rows, const uint32_t* qw,
                             const uint16_t* qs, int64_t table_rows, int64_t K, int bits,
                             int group_size, uint16_t* out, hipStream_t s) {
  const int64_t ng = (K + group_size - 1) / group_size;
  const int64_t nw = 4 * ng;
  const int64_t total = out_rows * nw;
  if (total == 0) return hipSuccess;
  const dim3 grid(static_cast<unsigned>((total + 255) / 256));
  if (bits == 4)
    hipLaunchKernelGGL(dequantize_kernel<4>, grid, dim3(256), 0, s, ids, out_rows, qw, qs,
                       table_rows, K, nw, ng, out);
  else
    hipLaunchKernelGGL(dequantize_kernel<3>, grid, dim3(256), 0, s, ids, out_rows, qw, qs,
                       table_rows, K, nw, ng, out);
  return hipGetLastError();
}

}  // namespace gq
