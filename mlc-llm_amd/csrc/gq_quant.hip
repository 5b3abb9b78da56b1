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
#include "gq_quant_common.hpp"

namespace gq {

// HALF_EVEN: the tie rule of the rounding (0: half away from zero, the llvm / rocm lowering of
// tirx.round; 1: half to even, what CUDA-converted weights carry).
template <int BITS, int HALF_EVEN>
__global__ __launch_bounds__(256) void quantize_kernel(const uint16_t* __restrict__ w,
                                                       int64_t rows, int64_t K, int64_t nw,
                                                       int64_t ng, int group_size, WordGrid gr,
                                                       uint32_t* __restrict__ qw,
                                                       uint16_t* __restrict__ qs) {
  using S = Scheme<BITS>;
  constexpr int E = S::kElem;
  constexpr int P = E / 2;  // half pairs per storage word
  int64_t row, wd;
  locate_word(gr, nw, row, wd);
  // inactive lanes (whole quads past the last row) still take part in the shuffles
  const bool live = row < rows;
  if (!live) { row = rows - 1; wd = nw - 1; }
  const int64_t g = wd >> 2;
  const int64_t k0 = g * group_size + (wd & 3) * E;
  const uint16_t* wr = w + row * K;

  // ---- the word's E values as half pairs; slots beyond K hold zero and are masked out of the
  //      maximum (the reference pads with fp16 lowest) and of the packed word
  uint32_t pr[P];
  const bool full = (k0 + E <= K);
  if (BITS == 4 && full && ((K & 7) == 0)) {
    const uint4 raw = *reinterpret_cast<const uint4*>(wr + k0);
    pr[0] = raw.x; pr[1] = raw.y; pr[2] = raw.z; pr[3] = raw.w;
  } else if (full && ((K & 1) == 0)) {
    const uint32_t* p = reinterpret_cast<const uint32_t*>(wr + k0);
#pragma unroll
    for (int i = 0; i < P; ++i) pr[i] = p[i];
  } else {
#pragma unroll
    for (int i = 0; i < P; ++i) {
      const uint32_t lo = (k0 + 2 * i) < K ? wr[k0 + 2 * i] : 0u;
      const uint32_t hi = (k0 + 2 * i + 1) < K ? wr[k0 + 2 * i + 1] : 0u;
      pr[i] = lo | (hi << 16);
    }
  }
  const int valid = full ? E : static_cast<int>(K > k0 ? K - k0 : 0);  // values of this word inside K

  // ---- group max of |w| (packed fp16 maxima ignore NaN operands, as the reference's
  //      compare-and-select does); zero padding cannot raise a maximum of absolute values
  half2_t mx = as_half2(pr[0] & 0x7fff7fffu);
#pragma unroll
  for (int i = 1; i < P; ++i) mx = __builtin_elementwise_max(mx, as_half2(pr[i] & 0x7fff7fffu));
  float amax = fmaxf(static_cast<float>(mx[0]), static_cast<float>(mx[1]));
  if (valid == 0) amax = -65504.0f;
  amax = fmaxf(amax, dpp_f<0xB1>(amax));
  amax = fmaxf(amax, dpp_f<0x4E>(amax));

  const float m = static_cast<float>(S::kMaxInt);
  const uint16_t sh = f2h(amax / m);  // fp16 divide: float divide, one rounding to half
  const float s = h2f(sh);
  // v / s for the E values of this word.  The fp16 quotient of two halves is the float quotient
  // rounded once more; a float quotient within half an ulp (plus a hair) rounds to the same half,
  // because a ratio of two 11-bit significands that is not itself a rounding boundary of fp16
  // stays more than 2^-23 (relative) away from one.  One Newton step on the hardware reciprocal
  // gives that accuracy for a third of the instructions of a correctly rounded divide.  A scale
  // that is zero (an all-zero group), infinite or NaN keeps the first product, which is then the
  // NaN / zero / NaN the plain divide yields.
  const float rs = __builtin_amdgcn_rcpf(s);
  const bool plain = !(s > 0.0f && s < __builtin_inff());
  // Everything after the divide is fp16 arithmetic on pairs: the add of m (rounded), then the
  // rounding to an integer.  t = quotient + m lies in [-0.004, 2m], so t + 0.5 is exact and its
  // truncation is round-half-away; (t + 1024) - 1024 is round-half-even (fp16 spacing is 1 there).
  // A NaN (0 / 0) becomes 0 in the packed maximum, like the reference's compare-and-select.
  const _Float16 hm = static_cast<_Float16>(m);
  const half2_t m2 = {hm, hm};
  const half2_t zero2 = {static_cast<_Float16>(0.0f), static_cast<_Float16>(0.0f)};
  const half2_t top2 = {static_cast<_Float16>(2.0f * m + 0.5f), static_cast<_Float16>(2.0f * m + 0.5f)};
  uint32_t word = 0;
  uint16_t qv[E];
#pragma unroll
  for (int i = 0; i < P; ++i) {
    const half2_t hv = as_half2(pr[i]);
    float quo[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const float v = static_cast<float>(hv[e]);
      const float q0 = v * rs;
      const float q1 = fmaf(fmaf(-q0, s, v), rs, q0);
      quo[e] = plain ? q0 : q1;
    }
    const half2_t qh = {static_cast<_Float16>(quo[0]), static_cast<_Float16>(quo[1])};  // fp16 divide
    const half2_t t = qh + m2;                                                            // fp16 add
    half2_t r;
    if (HALF_EVEN) {
      const half2_t big = {static_cast<_Float16>(1024.0f), static_cast<_Float16>(1024.0f)};
      r = (t + big) - big;
    } else {
      const half2_t hf = {static_cast<_Float16>(0.5f), static_cast<_Float16>(0.5f)};
      r = t + hf;  // truncated by the conversion below
    }
    r = __builtin_elementwise_min(__builtin_elementwise_max(r, zero2), top2);  // [0, 2m] and no NaN left
    qv[2 * i] = static_cast<uint16_t>(r[0]);  // truncation; the operand is in [0, 2m + 0.5]
    qv[2 * i + 1] = static_cast<uint16_t>(r[1]);
  }
  if (full) {
#pragma unroll
    for (int i = 0; i < E; ++i) word |= static_cast<uint32_t>(qv[i]) << (i * BITS);
  } else {  // a word that straddles K (the last group of a row): slots beyond K stay zero
#pragma unroll
    for (int i = 0; i < E; ++i) word |= (i < valid ? static_cast<uint32_t>(qv[i]) : 0u) << (i * BITS);
  }
  if (live) {
    qw[row * nw + wd] = word;
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
                                                         int64_t ng, WordGrid gr,
                                                         uint16_t* __restrict__ out) {
  using S = Scheme<BITS>;
  constexpr int E = S::kElem;
  int64_t orow, wd;
  locate_word(gr, nw, orow, wd);
  if (orow >= out_rows) return;
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
  unsigned blocks = 0;
  const WordGrid gr = plan_words(rows, nw, blocks);
  if (blocks == 0) return hipErrorInvalidValue;
  const dim3 grid(blocks);
  if (bits == 4 && round_mode == 0)
    hipLaunchKernelGGL((quantize_kernel<4, 0>), grid, dim3(256), 0, s, w, rows, K, nw, ng, group_size, gr, qw, qs);
  else if (bits == 4)
    hipLaunchKernelGGL((quantize_kernel<4, 1>), grid, dim3(256), 0, s, w, rows, K, nw, ng, group_size, gr, qw, qs);
  else if (round_mode == 0)
    hipLaunchKernelGGL((quantize_kernel<3, 0>), grid, dim3(256), 0, s, w, rows, K, nw, ng, group_size, gr, qw, qs);
  else
    hipLaunchKernelGGL((quantize_kernel<3, 1>), grid, dim3(256), 0, s, w, rows, K, nw, ng, group_size, gr, qw, qs);
  return hipGetLastError();
}

hipError_t launch_dequantize(const int32_t* ids, int64_t out_rows, const uint32_t* qw,
                             const uint16_t* qs, int64_t table_rows, int64_t K, int bits,
                             int group_size, uint16_t* out, hipStream_t s) {
  const int64_t ng = (K + group_size - 1) / group_size;
  const int64_t nw = 4 * ng;
  const int64_t total = out_rows * nw;
  if (total == 0) return hipSuccess;
  unsigned blocks = 0;
  const WordGrid gr = plan_words(out_rows, nw, blocks);
  if (blocks == 0) return hipErrorInvalidValue;
  const dim3 grid(blocks);
  if (bits == 4)
    hipLaunchKernelGGL(dequantize_kernel<4>, grid, dim3(256), 0, s, ids, out_rows, qw, qs,
                       table_rows, K, nw, ng, gr, out);
  else
    hipLaunchKernelGGL(dequantize_kernel<3>, grid, dim3(256), 0, s, ids, out_rows, qw, qs,
                       table_rows, K, nw, ng, gr, out);
  return hipGetLastError();
}

}  // namespace gq
