// quantize / dequantize / embedding take for the model dtypes other than float16: the
// `q4f32_1` (float32) and `q4bf16_*` (bfloat16) entries of the reference registry
// (python/mlc_llm/quantization/quantization.py:91-123).  Same tensor expressions as gq_quant.hip
// restates (group_quantization.py:155-186, 235-306; utils.py:15-48, 136-188) with `model_dtype`
// in place of float16: the weights, the scales and every intermediate of `_quantize` /
// `_dequantize` carry that type.
//
// Arithmetic: each operation is one float operation followed by a rounding to the model dtype.  For
// float32 that is IEEE single arithmetic as written.  For bfloat16 it is what TVM's bf16
// legalisation emits (operands widened to float32, the operation done there, the result rounded to
// nearest even): a quotient or sum of two 8-bit significands is far from any float32 rounding
// boundary that could move the second rounding, so this is also the correctly rounded bf16 result.
#include "gq_quant_common.hpp"

namespace gq {

template <int DT>
struct ModelT;

template <>
struct ModelT<MODEL_F32> {
  using storage = float;
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return static_cast<const float*>(p)[i]; }
  static __device__ __forceinline__ void save(void* p, int64_t i, float v) { static_cast<float*>(p)[i] = v; }
  static __device__ __forceinline__ float rnd(float v) { return v; }
  static constexpr float kLowest = -3.402823466e+38f;  // min_value(float32), the pad of the group maximum
  // E consecutive values at an even element index (a multiple of 8 when E == 8)
  template <int E>
  static __device__ __forceinline__ void load_word(const void* p, int64_t i, float (&v)[E]) {
    const float* f = static_cast<const float*>(p) + i;
    if constexpr (E == 8) {
      const float4 a = *reinterpret_cast<const float4*>(f), b = *reinterpret_cast<const float4*>(f + 4);
      v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
#pragma unroll
      for (int j = 0; j < E / 2; ++j) {
        const float2 a = *reinterpret_cast<const float2*>(f + 2 * j);
        v[2 * j] = a.x; v[2 * j + 1] = a.y;
      }
    }
  }
  template <int E>
  static __device__ __forceinline__ void save_word(void* p, int64_t i, const float (&v)[E]) {
    float* f = static_cast<float*>(p) + i;
    if constexpr (E == 8) {
      *reinterpret_cast<float4*>(f) = make_float4(v[0], v[1], v[2], v[3]);
      *reinterpret_cast<float4*>(f + 4) = make_float4(v[4], v[5], v[6], v[7]);
    } else {
#pragma unroll
      for (int j = 0; j < E / 2; ++j) *reinterpret_cast<float2*>(f + 2 * j) = make_float2(v[2 * j], v[2 * j + 1]);
    }
  }
};

template <>
struct ModelT<MODEL_BF16> {
  using storage = uint16_t;
  static __device__ __forceinline__ float load(const void* p, int64_t i) {
    return __builtin_bit_cast(float, static_cast<uint32_t>(static_cast<const uint16_t*>(p)[i]) << 16);
  }
  static __device__ __forceinline__ uint16_t bits(float v) {
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);  // NaN stays NaN
    return static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);                    // nearest even
  }
  static __device__ __forceinline__ void save(void* p, int64_t i, float v) { static_cast<uint16_t*>(p)[i] = bits(v); }
  static __device__ __forceinline__ float rnd(float v) {
    return __builtin_bit_cast(float, static_cast<uint32_t>(bits(v)) << 16);
  }
  static constexpr float kLowest = -3.38953139e+38f;  // min_value(bfloat16)
  template <int E>
  static __device__ __forceinline__ void load_word(const void* p, int64_t i, float (&v)[E]) {
    const uint16_t* h = static_cast<const uint16_t*>(p) + i;
    uint32_t pr[E / 2];
    if constexpr (E == 8) {
      const uint4 a = *reinterpret_cast<const uint4*>(h);
      pr[0] = a.x; pr[1] = a.y; pr[2] = a.z; pr[3] = a.w;
    } else {
#pragma unroll
      for (int j = 0; j < E / 2; ++j) pr[j] = reinterpret_cast<const uint32_t*>(h)[j];
    }
#pragma unroll
    for (int j = 0; j < E / 2; ++j) {
      v[2 * j] = __builtin_bit_cast(float, pr[j] << 16);
      v[2 * j + 1] = __builtin_bit_cast(float, pr[j] & 0xffff0000u);
    }
  }
  template <int E>
  static __device__ __forceinline__ void save_word(void* p, int64_t i, const float (&v)[E]) {
    uint16_t* h = static_cast<uint16_t*>(p) + i;
    uint32_t pr[E / 2];
#pragma unroll
    for (int j = 0; j < E / 2; ++j) pr[j] = static_cast<uint32_t>(bits(v[2 * j])) | (static_cast<uint32_t>(bits(v[2 * j + 1])) << 16);
    if constexpr (E == 8) {
      *reinterpret_cast<uint4*>(h) = make_uint4(pr[0], pr[1], pr[2], pr[3]);
    } else {
#pragma unroll
      for (int j = 0; j < E / 2; ++j) reinterpret_cast<uint32_t*>(h)[j] = pr[j];
    }
  }
};

// One thread per storage word, a lane quad per group (the layout of gq_quant.hip).
template <int BITS, int DT, int HALF_EVEN>
__global__ __launch_bounds__(256) void quantize_dt_kernel(const void* __restrict__ w, int64_t rows, int64_t K,
                                                          int64_t nw, int64_t ng, int group_size, WordGrid gr,
                                                          uint32_t* __restrict__ qw, void* __restrict__ qs) {
  using S = Scheme<BITS>;
  using T = ModelT<DT>;
  constexpr int E = S::kElem;
  int64_t row, wd;
  locate_word(gr, nw, row, wd);
  const bool live = row < rows;  // inactive lanes (whole quads) still take part in the shuffles
  if (!live) { row = rows - 1; wd = nw - 1; }
  const int64_t g = wd >> 2;
  const int64_t k0 = g * group_size + (wd & 3) * E;

  float v[E];
  bool ok[E];
  float amax = T::kLowest;  // lanes beyond K contribute the type's lowest value, as the reference pads
  if (k0 + E <= K && (K & 7) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0) {
    // whole word inside the row and rows 16-byte aligned: 8-byte (q3) or 16-byte (q4) loads
    T::template load_word<E>(w, row * K + k0, v);
#pragma unroll
    for (int i = 0; i < E; ++i) ok[i] = true;
  } else {
#pragma unroll
    for (int i = 0; i < E; ++i) {
      ok[i] = (k0 + i) < K;
      v[i] = ok[i] ? T::load(w, row * K + k0 + i) : 0.0f;
    }
  }
#pragma unroll
  for (int i = 0; i < E; ++i) {
    const float a = fabsf(v[i]);
    amax = (ok[i] && a > amax) ? a : amax;
  }
  amax = fmaxf(amax, dpp_f<0xB1>(amax));
  amax = fmaxf(amax, dpp_f<0x4E>(amax));

  const float m = static_cast<float>(S::kMaxInt);
  const float s = T::rnd(amax / m);
  // bfloat16: the quotient only has to round to the right bf16, and a ratio of two 8-bit significands
  // that is not itself a bf16 rounding boundary stays 2^-17 (relative) away from one, so the hardware
  // reciprocal with one Newton step (about 1 ulp of float32) rounds like the exact quotient; scales
  // of zero, infinity or NaN keep the first product (NaN / infinity / zero, as a divide gives).
  // float32 needs the correctly rounded divide itself.
  const float rs = __builtin_amdgcn_rcpf(s);
  const bool plain = !(s > 0.0f && s < __builtin_inff());
  uint32_t word = 0;
#pragma unroll
  for (int i = 0; i < E; ++i) {
    float quo;
    if constexpr (DT == MODEL_BF16) {
      const float q0 = v[i] * rs;
      quo = plain ? q0 : fmaf(fmaf(-q0, s, v[i]), rs, q0);
    } else {
      quo = v[i] / s;  // IEEE divide (0 / 0 = NaN for an all-zero group)
    }
    float t = T::rnd(quo);
    t = T::rnd(t + m);
    float r = HALF_EVEN ? rintf(t) : roundf(t);
    r = (r > 0.0f) ? r : 0.0f;  // compare-and-select max: NaN becomes 0
    r = (r < 2.0f * m) ? r : 2.0f * m;
    const uint32_t q = ok[i] ? static_cast<uint32_t>(r) : 0u;
    word |= q << (i * BITS);
  }
  if (live) {
    qw[row * nw + wd] = word;
    if ((wd & 3) == 0) T::save(qs, row * ng + g, s);
  }
}

// out[orow, k] = (unpack(qw[row, k]) - m) * qs[row, k / G] for k < K; row = ids ? ids[orow] : orow
template <int BITS, int DT>
__global__ __launch_bounds__(256) void dequantize_dt_kernel(const int32_t* __restrict__ ids, int64_t out_rows,
                                                            const uint32_t* __restrict__ qw,
                                                            const void* __restrict__ qs, int64_t table_rows,
                                                            int64_t K, int64_t nw, int64_t ng, WordGrid gr,
                                                            void* __restrict__ out) {
  using S = Scheme<BITS>;
  using T = ModelT<DT>;
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
  const float s = T::load(qs, row * ng + (wd >> 2));
  float o[E];
#pragma unroll
  for (int i = 0; i < E; ++i) {
    const int u = static_cast<int>((word >> (i * BITS)) & S::kMask);
    o[i] = static_cast<float>(u - S::kMaxInt) * s;  // (u - m) is exact in either type; one multiply, rounded at the store
  }
  if (k0 + E <= K && (K & 7) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
    T::template save_word<E>(out, orow * K + k0, o);
  } else {
#pragma unroll
    for (int i = 0; i < E; ++i)
      if (k0 + i < K) T::save(out, orow * K + k0 + i, o[i]);
  }
}

template <int BITS, int DT>
static hipError_t quantize_dt(const void* w, int64_t rows, int64_t K, int group_size, int round_mode,
                              uint32_t* qw, void* qs, hipStream_t s) {
  const int64_t ng = (K + group_size - 1) / group_size;
  const int64_t nw = 4 * ng;
  if (rows * nw == 0) return hipSuccess;
  unsigned blocks = 0;
  const WordGrid gr = plan_words(rows, nw, blocks);
  if (blocks == 0) return hipErrorInvalidValue;
  if (round_mode == 0)
    hipLaunchKernelGGL((quantize_dt_kernel<BITS, DT, 0>), dim3(blocks), dim3(256), 0, s, w, rows, K, nw, ng,
                       group_size, gr, qw, qs);
  else
    hipLaunchKernelGGL((quantize_dt_kernel<BITS, DT, 1>), dim3(blocks), dim3(256), 0, s, w, rows, K, nw, ng,
                       group_size, gr, qw, qs);
  return hipGetLastError();
}

hipError_t launch_quantize_dt(const void* w, int64_t rows, int64_t K, int bits, int group_size, int round_mode,
                              int model_dtype, uint32_t* qw, void* qs, hipStream_t s) {
  if (model_dtype == MODEL_F32)
    return bits == 4 ? quantize_dt<4, MODEL_F32>(w, rows, K, group_size, round_mode, qw, qs, s)
                     : quantize_dt<3, MODEL_F32>(w, rows, K, group_size, round_mode, qw, qs, s);
  if (model_dtype == MODEL_BF16)
    return bits == 4 ? quantize_dt<4, MODEL_BF16>(w, rows, K, group_size, round_mode, qw, qs, s)
                     : quantize_dt<3, MODEL_BF16>(w, rows, K, group_size, round_mode, qw, qs, s);
  return hipErrorInvalidValue;
}

template <int BITS, int DT>
static hipError_t dequantize_dt(const int32_t* ids, int64_t out_rows, const uint32_t* qw, const void* qs,
                                int64_t table_rows, int64_t K, int group_size, void* out, hipStream_t s) {
  const int64_t ng = (K + group_size - 1) / group_size;
  const int64_t nw = 4 * ng;
  if (out_rows * nw == 0) return hipSuccess;
  unsigned blocks = 0;
  const WordGrid gr = plan_words(out_rows, nw, blocks);
  if (blocks == 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL((dequantize_dt_kernel<BITS, DT>), dim3(blocks), dim3(256), 0, s, ids, out_rows, qw, qs,
                     table_rows, K, nw, ng, gr, out);
  return hipGetLastError();
}

hipError_t launch_dequantize_dt(const int32_t* ids, int64_t out_rows, const uint32_t* qw, const void* qs,
                                int64_t table_rows, int64_t K, int bits, int group_size, int model_dtype,
                                void* out, hipStream_t s) {
  if (model_dtype == MODEL_F32)
    return bits == 4 ? dequantize_dt<4, MODEL_F32>(ids, out_rows, qw, qs, table_rows, K, group_size, out, s)
                     : dequantize_dt<3, MODEL_F32>(ids, out_rows, qw, qs, table_rows, K, group_size, out, s);
  if (model_dtype == MODEL_BF16)
    return bits == 4 ? dequantize_dt<4, MODEL_BF16>(ids, out_rows, qw, qs, table_rows, K, group_size, out, s)
                     : dequantize_dt<3, MODEL_BF16>(ids, out_rows, qw, qs, table_rows, K, group_size, out, s);
  return hipErrorInvalidValue;
}

}  // namespace gq
