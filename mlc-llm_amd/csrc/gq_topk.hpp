// Top-k selection of the router (python/mlc_llm/op/moe_misc.py:135-235 of the reference), shared by the routing
// kernels and by the expert GEMV that routes its own token.
#pragma once
#include "gq_common.hpp"
#include "gq_internal.hpp"

namespace gq {

// Elements of the model dtype (MODEL_F16 | MODEL_F32 | MODEL_BF16): load as float, round a float to
// the dtype, store.  The float16 forms are the original kernels; the others follow the same rounding
// points with their own rounding (every op in fp32, its result rounded to the dtype).
template <int DT>
struct Elem;
template <>
struct Elem<MODEL_F16> {
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return h2f(static_cast<const uint16_t*>(p)[i]); }
  static __device__ __forceinline__ float rnd(float v) { return h2f(f2h(v)); }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { static_cast<uint16_t*>(p)[i] = f2h(v); }
  static constexpr float kLowest = -65504.0f;
};
template <>
struct Elem<MODEL_F32> {
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return static_cast<const float*>(p)[i]; }
  static __device__ __forceinline__ float rnd(float v) { return v; }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { static_cast<float*>(p)[i] = v; }
  static constexpr float kLowest = -3.402823466e38f;
};
template <>
struct Elem<MODEL_BF16> {
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return bf2f(static_cast<const uint16_t*>(p)[i]); }
  static __device__ __forceinline__ float rnd(float v) { return bf2f(f2bf(v)); }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) { static_cast<uint16_t*>(p)[i] = f2bf(v); }
  static constexpr float kLowest = -3.3895313892515355e38f;  // min_value(bfloat16)
};

// Insertion top-k with strict '>' (ties keep the lower expert index) over logits[row0 .. row0 + ne), into registers:
// val / idx hold the k best in descending order (slots past k keep min_value(dtype), expert 0).
template <int KMAX, int DT>
__device__ __forceinline__ void topk_insert(const void* __restrict__ logits, int64_t row0, int ne, int k,
                                            float (&val)[KMAX], int (&idx)[KMAX]) {
#pragma unroll
  for (int i = 0; i < KMAX; ++i) {
    val[i] = Elem<DT>::kLowest;  // min_value(dtype)
    idx[i] = 0;
  }
  for (int e = 0; e < ne; ++e) {
    const float v = Elem<DT>::load(logits, row0 + e);
    bool placed = false;
#pragma unroll
    for (int i = 0; i < KMAX; ++i) {
      if (i < k && !placed && v > val[i]) {
#pragma unroll
        for (int j = KMAX - 1; j > 0; --j) {
          if (j > i && j < k) {
            val[j] = val[j - 1];
            idx[j] = idx[j - 1];
          }
        }
        val[i] = v;
        idx[i] = e;
        placed = true;
      }
    }
  }
}

// softmax over the k selected logits in fp32, in slot order, and the stores of one token's results
template <int KMAX, int DT>
__device__ __forceinline__ void softmax_store(const float (&val)[KMAX], const int (&idx)[KMAX], int k,
                                              void* __restrict__ w, int64_t w0, int32_t* __restrict__ ids) {
  float mx = val[0];
#pragma unroll
  for (int i = 1; i < KMAX; ++i)
    if (i < k) mx = fmaxf(mx, val[i]);
  float ex[KMAX];
  float den = 0.f;
#pragma unroll
  for (int i = 0; i < KMAX; ++i) {
    if (i < k) {
      ex[i] = expf(val[i] - mx);
      den = (i == 0) ? ex[0] : den + ex[i];
    }
  }
#pragma unroll
  for (int i = 0; i < KMAX; ++i) {
    if (i < k) {
      Elem<DT>::store(w, w0 + i, ex[i] / den);
      ids[i] = idx[i];
    }
  }
}

}  // namespace gq
