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

// What a launcher knows about one GEMV.  The LDS-staged kernel takes the struct as its argument; the register kernel
// takes the fields of the first block as ten scalar arguments, which arrive in scalar registers with the wave, and the
// rest as a struct of its own behind them.  Why the split: a kernel's arguments sit in memory that every launch reads
// cold, 64 bytes per line; the read at the start of the batch-1 linear cost 0.4 us per launch, and each further line a
// kernel touched another 0.1-0.25 us (measured: 32 more bytes of arguments, which pushed the launch dimensions the
// kernel also read into one more line, took a 129-launch decode step from 1.177 to 1.204 ms; the first block alone in
// one line 1.179 -> 1.160; no read at all 1.161 -> 1.108).
struct GemvParams {
  // ---- every form (the register kernel's leading arguments, with nw = 4 * ng)
  const uint16_t* x;
  const uint32_t* qw;
  const uint16_t* qs;
  void* y;
  int N, K, ng, nw;
  int nsets = 0;   // row sets the launch walks (register kernel; set by its launcher)
  int nwaves = 0;  // waves of one grid row (register kernel; set by its launcher)
  int out_f32;
  int num_experts;
  int paired;  // fused gate/up form: y[.., N / 2] = silu(x . W[j]) * (x . W[N / 2 + j]), fp16
  int bf16;    // x, q_scale, bias, residual and a 16-bit y are bfloat16 (register kernel only)
  int routed = 0;
  int sum2 = 0;  // the two slots' results are weighted and summed in the launch (`residual` points at the two weights)
  int gc;  // groups staged per LDS chunk (multiple of 64; LDS kernel)
  // ---- bias / residual forms and expert forms
  const uint16_t* bias;
  const uint16_t* residual;  // [M, N] or null
  const int32_t* expert_ids;
  int64_t x_slot_stride;
  int64_t expert_w_stride;  // N * nw
  int64_t expert_s_stride;  // N * ng
  // rows sorted by expert instead of expert_ids (register kernel only): slot s belongs to the expert e with
  // indptr[e] <= s < indptr[e + 1] (slots outside every segment are left alone) and reads x row
  // x_row_index[s] (null: row s)
  const void* indptr;
  const int32_t* x_row_index;
  int indptr_i64;
  int x_src_rows;
  // The token routes itself (register kernel, fused gate/up form of one row): `routed` is set and three fields change
  // their meaning: `bias` holds the
  // token's num_experts router logits in the model dtype, `residual` points at the top_k softmax weights to write and
  // `expert_ids` at the top_k ids to write.  Every workgroup picks the top gridDim.y logits (the insertion of the
  // routing kernels) and serves slot blockIdx.y's expert; the first workgroup leaves ids and weights for the operators
  // that follow.
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

// The same for bfloat16 activations.  0x4300 | q is the bfloat16 128 + q (q < 128: the seven mantissa bits
// count ones there), so a field must sit at bit 0 of its half: one shift per field pair where the float16
// form rescales instead.  Pairs come in the same order as above, so permute_group serves both.
template <int BITS>
__device__ __forceinline__ float group_dot_bf16(const uint4 w4, const uint32_t* __restrict__ xr, float corr) {
  const uint32_t w[4] = {w4.x, w4.y, w4.z, w4.w};
  constexpr uint32_t kMagic = 0x43004300u;
  float a0 = 0.f, a1 = 0.f;
  if (BITS == 4) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a0 = dot2_bf16(and_or(w[i], 0x000f000fu, kMagic), xr[4 * i + 0], a0);
      a1 = dot2_bf16(and_or(w[i] >> 4, 0x000f000fu, kMagic), xr[4 * i + 1], a1);
      a0 = dot2_bf16(and_or(w[i] >> 8, 0x000f000fu, kMagic), xr[4 * i + 2], a0);
      a1 = dot2_bf16(and_or(w[i] >> 12, 0x000f000fu, kMagic), xr[4 * i + 3], a1);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // low half keeps fields 0-4, high half gets fields 5-9 aligned to bit 16
      const uint32_t t = (w[i] & 0x0000ffffu) | ((w[i] << 1) & 0xffff0000u);
      a0 = dot2_bf16(and_or(t, 0x00070007u, kMagic), xr[5 * i + 0], a0);
      a1 = dot2_bf16(and_or(t >> 3, 0x00070007u, kMagic), xr[5 * i + 1], a1);
      a0 = dot2_bf16(and_or(t >> 6, 0x00070007u, kMagic), xr[5 * i + 2], a0);
      a1 = dot2_bf16(and_or(t >> 9, 0x00070007u, kMagic), xr[5 * i + 3], a1);
      a0 = dot2_bf16(and_or(t >> 12, 0x00070007u, kMagic), xr[5 * i + 4], a0);
    }
  }
  return (a0 + a1) - corr;
}

// x pairs of one group in the order the unpack masks produce them, from the natural-order halves.
// v_perm_b32 picks the two 16-bit lanes directly: byte selectors 0-3 address S1, 4-7 address S0.
// BF: bfloat16 activations; every field then carries the same offset 128 + m.
template <int BITS, bool BF = false>
__device__ __forceinline__ float permute_group(const uint32_t* __restrict__ n /* G/2 natural pairs */,
                                               uint32_t* __restrict__ xr /* G/2 permuted pairs */) {
  constexpr uint32_t kLoLo = 0x05040100u;  // (lo16(S1), lo16(S0))
  constexpr uint32_t kHiHi = 0x07060302u;  // (hi16(S1), hi16(S0))
  constexpr uint32_t kLoHi = 0x07060100u;  // (lo16(S1), hi16(S0))
  constexpr uint32_t kHiLo = 0x05040302u;  // (hi16(S1), lo16(S0))
  float c = 0.f;
  if (BITS == 4) {
    // word w holds x[8w..8w+7] as pairs (0,1)(2,3)(4,5)(6,7); wanted (0,4)(1,5)(2,6)(3,7).
    // Fields 1,3,5,7 come out of the mask times 16: their 1024 shrinks to 64 after rescaling.
    const uint32_t c_lo = 0x64076407u;  // (1031, 1031)
    const uint32_t c_hi = 0x54705470u;  // (71, 71)
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      xr[4 * w + 0] = __builtin_amdgcn_perm(n[4 * w + 2], n[4 * w + 0], kLoLo);
      xr[4 * w + 1] = __builtin_amdgcn_perm(n[4 * w + 2], n[4 * w + 0], kHiHi);
      xr[4 * w + 2] = __builtin_amdgcn_perm(n[4 * w + 3], n[4 * w + 1], kLoLo);
      xr[4 * w + 3] = __builtin_amdgcn_perm(n[4 * w + 3], n[4 * w + 1], kHiHi);
      if constexpr (BF) {
#pragma unroll
        for (int j = 0; j < 4; ++j) c = dot2_bf16(xr[4 * w + j], 0x43074307u /* (135, 135) */, c);
      } else {
        c = dot2(xr[4 * w + 0], c_lo, c);
        c = dot2(xr[4 * w + 1], c_hi, c);
        c = dot2(xr[4 * w + 2], c_lo, c);
        c = dot2(xr[4 * w + 3], c_hi, c);
      }
    }
  } else {
    // word w holds x[10w..10w+9] as 5 natural pairs; wanted (j, j+5); pair j sits at mantissa
    // bit 3*(j mod 3), so its 1024 becomes 1024, 128 or 16 after rescaling (+ m = 3).
    const uint32_t c1 = 0x64036403u;   // (1027, 1027)
    const uint32_t c8 = 0x58185818u;   // (131, 131)
    const uint32_t c64 = 0x4cc04cc0u;  // (19, 19)
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t* r = n + 5 * w;
      xr[5 * w + 0] = __builtin_amdgcn_perm(r[2], r[0], kLoHi);
      xr[5 * w + 1] = __builtin_amdgcn_perm(r[3], r[0], kHiLo);
      xr[5 * w + 2] = __builtin_amdgcn_perm(r[3], r[1], kLoHi);
      xr[5 * w + 3] = __builtin_amdgcn_perm(r[4], r[1], kHiLo);
      xr[5 * w + 4] = __builtin_amdgcn_perm(r[4], r[2], kLoHi);
      if constexpr (BF) {
#pragma unroll
        for (int j = 0; j < 5; ++j) c = dot2_bf16(xr[5 * w + j], 0x43034303u /* (131, 131) */, c);
      } else {
        c = dot2(xr[5 * w + 0], c1, c);
        c = dot2(xr[5 * w + 1], c8, c);
        c = dot2(xr[5 * w + 2], c64, c);
        c = dot2(xr[5 * w + 3], c1, c);
        c = dot2(xr[5 * w + 4], c8, c);
      }
    }
  }
  return c;
}


// launchers of the kernel families (each in its own translation unit)
hipError_t launch_gemv_lds(const GemvParams& p, int bits, int nb, int slots, hipStream_t s);
// register-resident x, persistent waves; returns hipErrorNotSupported when the shape does not fit
hipError_t launch_gemv_reg(const GemvParams& p, int bits, int nb, int slots, hipStream_t s);

}  // namespace gq
