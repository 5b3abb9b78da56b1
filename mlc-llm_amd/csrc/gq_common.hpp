// Shared device helpers for the gfx950 group-quantization kernels.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gq {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;

// Compile-time facts of one scheme (group_quantization.py:57-61 of the reference).
template <int BITS>
struct Scheme {
  static constexpr int kBits = BITS;
  static constexpr int kElem = 32 / BITS;              // values per uint32: 8 | 10
  static constexpr int kMaxInt = (1 << (BITS - 1)) - 1;  // 7 | 3
  static constexpr uint32_t kMask = (1u << BITS) - 1u;
};

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ __forceinline__ uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }

// fp32-accumulating dot of two half pairs: v_dot2_f32_f16.
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2(as_half2(a), as_half2(b), c, false);
}

// the same for two bfloat16 pairs: v_dot2_f32_bf16 (exact products, fp32 accumulation)
typedef __bf16 bf16x2_dot_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_dot_t, a), __builtin_bit_cast(bf16x2_dot_t, b), c,
                                         false);
}
__device__ __forceinline__ float bf2f(uint16_t b) {
  return __builtin_bit_cast(float, static_cast<uint32_t>(b) << 16);
}
// round-to-nearest-even float -> bfloat16 (NaN stays NaN)
__device__ __forceinline__ uint16_t f2bf(float f) {
  const uint32_t u = __builtin_bit_cast(uint32_t, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
  return static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// (a & mask) | bits as ONE v_and_or_b32.  A VOP3 instruction takes a single 32-bit literal, so the
// compiler splits the two-constant form into v_and + v_or; keeping the mask in a VGPR and the OR
// bits in an SGPR makes the fused form encodable (both constants are loop invariant).
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t bits) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(mask), "s"(bits));
  return r;
}

// The same instruction, emitted by the compiler: the mask is laundered into a VGPR through an EMPTY asm statement
// (so that it is not folded back into a second literal) and the expression is left to instruction selection.
// This is the form for results that feed a matrix instruction directly.  An instruction inside an asm statement is
// invisible to the compiler's hazard handling and to its scheduler's latencies: with the asm form above, a
// v_and_or_b32 landed one instruction in front of the v_mfma_f32_4x4x4 that reads its result, and that matrix
// instruction used the register's old value (deterministic wrong sums in the first of two accumulator chains, q3
// forms with two chains per item); the compiler's own placement keeps seven or more instructions between them.
__device__ __forceinline__ uint32_t and_or_c(uint32_t a, uint32_t mask, uint32_t bits) {
  uint32_t m = mask;
  asm("" : "+v"(m));
  return (a & m) | bits;
}

__device__ __forceinline__ float h2f(uint16_t h) {
  return static_cast<float>(__builtin_bit_cast(_Float16, h));
}
// round-to-nearest-even float -> half (v_cvt_f16_f32 under the default rounding mode)
__device__ __forceinline__ uint16_t f2h(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

// Row of x that the (expert-sorted) activation row r reads: r itself, or x_rows[r] when the MoE
// layer's gather x[token_indices] is folded into the matmul; clamped into x.
__device__ __forceinline__ int64_t x_row(const int32_t* __restrict__ x_rows, int x_src_rows, int r) {
  if (x_rows == nullptr) return r;
  const int j = x_rows[r];
  return j < 0 ? 0 : (j >= x_src_rows ? x_src_rows - 1 : j);
}

// Fused gate/up form of a linear whose N stored rows are [gate rows; up rows] (N / 2 each): a kernel
// walks the rows in the interleaved order gate 0, up 0, gate 1, up 1, ... so that both halves of an
// output element are produced side by side.  Interleaved index -> stored row:
__device__ __forceinline__ int gate_up_row(int j, int N) { return (j >> 1) + (j & 1) * (N >> 1); }
// silu(gate) * up with the rounding points of the unfused sequence (fp16 matmul outputs, silu in
// fp32 rounded to fp16, fp16 product): bit-identical to linear followed by silu_mul
__device__ __forceinline__ uint16_t silu_mul_h(float gate, float up) {
  const float g = h2f(f2h(gate)), u = h2f(f2h(up));
  // hardware exp2 and reciprocal (1 ulp each): far inside the fp16 rounding of the result, and short
  // enough that the one lane that runs it in a GEMV epilogue does not hold its wave back
  const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896341f);
  const float silu = h2f(f2h(g * __builtin_amdgcn_rcpf(1.0f + e)));
  return f2h(silu * u);
}
// the same for a bfloat16 model: bfloat16 rounding points, hardware exp2 / reciprocal (1 ulp each, far inside
// the bfloat16 rounding); the element-wise silu_mul kernel of the bfloat16 models calls this very function
__device__ __forceinline__ uint16_t silu_mul_bf(float gate, float up) {
  const float g = bf2f(f2bf(gate)), u = bf2f(f2bf(up));
  const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896341f);
  const float silu = bf2f(f2bf(g * __builtin_amdgcn_rcpf(1.0f + e)));
  return f2bf(silu * u);
}
template <bool BF>
__device__ __forceinline__ uint16_t silu_mul_t(float gate, float up) {
  return BF ? silu_mul_bf(gate, up) : silu_mul_h(gate, up);
}

// Sum over the 64 lanes of a wave; every lane ends up with the total.
// quad_perm and row-mirror steps are DPP moves, the two widest steps cross rows via bpermute.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f<0x141>(v);  // row_half_mirror: lane i <-> 7-i inside each 8
  v += dpp_f<0x140>(v);  // row_mirror: lane i <-> 15-i inside each 16
  v += __shfl_xor(v, 16, kWave);
  v += __shfl_xor(v, 32, kWave);
  return v;
}

// Sum over the 64 lanes with DPP only; the total is valid in lane 63 alone.
// row_bcast15 adds lane 15 of the previous row into rows 1 and 3, row_bcast31 adds lane 31
// (rows 0+1) into rows 2 and 3.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_masked_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL,
                                                                ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float wave_sum_last(float v) {
  v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_f<0x141>(v);  // row_half_mirror
  v += dpp_f<0x140>(v);  // row_mirror: every lane now holds its row's sum
  v += dpp_masked_f<0x142, 0xA>(v);  // row_bcast15
  v += dpp_masked_f<0x143, 0xC>(v);  // row_bcast31
  return v;
}

}  // namespace gq
