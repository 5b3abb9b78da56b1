// Pieces shared by the MFMA GEMM kernels: scheme traits, kernel parameters, the segment walk of
// the grouped (MoE) form and the in-register dequantisation of one group.
#pragma once

#include "gq_common.hpp"
#include "gq_internal.hpp"

namespace gq {

template <int BITS>
struct GemmTraits;
template <>
struct GemmTraits<4> {
  static constexpr int G = 32;
};
template <>
struct GemmTraits<3> {
  static constexpr int G = 40;
};

struct GemmParams {
  const uint16_t* x;
  const uint32_t* qw;
  const uint16_t* qs;
  const uint16_t* bias;
  const uint16_t* residual;  // [rows, N] or null
  void* y;
  const void* indptr;
  int64_t expert_w_stride, expert_s_stride;
  int rows, N, K, ng, nw;
  int num_experts;
  int out_f32, indptr_i64;
  // split-K: workgroup z multiplies K tiles [z * kt_per_split, (z + 1) * kt_per_split) and, when
  // `partial` is set, leaves its fp32 tile in partial[z][rows][N] for the reduction kernel
  float* partial;
  int kt_per_split;
  int bm_hint;  // rows per tile chosen by plan_split_k (0: regular tiles)
  // Fused gate/up form: y[rows, N / 2] = silu(x . W[j]) * (x . W[N / 2 + j]).  A tile's columns walk
  // the stored rows in blocks of 32 gate rows then the matching 32 up rows, so both halves of an
  // output element sit in the same lane and register of neighbouring 32 x 32 accumulators (blocks of
  // 16 + 16 in the one tile whose waves own a single accumulator).
  int paired;
  const int32_t* x_rows;  // null, or the row of x each activation row reads (int32 [rows])
  int x_src_rows;         // rows of x when x_rows is set
  int bf16;               // x, q_scale, bias and a 16-bit y are bfloat16 (q4bf16_* models), not float16
  // columns (in tile order) this launch covers: [n_begin, n_end), n_end = 0 for all; a launch can leave the columns
  // of its last, partly filled round of workgroups to a second launch with another tile
  int n_begin = 0, n_end = 0;
  // every byte offset into x, one expert's q_weight and q_scale fits 32 bits, and K is whole K tiles of two groups
  // (set by the launcher; lets interior workgroups address with a uniform base plus a 32-bit lane offset)
  int fast_ok = 0;
  uint32_t x_bytes = 0;  // size of x (the form without zero-selects, whose offsets fit 32 bits)
};

// column c of the block-interleaved order above -> stored weight row (clamped into its half).
// PB: gate rows per block; 32 where a wave owns pairs of 32-column accumulators, 16 where it owns a
// single one (then lanes l and l ^ 16 hold the two halves of an output element).
template <int PB>
__device__ __forceinline__ int gate_up_row_blk(int c, int N) {
  const int half = N >> 1;
  const int o = min((c / (2 * PB)) * PB + (c % PB), half - 1);
  return (c & PB) ? half + o : o;
}

__global__ void splitk_reduce_kernel(const float* partial, int split, int64_t count, int N,
                                     const uint16_t* bias, const uint16_t* residual, void* y, int out_f32, int bf16);
// fused gate/up form: partial[split][rows][N] in the block-interleaved column order -> y fp16 [rows, N / 2]
__global__ void splitk_reduce_silu_kernel(const float* partial, int split, int64_t rows, int N, int pb,
                                          uint16_t* y, int bf16);
// gate rows per column block (32 | 16) of the tile launch_gemm_pipe picks for these parameters
int gemm_pipe_pair_block(const GemmParams& p, int bits);

// How a few-row GEMM is cut so that every CU streams weights: rows per tile and K splits.
struct SplitPlan {
  int bm;            // 0: not a few-row problem, use the regular tiles
  int split;         // workgroups along K (1: no reduction pass)
  int kt_per_split;  // K tiles (2 groups each) per workgroup
};
SplitPlan plan_split_k(int64_t rows, int64_t N, int64_t K, int bits, int group_size, bool grouped);

// One group (4 storage words) -> G halves in natural k order, (q - m) * s with fp16 rounding.
template <int BITS>
__device__ __forceinline__ void dequant_group(const uint4 w4, const uint16_t scale_bits,
                                              uint32_t* __restrict__ out /* G/2 half pairs */) {
  constexpr uint32_t kMagic = 0x64006400u;  // 1024.0 in both halves
  const uint32_t w[4] = {w4.x, w4.y, w4.z, w4.w};
  const _Float16 s = __builtin_bit_cast(_Float16, scale_bits);
  const half2_t s2 = {s, s};
  if (BITS == 4) {
    const half2_t off = {static_cast<_Float16>(-1031.0f), static_cast<_Float16>(-1031.0f)};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t t1 = w[i] >> 4;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // byte j of w -> low half (field 2j in its low nibble), byte j of w>>4 -> high half
        const uint32_t sel = 0x0c000c00u | ((4u + j) << 16) | static_cast<uint32_t>(j);
        const uint32_t r = and_or(__builtin_amdgcn_perm(t1, w[i], sel), 0x000f000fu, kMagic);
        out[4 * i + j] = as_u32((as_half2(r) + off) * s2);
      }
    }
  } else {
    const half2_t off = {static_cast<_Float16>(-1027.0f), static_cast<_Float16>(-1027.0f)};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int j = 0; j < 5; ++j) {
        const uint32_t t = w[i] >> (6 * j);
        const uint32_t r = and_or(t << 13, 0x00070000u, and_or(t, 0x00000007u, kMagic));
        out[5 * i + j] = as_u32((as_half2(r) + off) * s2);
      }
    }
  }
}


// 16-byte chunk c (0..4) of a q3 group: halves 8c .. 8c+7 = pairs 4c .. 4c+3 of the group, pair p being
// fields (2j, 2j+1) of word p / 5 with j = p % 5 (a pair never straddles two words).
__device__ __forceinline__ void dequant_chunk3(const uint4 w4, const uint16_t scale_bits, const int c,
                                               uint32_t* __restrict__ out) {
  constexpr uint32_t kMagic = 0x64006400u;
  const uint32_t w[4] = {w4.x, w4.y, w4.z, w4.w};
  const _Float16 s = __builtin_bit_cast(_Float16, scale_bits);
  const half2_t s2 = {s, s};
  const half2_t off = {static_cast<_Float16>(-1027.0f), static_cast<_Float16>(-1027.0f)};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int pr = 4 * c + i;
    const uint32_t t = w[pr / 5] >> (6 * (pr % 5));
    const uint32_t r = and_or(t << 13, 0x00070000u, and_or(t, 0x00000007u, kMagic));
    out[i] = as_u32((as_half2(r) + off) * s2);
  }
}

// One q4 storage word -> 8 halves in natural k order (4 half pairs), (q - 7) * s.
__device__ __forceinline__ void dequant_word4(const uint32_t w, const uint16_t scale_bits,
                                              uint32_t* __restrict__ out) {
  constexpr uint32_t kMagic = 0x64006400u;
  const _Float16 s = __builtin_bit_cast(_Float16, scale_bits);
  const half2_t s2 = {s, s};
  const half2_t off = {static_cast<_Float16>(-1031.0f), static_cast<_Float16>(-1031.0f)};
  const uint32_t t1 = w >> 4;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t sel = 0x0c000c00u | ((4u + j) << 16) | static_cast<uint32_t>(j);
    const uint32_t r = and_or(__builtin_amdgcn_perm(t1, w, sel), 0x000f000fu, kMagic);
    out[j] = as_u32((as_half2(r) + off) * s2);
  }
}

// bfloat16 models (q4bf16_*): the same, with the product (q - m) * s formed exactly in float32
// (a 4-bit by an 8-bit significand) and rounded to a bf16 pair by v_cvt_pk_bf16_f32, which is the
// rounding GroupQuantize._dequantize applies in that dtype.  scale_bits are bfloat16 bits.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t bf16_pair(float a, float b) {
  const float2_t f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}
__device__ __forceinline__ uint16_t bf16_bits_of(float v) {
  return static_cast<uint16_t>(bf16_pair(v, 0.0f) & 0xffffu);
}
__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
  return __builtin_bit_cast(float, static_cast<uint32_t>(b) << 16);
}
__device__ __forceinline__ void dequant_word4_bf16(const uint32_t w, const uint16_t scale_bits,
                                                   uint32_t* __restrict__ out) {
  const float s = bf16_to_f32(scale_bits), ms = -7.0f * s;
  const uint32_t t0 = w & 0x0f0f0f0fu, t1 = (w >> 4) & 0x0f0f0f0fu;  // even / odd fields, one per byte
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float lo = static_cast<float>((t0 >> (8 * j)) & 0xffu), hi = static_cast<float>((t1 >> (8 * j)) & 0xffu);
    out[j] = bf16_pair(fmaf(lo, s, ms), fmaf(hi, s, ms));
  }
}
template <int BITS>
__device__ __forceinline__ void dequant_group_bf16(const uint4 w4, const uint16_t scale_bits,
                                                   uint32_t* __restrict__ out /* G/2 bf16 pairs */) {
  using S = Scheme<BITS>;
  constexpr int E = S::kElem;
  const uint32_t w[4] = {w4.x, w4.y, w4.z, w4.w};
  const float s = bf16_to_f32(scale_bits), ms = -static_cast<float>(S::kMaxInt) * s;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < E / 2; ++j) {
      const float lo = static_cast<float>((w[i] >> (2 * j * BITS)) & S::kMask);
      const float hi = static_cast<float>((w[i] >> ((2 * j + 1) * BITS)) & S::kMask);
      out[(E / 2) * i + j] = bf16_pair(fmaf(lo, s, ms), fmaf(hi, s, ms));
    }
}

// Which activation rows [seg_lo, seg_hi) and which expert the m-tile `t` of a launch belongs to.
// Plain linear: one segment.  Grouped: walk indptr (python/mlc_llm/op/moe_matmul.py:653-679 of
// the reference does the same walk per tile).  Returns false when the tile does not exist.
template <int BM>
__device__ __forceinline__ bool locate_tile(const GemmParams& p, int t, int& seg_lo, int& seg_hi,
                                            int& mt, int& expert) {
  seg_lo = 0; seg_hi = p.rows; mt = t; expert = 0;
  if (p.indptr == nullptr) return t * BM < p.rows;
  for (int e = 0; e < p.num_experts; ++e) {
    int64_t lo, hi;
    if (p.indptr_i64) {
      lo = static_cast<const int64_t*>(p.indptr)[e];
      hi = static_cast<const int64_t*>(p.indptr)[e + 1];
    } else {
      lo = static_cast<const int32_t*>(p.indptr)[e];
      hi = static_cast<const int32_t*>(p.indptr)[e + 1];
    }
    lo = lo < 0 ? 0 : (lo > p.rows ? p.rows : lo);  // a corrupt indptr must not leave the tensors
    hi = hi < lo ? lo : (hi > p.rows ? p.rows : hi);
    const int tiles = static_cast<int>((hi - lo + BM - 1) / BM);
    if (t < tiles) {
      seg_lo = static_cast<int>(lo); seg_hi = static_cast<int>(hi); mt = t; expert = e;
      return true;
    }
    t -= tiles;
  }
  return false;
}

// software-pipelined kernel family (needs K % 8 == 0); hipErrorNotSupported otherwise
hipError_t launch_gemm_pipe(const GemmParams& p, int bits, hipStream_t s);

}  // namespace gq
