// Prefill GEMM and MoE grouped GEMM: y[m, n] = sum_k x[m, k] * dequant(W)[n, k] on fp16 MFMA.
//
// Replaces the TVM-generated fused_dequantize*_NT_matmul kernel for M > 8
// (python/mlc_llm/quantization/group_quantization.py:390-437 through
// compiler_pass/low_batch_specialization.py:44-57) and moe_matmul.dequantize_group_gemm
// (python/mlc_llm/op/moe_matmul.py:562-768; the indptr segment walk of :653-679 is the
// tile-to-expert mapping below).
//
// MFMA-bound.  A workgroup (4 waves) owns a BM x BN output tile and walks K in tiles of two
// quantisation groups.  Per K tile:
//  * activations go global -> registers -> LDS unchanged (16-byte chunks);
//  * packed weights go global -> registers (one 128-bit load = one group), are dequantised in
//    registers exactly as the reference does (fp16 (q - m), then one fp16 multiply by the scale)
//    and are written to LDS in natural k order;
//  * both LDS tiles are k-contiguous with rows padded by 16 bytes, which makes every
//    ds_read_b128 / ds_write_b128 of 16 consecutive lanes hit 64 distinct banks;
//  * each wave feeds v_mfma_f32_32x32x16_f16 from 16-byte LDS fragments, fp32 accumulators;
//  * global loads of tile t+1 are issued before the MFMAs of tile t, dequantisation and the LDS
//    stores of t+1 after them (two LDS stages, one barrier per tile).
#include "gq_gemm_common.hpp"

namespace gq {

template <int BITS, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(64 * (BM / WM) * (BN / WN)) void gemm_kernel(const GemmParams p) {
  using T = GemmTraits<BITS>;
  constexpr int G = T::G;
  constexpr int BK = 2 * G;            // 64 | 80
  constexpr int KSTEPS = BK / 16;      // MFMA k = 16
  constexpr int CPR = BK / 8;          // 16-byte chunks per tile row
  constexpr int LDA = BK + 8;          // padded row, in halves
  constexpr int WAVES_N = BN / WN;
  constexpr int NT = 64 * (BM / WM) * (BN / WN);  // threads per workgroup (4 or 8 waves)
  static_assert(NT == 256 || NT == 512, "4 or 8 waves per workgroup");
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int A_CHUNKS = BM * CPR / NT;  // 16-byte chunks of x per thread per tile
  constexpr int W_GROUPS = BN * 2 / NT;    // groups of W per thread per tile
  static_assert(BM * CPR % NT == 0 && BN * 2 % NT == 0, "tile / thread mismatch");

  extern __shared__ uint4 smem[];
  uint16_t* lds = reinterpret_cast<uint16_t*>(smem);
  // stage s: A at s*(BM+BN)*LDA, W right after A
  auto a_tile = [&](int s) { return lds + s * (BM + BN) * LDA; };
  auto w_tile = [&](int s) { return lds + s * (BM + BN) * LDA + BM * LDA; };

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;

  // ---- which rows / which expert does this workgroup own
  int seg_lo, seg_hi, mt, expert;
  if (!locate_tile<BM>(p, blockIdx.y, seg_lo, seg_hi, mt, expert)) return;  // uniform
  const int m0 = seg_lo + mt * BM;
  if (m0 >= seg_hi) return;
  const int n0 = blockIdx.x * BN;
  const uint32_t* qw = p.qw + expert * p.expert_w_stride;
  const uint16_t* qs = p.qs + expert * p.expert_s_stride;

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  uint4 a_reg[A_CHUNKS];
  uint4 w_reg[W_GROUPS];
  uint16_t s_reg[W_GROUPS];
  const bool k_vec = (p.K & 7) == 0;

  auto load_tile = [&](int kt) {
    const int k_base = kt * BK;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int idx = tid + NT * i;
      const int r = idx / CPR, c = idx - r * CPR;
      const int row = m0 + r, k = k_base + 8 * c;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (row < seg_hi && k < p.K) {
        const uint16_t* src = p.x + x_row(p.x_rows, p.x_src_rows, row) * p.K + k;
        if (k_vec) {
          v = *reinterpret_cast<const uint4*>(src);
        } else {
          uint16_t e[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) e[q] = (k + q < p.K) ? src[q] : uint16_t(0);
          v.x = e[0] | (uint32_t(e[1]) << 16); v.y = e[2] | (uint32_t(e[3]) << 16);
          v.z = e[4] | (uint32_t(e[5]) << 16); v.w = e[6] | (uint32_t(e[7]) << 16);
        }
      }
      a_reg[i] = v;
    }
#pragma unroll
    for (int i = 0; i < W_GROUPS; ++i) {
      const int idx = tid + NT * i;
      const int r = idx >> 1, gsel = idx & 1;
      const int row = min(n0 + r, p.N - 1);
      const int g = 2 * kt + gsel;
      if (g < p.ng) {
        w_reg[i] = *reinterpret_cast<const uint4*>(qw + static_cast<int64_t>(row) * p.nw + 4 * g);
        s_reg[i] = qs[static_cast<int64_t>(row) * p.ng + g];
      } else {
        w_reg[i] = make_uint4(0, 0, 0, 0);
        s_reg[i] = 0;  // scale +0.0: the whole group dequantises to (-m) * 0 = -0.0
      }
    }
  };

  auto store_tile = [&](int s) {
    uint16_t* at = a_tile(s);
    uint16_t* wt = w_tile(s);
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int idx = tid + NT * i;
      const int r = idx / CPR, c = idx - r * CPR;
      *reinterpret_cast<uint4*>(at + r * LDA + 8 * c) = a_reg[i];
    }
#pragma unroll
    for (int i = 0; i < W_GROUPS; ++i) {
      const int idx = tid + NT * i;
      const int r = idx >> 1, gsel = idx & 1;
      uint32_t d[G / 2];
      dequant_group<BITS>(w_reg[i], s_reg[i], d);
      uint4* dst = reinterpret_cast<uint4*>(wt + r * LDA + gsel * G);
#pragma unroll
      for (int c = 0; c < G / 8; ++c) dst[c] = make_uint4(d[4 * c], d[4 * c + 1], d[4 * c + 2], d[4 * c + 3]);
    }
  };

  const int nk = (p.ng + 1) / 2;
  if (nk > 0) {
    load_tile(0);
    store_tile(0);
  }
  __syncthreads();

  const int frag_row = lane & 31, frag_k = 8 * (lane >> 5);
  for (int kt = 0; kt < nk; ++kt) {
    const int s = kt & 1;
    if (kt + 1 < nk) load_tile(kt + 1);
    const uint16_t* at = a_tile(s) + (wm0 + frag_row) * LDA + frag_k;
    const uint16_t* wt = w_tile(s) + (wn0 + frag_row) * LDA + frag_k;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      half8_t af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *reinterpret_cast<const half8_t*>(at + i * 32 * LDA + ks * 16);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bf[j] = *reinterpret_cast<const half8_t*>(wt + j * 32 * LDA + ks * 16);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) store_tile(s ^ 1);
    __syncthreads();
  }

  // ---- epilogue: D[i][j] of a 32x32 tile sits in lane (j + 32*((i/4)%2)), register 4*(i/8) + i%4
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + wn0 + j * 32 + (lane & 31);
      const float b = (p.bias != nullptr && col < p.N) ? h2f(p.bias[col]) : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm0 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (row < seg_hi && col < p.N) {
          const int64_t o = static_cast<int64_t>(row) * p.N + col;
          const float v = acc[i][j][r] + b + (p.residual != nullptr ? h2f(p.residual[o]) : 0.f);
          if (p.out_f32) static_cast<float*>(p.y)[o] = v;
          else static_cast<uint16_t*>(p.y)[o] = f2h(v);
        }
      }
    }
  }
}

template <int BITS, int BM, int BN, int WM, int WN>
static hipError_t launch_cfg(const GemmParams& p, hipStream_t s) {
  constexpr int BK = 2 * GemmTraits<BITS>::G;
  constexpr int LDA = BK + 8;
  constexpr size_t lds = size_t(2) * (BM + BN) * LDA * 2;
  auto kern = gemm_kernel<BITS, BM, BN, WM, WN>;
  if (lds > 65536) {
    const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kern));
    if (e != hipSuccess) return e;
  }
  const int m_tiles = p.indptr ? (p.rows + BM - 1) / BM + p.num_experts : (p.rows + BM - 1) / BM;
  const dim3 grid((p.N + BN - 1) / BN, m_tiles);
  note_kernel("gq::gemm_kernel<%d,%d,%d,%d,%d>", BITS, BM, BN, WM, WN);
  hipLaunchKernelGGL(kern, grid, dim3(64 * (BM / WM) * (BN / WN)), lds, s, p);
  return hipGetLastError();
}

hipError_t launch_gemm(const GemmArgs& a, hipStream_t s) {
  GemmParams p;
  p.x = a.x; p.qw = a.q_weight; p.qs = a.q_scale; p.bias = a.bias; p.residual = a.residual; p.y = a.y;
  p.indptr = a.indptr; p.indptr_i64 = a.indptr_i64;
  p.rows = static_cast<int>(a.rows); p.N = static_cast<int>(a.N); p.K = static_cast<int>(a.K);
  p.ng = static_cast<int>((a.K + a.group_size - 1) / a.group_size);
  p.nw = 4 * p.ng;
  p.expert_w_stride = a.N * p.nw;
  p.expert_s_stride = a.N * p.ng;
  p.num_experts = static_cast<int>(a.num_experts);
  p.out_f32 = a.out_f32;
  p.partial = nullptr;
  p.kt_per_split = 1 << 28;  // one workgroup walks all of K
  p.bm_hint = 0;
  p.paired = a.paired;
  p.x_rows = a.x_rows; p.x_src_rows = static_cast<int>(a.x_src_rows);
  p.bf16 = a.bf16;
  {
    const int64_t x_rows_total = a.x_rows != nullptr ? a.x_src_rows : a.rows;
    const int64_t limit = int64_t(1) << 32;
    // (q3f16_1 handles a last K tile that reaches past K inside that form: 80-wide tiles divide no power of two)
    const bool k_ok = a.bits == 3 ? a.K % 8 == 0 : a.K % (2 * a.group_size) == 0;
    p.fast_ok = k_ok && x_rows_total * a.K * 2 < limit && a.N * p.nw * 4 < limit &&
                options().gemm_fast_loop != 0;  // (tuning / test override: general loop only)
    p.x_bytes = p.fast_ok ? static_cast<uint32_t>(x_rows_total * a.K * 2) : 0u;
  }
  if (a.rows == 0 || a.N == 0) return hipSuccess;
  const int variant = options().gemm_variant;
  if (variant < 0 || a.bf16) {
    const SplitPlan plan = plan_split_k(a.rows, a.N, a.K, a.bits, a.group_size, a.indptr != nullptr);
    p.bm_hint = plan.bm;
    const int64_t need = static_cast<int64_t>(plan.split) * a.rows * a.N * 4;
    // without (enough) scratch the same tiles run unsplit: slower, never wrong
    // (fused gate/up form: the partial sums keep the tile's column order, which only lines up with
    //  rows of N floats when the gate half is whole 32-row blocks)
    if (plan.bm > 0 && plan.split > 1 && a.workspace != nullptr && a.workspace_bytes >= need &&
        (reinterpret_cast<uintptr_t>(a.workspace) & 15) == 0 && (!a.paired || (a.N % 64) == 0)) {
      p.partial = static_cast<float*>(a.workspace);
      p.kt_per_split = plan.kt_per_split;
    }
  }
  if (a.bf16 || (variant != 3 && variant != 4 && variant != 5)) {
    const hipError_t e = launch_gemm_pipe(p, a.bits, s);
    if (e == hipSuccess && p.partial != nullptr) {
      const int64_t count = a.rows * a.N;
      const int nk = (p.ng + 1) / 2;
      const int split = (nk + p.kt_per_split - 1) / p.kt_per_split;
      int64_t blocks = (count / 4 + 255) / 256;
      blocks = blocks < 1 ? 1 : (blocks > 2048 ? 2048 : blocks);
      if (p.paired) {
        hipLaunchKernelGGL(splitk_reduce_silu_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s,
                           p.partial, split, a.rows, p.N, gemm_pipe_pair_block(p, a.bits),
                           static_cast<uint16_t*>(p.y), p.bf16);
        return hipGetLastError();
      }
      hipLaunchKernelGGL(splitk_reduce_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s,
                         p.partial, split, count, p.N, p.bias, p.residual, p.y, p.out_f32, p.bf16);
      return hipGetLastError();
    }
    if (e != hipErrorNotSupported || a.bf16) return e;  // (bfloat16 models: the pipelined kernel or nothing)
  }
  if (p.paired) return hipErrorNotSupported;  // the fused form exists in the pipelined kernel only
  if (a.bits == 4) {
    // big tile (256 x 256, 128 x 128 per wave) once there are enough tiles to fill 256 CUs
    const int64_t big_tiles = ((a.rows + 255) / 256) * ((a.N + 255) / 256);
    const bool big = variant == 4 ? true : (variant == 3 ? false : (a.indptr == nullptr && big_tiles >= 128));
    if (variant == 5) return launch_cfg<4, 256, 256, 128, 128>(p, s);
    if (big) return launch_cfg<4, 256, 256, 128, 64>(p, s);
    return launch_cfg<4, 128, 128, 64, 64>(p, s);
  }
  return launch_cfg<3, 128, 128, 64, 64>(p, s);
}

int64_t gemm_workspace_bytes(int64_t rows, int64_t N, int64_t K, int bits, int group_size) {
  if (options().gemm_variant >= 0) return 0;
  const SplitPlan plan = plan_split_k(rows, N, K, bits, group_size, false);
  return plan.bm > 0 && plan.split > 1 ? static_cast<int64_t>(plan.split) * rows * N * 4 : 0;
}

}  // namespace gq
