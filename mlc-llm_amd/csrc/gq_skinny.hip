// Skinny matmul on MFMA for q4f16_1: 3..16 activation rows against streamed weights.
//
// Replaces the low-batch GEMV buckets the reference schedules for 2 < M <= 8
// (python/mlc_llm/compiler_pass/low_batch_specialization.py:22-57) and the small-segment case of
// moe_matmul.dequantize_group_gemm (python/mlc_llm/op/moe_matmul.py:562-768), where an expert
// sees only a handful of tokens and the layer is bound by streaming the experts' weights.
//
// Still HBM-bound, but with more than two activation rows a per-row dot product would spend more
// VALU issue slots than the weight stream leaves, so the products go to the matrix core:
// v_mfma_f32_16x16x32_f16 computes D[b][n] += sum_k X[b][k] * W[n][k] for 16 batch rows (the rows
// past M are zero) x 16 weight rows x 32 k.  Lane (c = lane % 16, j = lane / 16) supplies 8
// consecutive k of weight row c, i.e. exactly one uint32 storage word, so:
//  * per step a lane loads ONE 128-bit group (row c, group 4q + j) and its scale, and feeds four
//    MFMAs, the m-th taking word m of every lane's group; the k order inside a word is the pair
//    order (0,4)(1,5)(2,6)(3,7) that the masks produce, and x is staged in LDS in that same order;
//  * words are dequantised the way the reference does ((q - 7) exactly, one fp16 multiply by
//    the scale) because one MFMA mixes four groups and cannot be rescaled afterwards;
//  * a workgroup owns RT tiles of 16 weight rows; its 4 waves split every K chunk four ways and
//    add their accumulators through LDS at the end;
//  * x (M rows, zero padded to MR in {4, 8, 16}) is staged chunk by chunk, rows padded by 16 bytes
//    so that the 16 lanes of a k slice read 16 distinct bank groups.
#include "gq_common.hpp"
#include "gq_internal.hpp"

namespace gq {

struct SkinnyParams {
  const uint16_t* x;
  const uint32_t* qw;
  const uint16_t* qs;
  const uint16_t* bias;
  void* y;
  const void* indptr;  // null: one segment [0, rows)
  int64_t expert_w_stride, expert_s_stride;
  int rows, N, K, ng, nw;
  int indptr_i64, out_f32;
};

template <int MR, int RT>
__global__ __launch_bounds__(256) void skinny_q4_kernel(const SkinnyParams p) {
  constexpr int KCG = MR <= 8 ? 64 : 32;  // groups per staged chunk
  constexpr int KC = KCG * 32;            // k per chunk
  constexpr int LDX = KC + 8;             // halves per staged x row (16-byte pad)
  constexpr int STEPS = KCG / 16;         // steps (4 groups each) per wave per chunk
  constexpr uint32_t kMagic = 0x64006400u;

  extern __shared__ uint4 smem[];
  uint16_t* xs = reinterpret_cast<uint16_t*>(smem);

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, j = lane >> 4;

  // ---- segment of activation rows and the expert they meet
  int seg_lo = 0, seg_hi = p.rows;
  const int expert = blockIdx.y;
  if (p.indptr != nullptr) {
    int64_t lo, hi;
    if (p.indptr_i64) {
      lo = static_cast<const int64_t*>(p.indptr)[expert];
      hi = static_cast<const int64_t*>(p.indptr)[expert + 1];
    } else {
      lo = static_cast<const int32_t*>(p.indptr)[expert];
      hi = static_cast<const int32_t*>(p.indptr)[expert + 1];
    }
    lo = lo < 0 ? 0 : (lo > p.rows ? p.rows : lo);
    hi = hi < lo ? lo : (hi > p.rows ? p.rows : hi);
    seg_lo = static_cast<int>(lo);
    seg_hi = static_cast<int>(hi);
  }
  const int m0 = seg_lo + blockIdx.z * 16;
  if (m0 >= seg_hi) return;  // uniform: this expert has no (more) rows
  const int m_valid = min(16, seg_hi - m0);
  const uint32_t* qw = p.qw + expert * p.expert_w_stride;
  const uint16_t* qs = p.qs + expert * p.expert_s_stride;
  const int n0 = blockIdx.x * (16 * RT);

  float4_t acc[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) acc[rt] = float4_t{0.f, 0.f, 0.f, 0.f};

  const uint32_t* wrow[RT];
  const uint16_t* srow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = min(n0 + rt * 16 + c, p.N - 1);  // clamped rows are computed and dropped
    wrow[rt] = qw + static_cast<int64_t>(row) * p.nw;
    srow[rt] = qs + static_cast<int64_t>(row) * p.ng;
  }
  const bool k_vec = (p.K & 7) == 0;
  const half2_t off = {static_cast<_Float16>(-1031.0f), static_cast<_Float16>(-1031.0f)};

  const int nchunks = (p.ng + KCG - 1) / KCG;
  for (int ci = 0; ci < nchunks; ++ci) {
    // ---- this wave's weight groups of the chunk: all loads go out before x is touched
    uint4 wreg[RT][STEPS];
    uint32_t sreg[RT][STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int g = ci * KCG + (wave * STEPS + s) * 4 + j;
      const bool ok = g < p.ng;
      const int gc = ok ? g : p.ng - 1;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        wreg[rt][s] = *reinterpret_cast<const uint4*>(wrow[rt] + 4 * gc);
        sreg[rt][s] = ok ? static_cast<uint32_t>(srow[rt][gc]) : 0u;  // +0.0 scale: group adds nothing
      }
    }

    // ---- stage x[m0 .. m0+MR, chunk] in pair order; zero beyond K and beyond the segment
    if (ci > 0) __syncthreads();
    for (int i = tid; i < MR * (KC / 8); i += 256) {
      const int b = i / (KC / 8);
      const int kk = (i - b * (KC / 8)) * 8;
      const int k = ci * KC + kk;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (b < m_valid && k < p.K) {
        const uint16_t* src = p.x + static_cast<int64_t>(m0 + b) * p.K + k;
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
      // natural (0,1)(2,3)(4,5)(6,7) -> (0,4)(1,5)(2,6)(3,7)
      uint4 o;
      o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
      o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
      o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
      o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
      *reinterpret_cast<uint4*>(xs + b * LDX + kk) = o;
    }
    __syncthreads();

    // ---- 4 MFMAs per step: word m of every lane's group against the matching x slice
    const uint16_t* xa = xs + (c < MR ? c : 0) * LDX + (wave * STEPS * 4 + j) * 32;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      half8_t af[4];
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        af[m] = *reinterpret_cast<const half8_t*>(xa + s * 128 + 8 * m);
        if (c >= MR) af[m] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const uint32_t w4[4] = {wreg[rt][s].x, wreg[rt][s].y, wreg[rt][s].z, wreg[rt][s].w};
        const _Float16 sc = __builtin_bit_cast(_Float16, static_cast<uint16_t>(sreg[rt][s]));
        const half2_t s2 = {sc, sc};
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          uint32_t d[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t h = and_or(w4[m] >> (4 * i), 0x000f000fu, kMagic);  // (1024+q_i, 1024+q_{i+4})
            d[i] = as_u32((as_half2(h) + off) * s2);
          }
          const uint4 dv = make_uint4(d[0], d[1], d[2], d[3]);
          acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[m], __builtin_bit_cast(half8_t, dv),
                                                           acc[rt], 0, 0, 0);
        }
      }
    }
  }

  // ---- add the four waves' accumulators through LDS, then store D[b][n] for b < m_valid
  __syncthreads();
  float4_t* red = reinterpret_cast<float4_t*>(smem);
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) red[(wave * RT + rt) * 64 + lane] = acc[rt];
  __syncthreads();
  for (int rt = wave; rt < RT; rt += 4) {
    float4_t v = red[rt * 64 + lane];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      const float4_t o = red[(w * RT + rt) * 64 + lane];
      v[0] += o[0]; v[1] += o[1]; v[2] += o[2]; v[3] += o[3];
    }
    const int col = n0 + rt * 16 + c;
    if (col < p.N) {
      const float bias = p.bias != nullptr ? h2f(p.bias[col]) : 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int b = 4 * j + r;
        if (b < m_valid) {
          const int64_t oi = static_cast<int64_t>(m0 + b) * p.N + col;
          const float o = v[r] + bias;
          if (p.out_f32) static_cast<float*>(p.y)[oi] = o;
          else static_cast<uint16_t*>(p.y)[oi] = f2h(o);
        }
      }
    }
  }
}

template <int MR, int RT>
static hipError_t launch_skinny_cfg(const SkinnyParams& p, int experts, int mtiles, hipStream_t s) {
  constexpr int KCG = MR <= 8 ? 64 : 32;
  constexpr size_t lds_x = size_t(MR) * (KCG * 32 + 8) * 2;
  constexpr size_t lds_red = size_t(4) * RT * 64 * 16;
  constexpr size_t lds = lds_x > lds_red ? lds_x : lds_red;
  static_assert(lds <= 65536, "LDS budget");
  const dim3 grid((p.N + 16 * RT - 1) / (16 * RT), experts, mtiles);
  hipLaunchKernelGGL((skinny_q4_kernel<MR, RT>), grid, dim3(256), lds, s, p);
  return hipGetLastError();
}

// rows_max: largest number of activation rows any segment holds (M for a plain linear)
hipError_t launch_skinny(const GemmArgs& a, int rows_max, hipStream_t s) {
  if (a.bits != 4) return hipErrorNotSupported;
  SkinnyParams p;
  p.x = a.x; p.qw = a.q_weight; p.qs = a.q_scale; p.bias = a.bias; p.y = a.y;
  p.indptr = a.indptr; p.indptr_i64 = a.indptr_i64;
  p.rows = static_cast<int>(a.rows); p.N = static_cast<int>(a.N); p.K = static_cast<int>(a.K);
  p.ng = static_cast<int>((a.K + a.group_size - 1) / a.group_size);
  p.nw = 4 * p.ng;
  p.expert_w_stride = a.N * p.nw;
  p.expert_s_stride = a.N * p.ng;
  p.out_f32 = a.out_f32;
  if (a.rows == 0 || a.N == 0) return hipSuccess;
  const int experts = a.indptr ? static_cast<int>(a.num_experts) : 1;
  const int mtiles = (rows_max + 15) / 16;
  const int mr = rows_max <= 4 ? 4 : (rows_max <= 8 ? 8 : 16);
  // row tiles per workgroup: enough workgroups for 256 CUs first, then fewer re-reads of x
  const int64_t tiles = (a.N + 15) / 16 * experts * mtiles;
  int rt = options().gemv_rows_per_wave;  // tuning override
  if (rt != 1 && rt != 2 && rt != 4) rt = tiles >= 4096 ? 4 : (tiles >= 1024 ? 2 : 1);
  if (mr == 4) {
    if (rt == 4) return launch_skinny_cfg<4, 4>(p, experts, mtiles, s);
    if (rt == 2) return launch_skinny_cfg<4, 2>(p, experts, mtiles, s);
    return launch_skinny_cfg<4, 1>(p, experts, mtiles, s);
  }
  if (mr == 8) {
    if (rt == 4) return launch_skinny_cfg<8, 4>(p, experts, mtiles, s);
    if (rt == 2) return launch_skinny_cfg<8, 2>(p, experts, mtiles, s);
    return launch_skinny_cfg<8, 1>(p, experts, mtiles, s);
  }
  if (rt == 4) return launch_skinny_cfg<16, 4>(p, experts, mtiles, s);
  if (rt == 2) return launch_skinny_cfg<16, 2>(p, experts, mtiles, s);
  return launch_skinny_cfg<16, 1>(p, experts, mtiles, s);
}

}  // namespace gq
