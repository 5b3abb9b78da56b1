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
  const uint16_t* residual;  // [rows, N] or null
  void* y;
  const void* indptr;  // null: one segment [0, rows)
  int64_t expert_w_stride, expert_s_stride;
  int rows, N, K, ng, nw;
  int indptr_i64, out_f32;
  int paired;  // fused gate/up form: columns walk gate 0, up 0, gate 1, ...; y is [rows, N / 2] fp16
  const int32_t* x_rows;  // null, or the row of x each activation row reads (int32 [rows])
  int x_src_rows;
};


// Fused gate/up store of a 16 x 16 result tile: lane c holds column `col` for the batch rows 4j .. 4j+3,
// and columns col, col + 1 (lanes c, c ^ 1) are the gate and the up projection of output element col / 2.
// Every lane must arrive here: the neighbour's values come over a DPP swap.
__device__ __forceinline__ void store_gate_up(const SkinnyParams& p, const float4_t v, int col, int c, int j,
                                              int m0, int m_valid) {
  float up[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) up[r] = dpp_f<0xB1>(v[r]);  // quad_perm [1,0,3,2]
  if ((c & 1) == 0 && col < p.N) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int b = 4 * j + r;
      if (b < m_valid)
        static_cast<uint16_t*>(p.y)[static_cast<int64_t>(m0 + b) * (p.N >> 1) + (col >> 1)] =
            silu_mul_h(v[r], up[r]);
    }
  }
}

// Unpipelined form: one chunk at a time, few registers, many workgroups per CU.  Large N hides
// latency with occupancy and runs this one; small N has too few workgroups for that and runs the
// chunk-pipelined kernel below.
template <int MR, int RT>
__global__ __launch_bounds__(256) void skinny_q4_simple_kernel(const SkinnyParams p) {
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
    int row = min(n0 + rt * 16 + c, p.N - 1);  // clamped rows are computed and dropped
    if (p.paired) row = gate_up_row(row, p.N);
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
        const uint16_t* src = p.x + x_row(p.x_rows, p.x_src_rows, m0 + b) * p.K + k;
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
    if (p.paired) {  // uniform
      store_gate_up(p, v, col, c, j, m0, m_valid);
      continue;
    }
    if (col < p.N) {
      const float bias = p.bias != nullptr ? h2f(p.bias[col]) : 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int b = 4 * j + r;
        if (b < m_valid) {
          const int64_t oi = static_cast<int64_t>(m0 + b) * p.N + col;
          const float o = v[r] + bias + (p.residual != nullptr ? h2f(p.residual[oi]) : 0.f);
          if (p.out_f32) static_cast<float*>(p.y)[oi] = o;
          else static_cast<uint16_t*>(p.y)[oi] = f2h(o);
        }
      }
    }
  }
}

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
    int row = min(n0 + rt * 16 + c, p.N - 1);  // clamped rows are computed and dropped
    if (p.paired) row = gate_up_row(row, p.N);
    wrow[rt] = qw + static_cast<int64_t>(row) * p.nw;
    srow[rt] = qs + static_cast<int64_t>(row) * p.ng;
  }
  const bool k_vec = (p.K & 7) == 0;
  const half2_t off = {static_cast<_Float16>(-1031.0f), static_cast<_Float16>(-1031.0f)};

  // ---- per-thread x staging slots (16-byte chunks of the [MR][KC] tile)
  constexpr int XS = MR * (KC / 8) / 256;
  static_assert(MR * (KC / 8) % 256 == 0, "x tile / thread mismatch");
  int x_b[XS], x_kk[XS];
  const uint16_t* x_src[XS];
#pragma unroll
  for (int i = 0; i < XS; ++i) {
    const int idx = tid + 256 * i;
    x_b[i] = idx / (KC / 8);
    x_kk[i] = (idx - x_b[i] * (KC / 8)) * 8;
    x_src[i] = p.x + x_row(p.x_rows, p.x_src_rows, m0 + (x_b[i] < m_valid ? x_b[i] : 0)) * p.K + x_kk[i];
  }
  uint4 xreg[XS];
  // branch-free chunk loads (clamped address; validity is applied when the chunk is stored)
  auto load_x = [&](int ci) {
#pragma unroll
    for (int i = 0; i < XS; ++i) {
      const int k = ci * KC + x_kk[i];
      const bool ok = k_vec && k + 8 <= p.K;
      xreg[i] = *reinterpret_cast<const uint4*>(ok ? x_src[i] + ci * KC : x_src[i] - x_kk[i]);
    }
  };
  auto store_x = [&](int ci) {
#pragma unroll
    for (int i = 0; i < XS; ++i) {
      const int k = ci * KC + x_kk[i];
      uint4 v = xreg[i];
      if (!(k_vec && k + 8 <= p.K && x_b[i] < m_valid)) v = make_uint4(0, 0, 0, 0);
      if (!k_vec && x_b[i] < m_valid && k < p.K) {  // unaligned rows: element-wise, rare
        const uint16_t* src = p.x + x_row(p.x_rows, p.x_src_rows, m0 + x_b[i]) * p.K + k;
        uint16_t e[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) e[q] = (k + q < p.K) ? src[q] : uint16_t(0);
        v.x = e[0] | (uint32_t(e[1]) << 16); v.y = e[2] | (uint32_t(e[3]) << 16);
        v.z = e[4] | (uint32_t(e[5]) << 16); v.w = e[6] | (uint32_t(e[7]) << 16);
      }
      // natural (0,1)(2,3)(4,5)(6,7) -> (0,4)(1,5)(2,6)(3,7)
      uint4 o;
      o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
      o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
      o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
      o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
      *reinterpret_cast<uint4*>(xs + x_b[i] * LDX + x_kk[i]) = o;
    }
  };

  // ---- weight groups of one chunk for this wave; branch-free, a group past the end gets scale +0
  struct WStage {
    uint4 w[RT][STEPS];
    uint32_t s[RT][STEPS];  // fp16 bits, 32 bits wide while in flight
  };
  WStage wa, wb;
  auto load_w = [&](int ci, WStage& st) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int g = ci * KCG + (wave * STEPS + s) * 4 + j;
      const int gc = g < p.ng ? g : 0;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        st.w[rt][s] = *reinterpret_cast<const uint4*>(wrow[rt] + 4 * gc);
        st.s[rt][s] = srow[rt][gc];
      }
    }
  };
  // 4 MFMAs per step: word m of every lane's group against the matching x slice
  auto compute = [&](int ci, const WStage& st) {
    const uint16_t* xa = xs + (c < MR ? c : 0) * LDX + (wave * STEPS * 4 + j) * 32;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      half8_t af[4];
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        af[m] = *reinterpret_cast<const half8_t*>(xa + s * 128 + 8 * m);
        if (c >= MR) af[m] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      }
      const bool ok = ci * KCG + (wave * STEPS + s) * 4 + j < p.ng;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const uint32_t w4[4] = {st.w[rt][s].x, st.w[rt][s].y, st.w[rt][s].z, st.w[rt][s].w};
        const _Float16 sc = __builtin_bit_cast(_Float16, ok ? static_cast<uint16_t>(st.s[rt][s]) : uint16_t(0));
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
  };

  // ---- chunk pipeline: weights and x of chunk c+1 are in flight while chunk c is multiplied
  const int nchunks = (p.ng + KCG - 1) / KCG;
  load_w(0, wa);
  load_x(0);
  load_w(1, wb);
  store_x(0);
  __syncthreads();
  for (int ci = 0; ci < nchunks; ci += 2) {
    load_x(ci + 1);
    compute(ci, wa);
    load_w(ci + 2, wa);
    __syncthreads();  // everyone is done reading x(ci)
    store_x(ci + 1);
    __syncthreads();
    load_x(ci + 2);
    compute(ci + 1, wb);  // a chunk past the end has zero scales and zero x: adds nothing
    load_w(ci + 3, wb);
    __syncthreads();
    store_x(ci + 2);
    __syncthreads();
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
    if (p.paired) {  // uniform
      store_gate_up(p, v, col, c, j, m0, m_valid);
      continue;
    }
    if (col < p.N) {
      const float bias = p.bias != nullptr ? h2f(p.bias[col]) : 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int b = 4 * j + r;
        if (b < m_valid) {
          const int64_t oi = static_cast<int64_t>(m0 + b) * p.N + col;
          const float o = v[r] + bias + (p.residual != nullptr ? h2f(p.residual[oi]) : 0.f);
          if (p.out_f32) static_cast<float*>(p.y)[oi] = o;
          else static_cast<uint16_t*>(p.y)[oi] = f2h(o);
        }
      }
    }
  }
}

// Persistent form for activations that fit LDS whole (M rows x K): x is staged once, then every
// wave walks its own row tiles over the full K with no barrier and no cross-wave reduction, eight
// steps (32 groups per weight row) of 128-bit loads in flight while the previous eight are
// multiplied.  (tile, k-block) pairs form one flat sequence per wave, so the prefetch runs across
// tile boundaries.  All loads are branch-free; a step past the end reads one cached line and gets
// scale +0.
template <int MR>
__global__ __launch_bounds__(512) void skinny_q4_persist_kernel(const SkinnyParams p, int ntiles, int nblk) {
  constexpr int SB = 8;  // steps per k-block (4 groups each)
  constexpr uint32_t kMagic = 0x64006400u;
  extern __shared__ uint4 smem[];
  uint16_t* xs = reinterpret_cast<uint16_t*>(smem);
  const int kpad = nblk * SB * 128;
  const int ldx = kpad + 8;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, j = lane >> 4;

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
  if (m0 >= seg_hi) return;  // uniform
  const int m_valid = min(16, seg_hi - m0);
  const uint32_t* qw = p.qw + expert * p.expert_w_stride;
  const uint16_t* qs = p.qs + expert * p.expert_s_stride;

  const int wpb = blockDim.x >> 6;
  const int gw = blockIdx.x * wpb + wave;
  const int nwaves = gridDim.x * wpb;
  const int my_tiles = gw < ntiles ? (ntiles - gw + nwaves - 1) / nwaves : 0;
  const int total = my_tiles * nblk;  // (tile, k-block) pairs of this wave

  struct WStage {
    uint4 w[SB];
    uint32_t s[SB];
  };
  WStage wa, wb;
  // sequence cursor of the issue side: (tile, blk) advance without division or branches
  int i_tile = gw, i_blk = 0, i_seq = 0;
  auto issue = [&](WStage& st) {
    const bool live = i_seq < total;
    int row = min(i_tile * 16 + c, p.N - 1);
    if (p.paired) row = gate_up_row(row, p.N);
    const uint32_t* wr = qw + static_cast<int64_t>(row) * p.nw;
    const uint16_t* sr = qs + static_cast<int64_t>(row) * p.ng;
#pragma unroll
    for (int s = 0; s < SB; ++s) {
      const int g = (i_blk * SB + s) * 4 + j;
      const bool ok = live && g < p.ng;
      st.w[s] = *reinterpret_cast<const uint4*>(ok ? wr + 4 * g : qw);
      st.s[s] = *(ok ? sr + g : qs);
    }
    ++i_seq;
    const bool wrap = i_blk + 1 == nblk;
    i_blk = wrap ? 0 : i_blk + 1;
    i_tile = wrap ? i_tile + nwaves : i_tile;
  };
  issue(wa);
  issue(wb);

  // ---- stage x[m0 .. m0+MR, 0 .. kpad) in pair order, zero beyond K and beyond the segment
  {
    const bool k_vec = (p.K & 7) == 0;
    const int cpr = kpad / 8;
    for (int i = tid; i < MR * cpr; i += blockDim.x) {
      const int b = i / cpr;
      const int k = (i - b * cpr) * 8;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (b < m_valid && k < p.K) {
        const uint16_t* src = p.x + x_row(p.x_rows, p.x_src_rows, m0 + b) * p.K + k;
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
      uint4 o;
      o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
      o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
      o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
      o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
      *reinterpret_cast<uint4*>(xs + b * ldx + k) = o;
    }
  }
  __syncthreads();

  const half2_t off = {static_cast<_Float16>(-1031.0f), static_cast<_Float16>(-1031.0f)};
  const uint16_t* xa = xs + (c < MR ? c : 0) * ldx + j * 32;
  float4_t acc = {0.f, 0.f, 0.f, 0.f};
  int c_tile = gw, c_blk = 0;  // cursor of the compute side
  auto compute = [&](const WStage& st) {
#pragma unroll
    for (int s = 0; s < SB; ++s) {
      const int g = (c_blk * SB + s) * 4 + j;
      const uint16_t* xp = xa + (c_blk * SB + s) * 128;
      half8_t af[4];
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        af[m] = *reinterpret_cast<const half8_t*>(xp + 8 * m);
        if (c >= MR) af[m] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      }
      const uint32_t w4[4] = {st.w[s].x, st.w[s].y, st.w[s].z, st.w[s].w};
      const _Float16 sc = __builtin_bit_cast(_Float16, g < p.ng ? static_cast<uint16_t>(st.s[s]) : uint16_t(0));
      const half2_t s2 = {sc, sc};
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        uint32_t d[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t h = and_or(w4[m] >> (4 * i), 0x000f000fu, kMagic);
          d[i] = as_u32((as_half2(h) + off) * s2);
        }
        const uint4 dv = make_uint4(d[0], d[1], d[2], d[3]);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[m], __builtin_bit_cast(half8_t, dv), acc, 0, 0, 0);
      }
    }
    // last k-block of a tile: store D[b][n] for b < m_valid, start the next tile
    if (c_blk + 1 == nblk) {
      const int col = c_tile * 16 + c;
      if (p.paired) {  // uniform
        store_gate_up(p, acc, col, c, j, m0, m_valid);
      } else if (col < p.N) {
        const float bias = p.bias != nullptr ? h2f(p.bias[col]) : 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int b = 4 * j + r;
          if (b < m_valid) {
            const int64_t oi = static_cast<int64_t>(m0 + b) * p.N + col;
            const float o = acc[r] + bias + (p.residual != nullptr ? h2f(p.residual[oi]) : 0.f);
            if (p.out_f32) static_cast<float*>(p.y)[oi] = o;
            else static_cast<uint16_t*>(p.y)[oi] = f2h(o);
          }
        }
      }
      acc = float4_t{0.f, 0.f, 0.f, 0.f};
      c_blk = 0;
      c_tile += nwaves;
    } else {
      ++c_blk;
    }
  };
  for (int seq = 0; seq < total; seq += 2) {
    compute(wa);
    issue(wa);
    if (seq + 1 < total) compute(wb);
    issue(wb);
  }
}

template <int MR, int RT>
static hipError_t launch_skinny_cfg(const SkinnyParams& p, int experts, int mtiles, bool pipelined,
                                    hipStream_t s) {
  constexpr int KCG = MR <= 8 ? 64 : 32;
  constexpr size_t lds_x = size_t(MR) * (KCG * 32 + 8) * 2;
  constexpr size_t lds_red = size_t(4) * RT * 64 * 16;
  constexpr size_t lds = lds_x > lds_red ? lds_x : lds_red;
  static_assert(lds <= 65536, "LDS budget");
  const dim3 grid((p.N + 16 * RT - 1) / (16 * RT), experts, mtiles);
  note_kernel(pipelined ? "gq::skinny_q4_kernel<%d,%d>" : "gq::skinny_q4_simple_kernel<%d,%d>", MR, RT);
  if (pipelined) hipLaunchKernelGGL((skinny_q4_kernel<MR, RT>), grid, dim3(256), lds, s, p);
  else hipLaunchKernelGGL((skinny_q4_simple_kernel<MR, RT>), grid, dim3(256), lds, s, p);
  return hipGetLastError();
}

// rows_max: largest number of activation rows any segment holds (M for a plain linear)
hipError_t launch_skinny(const GemmArgs& a, int rows_max, hipStream_t s) {
  if (a.bits != 4 || (a.paired && (a.N & 1))) return hipErrorNotSupported;
  SkinnyParams p;
  p.x = a.x; p.qw = a.q_weight; p.qs = a.q_scale; p.bias = a.bias; p.residual = a.residual; p.y = a.y;
  p.indptr = a.indptr; p.indptr_i64 = a.indptr_i64;
  p.rows = static_cast<int>(a.rows); p.N = static_cast<int>(a.N); p.K = static_cast<int>(a.K);
  p.ng = static_cast<int>((a.K + a.group_size - 1) / a.group_size);
  p.nw = 4 * p.ng;
  p.expert_w_stride = a.N * p.nw;
  p.expert_s_stride = a.N * p.ng;
  p.out_f32 = a.out_f32;
  p.paired = a.paired;
  p.x_rows = a.x_rows; p.x_src_rows = static_cast<int>(a.x_src_rows);
  if (a.rows == 0 || a.N == 0) return hipSuccess;
  const int experts = a.indptr ? static_cast<int>(a.num_experts) : 1;
  const int mtiles = (rows_max + 15) / 16;
  const int mr = rows_max <= 4 ? 4 : (rows_max <= 8 ? 8 : 16);
  // row tiles per workgroup: enough workgroups for 256 CUs first, then fewer re-reads of x
  const int64_t tiles = (a.N + 15) / 16 * experts * mtiles;
  // Measured: below ~800 row tiles the chunk-pipelined kernel (one tile per workgroup) wins, above
  // it the unpipelined one with 2-4 tiles per workgroup (occupancy hides the latency instead).
  const int mode = options().gemv_variant;  // tuning override: 2 simple, 3 pipelined, 4 persistent, 5 never persistent
  // persistent kernel whenever the activations fit LDS whole (k padded to 1024)
  {
    const int nblk = (p.ng + 31) / 32;
    const size_t lds_p = static_cast<size_t>(mr) * (static_cast<size_t>(nblk) * 1024 + 8) * 2;
    const size_t lds_cap = 144 * 1024;
    const int64_t tiles_all = (static_cast<int64_t>(p.N) + 15) / 16;
    if (mode != 2 && mode != 3 && mode != 5 && lds_p <= lds_cap && (mode == 4 || tiles_all >= 4096)) {
      const int ntiles = (p.N + 15) / 16;
      int waves = options().gemv_waves > 0 ? options().gemv_waves : 2048;
      waves = (waves + experts * mtiles - 1) / (experts * mtiles);
      const int rounds = (ntiles + waves - 1) / waves;
      const int wpb = options().gemv_rows_per_wave == 4 ? 4 : 8;  // waves per workgroup (8 unless tuning says 4)
      const int blocks = ((ntiles + rounds - 1) / rounds + wpb - 1) / wpb;
      const dim3 grid(blocks, experts, mtiles);
      auto launch = [&](auto kern) -> hipError_t {
        if (lds_p > 65536) {
          const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kern));
          if (e != hipSuccess) return e;
        }
        note_kernel("gq::skinny_q4_persist_kernel<%d>", mr);
        hipLaunchKernelGGL(kern, grid, dim3(64 * wpb), lds_p, s, p, ntiles, nblk);
        return hipGetLastError();
      };
      if (mr == 4) return launch(skinny_q4_persist_kernel<4>);
      if (mr == 8) return launch(skinny_q4_persist_kernel<8>);
      return launch(skinny_q4_persist_kernel<16>);
    }
  }
  // (a sweep over 7B..70B projection shapes put the hand-over between 640 and 960 tiles: 70B qkv, 640 tiles,
  //  27.5 us pipelined against 30-36 unpipelined; 13B qkv, 960 tiles, 29.4 against 24.1-24.9; and four row tiles
  //  per workgroup from about 3000 tiles on: 70B gate_up 98-106 us against 107-113 with two)
  const bool pipelined = mode == 3 ? true : (mode == 2 ? false : tiles < 800);
  int rt = options().gemv_rows_per_wave;  // tuning override
  if (rt != 1 && rt != 2 && rt != 4) rt = pipelined ? 1 : (tiles >= 3072 ? 4 : 2);
  if (mr == 4) {
    if (rt == 4) return launch_skinny_cfg<4, 4>(p, experts, mtiles, pipelined, s);
    if (rt == 2) return launch_skinny_cfg<4, 2>(p, experts, mtiles, pipelined, s);
    return launch_skinny_cfg<4, 1>(p, experts, mtiles, pipelined, s);
  }
  if (mr == 8) {
    if (rt == 4) return launch_skinny_cfg<8, 4>(p, experts, mtiles, pipelined, s);
    if (rt == 2) return launch_skinny_cfg<8, 2>(p, experts, mtiles, pipelined, s);
    return launch_skinny_cfg<8, 1>(p, experts, mtiles, pipelined, s);
  }
  if (rt == 4) return launch_skinny_cfg<16, 4>(p, experts, mtiles, pipelined, s);
  if (rt == 2) return launch_skinny_cfg<16, 2>(p, experts, mtiles, pipelined, s);
  return launch_skinny_cfg<16, 1>(p, experts, mtiles, pipelined, s);
}

}  // namespace gq
