// KN-layout group-quantized weights (q4f16_0 / q3f16_0 / q4bf16_0 of the reference registry,
// python/mlc_llm/quantization/quantization.py:47-57, 69-79): `quantize_weight(output_transpose=True)` stores the
// transposed tensors (python/mlc_llm/quantization/group_quantization.py:125-130, 299-305),
//   q_weight uint32 [nw, N],  q_scale fp16 [ng, N]
// and GroupQuantizeLinear.forward dequantises along axis 0 and multiplies without a transpose (:404-437).
//
// Here: the two transposes between the layouts (bit moves), the dequantisation to [K, N], and a decode GEMV that
// streams the KN tensors as they are stored.  In KN a row of q_weight holds ONE storage word of every output column,
// so a lane owns four neighbouring columns (one 128-bit load = the same word of four columns, a wave load = 1 KiB
// contiguous) and nothing is reduced across lanes; what has to be split is K: the 4 waves of a workgroup and, on
// matrices with few column blocks, several workgroups share a column block's groups, and their partial sums meet in
// LDS and in the caller's workspace (a second, tiny launch adds them, the bias, and casts).
#include "gq_gemv_common.hpp"

namespace gq {

namespace {

// dst[c][r] = src[r][c] for a dense [rows, cols] matrix of 32-bit (T = uint32_t) or 16-bit (T = uint16_t) elements
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ src, int rows, int cols, T* __restrict__ dst) {
  __shared__ T tile[64][65];
  const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int j = ty; j < 64; j += 4) {
    const int r = r0 + j, c = c0 + tx;
    if (r < rows && c < cols) tile[j][tx] = src[static_cast<int64_t>(r) * cols + c];
  }
  __syncthreads();
  for (int j = ty; j < 64; j += 4) {
    const int c = c0 + j, r = r0 + tx;
    if (r < rows && c < cols) dst[static_cast<int64_t>(c) * rows + r] = tile[tx][j];
  }
}

template <typename T>
hipError_t launch_transpose(const T* src, int64_t rows, int64_t cols, T* dst, hipStream_t s) {
  if (rows == 0 || cols == 0) return hipSuccess;
  const dim3 grid(static_cast<unsigned>((cols + 63) / 64), static_cast<unsigned>((rows + 63) / 64));
  hipLaunchKernelGGL(transpose_kernel<T>, grid, dim3(256), 0, s, src, static_cast<int>(rows), static_cast<int>(cols), dst);
  return hipGetLastError();
}

// out[k][n] = (field k % E of q_weight[k / E][n] - m) * q_scale[k / G][n], k < K: one thread per (word row, column),
// the fp16 subtract and multiply of GroupQuantize._dequantize (group_quantization.py:155-186) with axis = 0
template <int BITS>
__global__ __launch_bounds__(256) void dequantize_kn_kernel(const uint32_t* __restrict__ qw, const uint16_t* __restrict__ qs,
                                                            int N, int K, int nw, uint16_t* __restrict__ out) {
  constexpr int E = Scheme<BITS>::kElem, G = GemvTraits<BITS>::G;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(nw) * N) return;
  const int i = static_cast<int>(idx / N), n = static_cast<int>(idx - static_cast<int64_t>(i) * N);
  const uint32_t w = qw[idx];
  const int k0 = i * E;
  if (k0 >= K) return;
  const _Float16 scale = __builtin_bit_cast(_Float16, qs[static_cast<int64_t>(k0 / G) * N + n]);  // (E divides G)
#pragma unroll
  for (int r = 0; r < E; ++r) {
    if (k0 + r < K) {
      const _Float16 d = static_cast<_Float16>(static_cast<float>((w >> (r * BITS)) & Scheme<BITS>::kMask)) -
                         static_cast<_Float16>(static_cast<float>(Scheme<BITS>::kMaxInt));
      out[static_cast<int64_t>(k0 + r) * N + n] = __builtin_bit_cast(uint16_t, static_cast<_Float16>(d * scale));
    }
  }
}

struct KnParams {
  const uint16_t* x;    // [M, K]
  const uint32_t* qw;   // [nw, N]
  const uint16_t* qs;   // [ng, N]
  const uint16_t* bias; // [N] or null (used when the launch is not split across workgroups)
  void* y;              // [M, N] (fp16 / fp32), or the fp32 partial sums [slices, M, N] when slices > 1
  int N, K, ng, slices, gps;  // gps: groups per slice
  int out_f32;
  int x_vec;  // x rows are 16-byte aligned (K % 8 == 0, aligned base)
};

// grid (column blocks of 256, K slices); a workgroup's 4 waves take the groups of its slice round robin
template <int BITS, int NB>
__global__ __launch_bounds__(256) void gemv_kn_kernel(const KnParams p) {
  constexpr int G = GemvTraits<BITS>::G, CH = GemvTraits<BITS>::CH, HP = G / 2;
  extern __shared__ uint4 smem[];  // x of the slice in pair order [NB][gps][CH] uint4, then corr [NB][gps], then sums
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = blockIdx.x * 256 + lane * 4;  // this lane's four columns
  const int g0 = blockIdx.y * p.gps;
  const int gcount = min(p.gps, p.ng - g0);
  float* const corr_lds = reinterpret_cast<float*>(smem + NB * p.gps * CH);
  float* const sum_lds = corr_lds + ((NB * p.gps + 3) & ~3);  // (16-byte aligned)

  // ---- stage this slice of x: one thread per (row, group), natural order -> pair order + offset term
  for (int q = threadIdx.x; q < NB * gcount; q += 256) {
    const int b = q / gcount, gl = q - b * gcount;
    const int k0 = (g0 + gl) * G;
    uint32_t nat[HP], xr[HP];
    if (p.x_vec) {  // K % 8 == 0 and a 16-byte aligned x: whole 16-byte chunks, inside or outside K
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int k = k0 + 8 * c;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (k + 8 <= p.K) v = *reinterpret_cast<const uint4*>(p.x + static_cast<int64_t>(b) * p.K + k);
        nat[4 * c] = v.x; nat[4 * c + 1] = v.y; nat[4 * c + 2] = v.z; nat[4 * c + 3] = v.w;
      }
    } else {
#pragma unroll
      for (int h = 0; h < HP; ++h) {
        const int k = k0 + 2 * h;
        const uint32_t lo = k < p.K ? p.x[static_cast<int64_t>(b) * p.K + k] : 0u;
        const uint32_t hi = k + 1 < p.K ? p.x[static_cast<int64_t>(b) * p.K + k + 1] : 0u;
        nat[h] = lo | (hi << 16);
      }
    }
    corr_lds[b * p.gps + gl] = permute_group<BITS>(nat, xr);
#pragma unroll
    for (int c = 0; c < CH; ++c)
      smem[(b * p.gps + gl) * CH + c] = make_uint4(xr[4 * c], xr[4 * c + 1], xr[4 * c + 2], xr[4 * c + 3]);
  }
  __syncthreads();

  float acc[NB][4];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[b][c] = 0.f;
  const bool col_ok = n0 < p.N;  // (N is a multiple of 4: a lane's four columns are all inside or all outside)
  const int nc = col_ok ? n0 : 0;
  // one group = 4 word rows; the next group's loads are in flight while this one is multiplied
  uint4 wn[4];
  uint2 sn;
  auto issue = [&](int gl) {
    const int g = g0 + min(gl, gcount - 1);
#pragma unroll
    for (int r = 0; r < 4; ++r)
      wn[r] = *reinterpret_cast<const uint4*>(p.qw + static_cast<int64_t>(4 * g + r) * p.N + nc);
    sn = *reinterpret_cast<const uint2*>(p.qs + static_cast<int64_t>(g) * p.N + nc);
  };
  issue(wave);
  for (int gl = wave; gl < gcount; gl += 4) {
    uint4 wc[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) wc[r] = wn[r];
    const uint2 sc = sn;
    issue(gl + 4);
    const float scale[4] = {h2f(static_cast<uint16_t>(sc.x & 0xffffu)), h2f(static_cast<uint16_t>(sc.x >> 16)),
                            h2f(static_cast<uint16_t>(sc.y & 0xffffu)), h2f(static_cast<uint16_t>(sc.y >> 16))};
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      uint32_t xr[HP];
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const uint4 v = smem[(b * p.gps + gl) * CH + c];  // the same address in every lane: a broadcast
        xr[4 * c] = v.x; xr[4 * c + 1] = v.y; xr[4 * c + 2] = v.z; xr[4 * c + 3] = v.w;
      }
      const float corr = corr_lds[b * p.gps + gl];
      // column c of this lane: its four words of the group sit in the four word rows
      acc[b][0] = fmaf(scale[0], group_dot<BITS>(make_uint4(wc[0].x, wc[1].x, wc[2].x, wc[3].x), xr, corr), acc[b][0]);
      acc[b][1] = fmaf(scale[1], group_dot<BITS>(make_uint4(wc[0].y, wc[1].y, wc[2].y, wc[3].y), xr, corr), acc[b][1]);
      acc[b][2] = fmaf(scale[2], group_dot<BITS>(make_uint4(wc[0].z, wc[1].z, wc[2].z, wc[3].z), xr, corr), acc[b][2]);
      acc[b][3] = fmaf(scale[3], group_dot<BITS>(make_uint4(wc[0].w, wc[1].w, wc[2].w, wc[3].w), xr, corr), acc[b][3]);
    }
  }

  // ---- the four waves' shares meet in LDS: [wave][row][256 columns]
  float4* const sums = reinterpret_cast<float4*>(sum_lds);
#pragma unroll
  for (int b = 0; b < NB; ++b) sums[(wave * NB + b) * 64 + lane] = make_float4(acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
  __syncthreads();
  for (int q = threadIdx.x; q < NB * 64; q += 256) {
    const int b = q >> 6, l = q & 63;
    const int n = blockIdx.x * 256 + l * 4;
    if (n >= p.N) continue;
    float4 v = sums[b * 64 + l];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      const float4 t = sums[(w * NB + b) * 64 + l];
      v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
    }
    if (p.slices > 1) {  // fp32 partial sums [slice][row][N]; the reduction adds the bias
      *reinterpret_cast<float4*>(static_cast<float*>(p.y) + (static_cast<int64_t>(blockIdx.y) * NB + b) * p.N + n) = v;
      continue;
    }
    if (p.bias != nullptr) {
      const uint2 bb = *reinterpret_cast<const uint2*>(p.bias + n);
      v.x += h2f(static_cast<uint16_t>(bb.x & 0xffffu)); v.y += h2f(static_cast<uint16_t>(bb.x >> 16));
      v.z += h2f(static_cast<uint16_t>(bb.y & 0xffffu)); v.w += h2f(static_cast<uint16_t>(bb.y >> 16));
    }
    const int64_t oi = static_cast<int64_t>(b) * p.N + n;
    if (p.out_f32) {
      *reinterpret_cast<float4*>(static_cast<float*>(p.y) + oi) = v;
    } else {
      uint2 o;
      o.x = static_cast<uint32_t>(f2h(v.x)) | (static_cast<uint32_t>(f2h(v.y)) << 16);
      o.y = static_cast<uint32_t>(f2h(v.z)) | (static_cast<uint32_t>(f2h(v.w)) << 16);
      *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.y) + oi) = o;
    }
  }
}

// ---- up to 8 rows on the 4x4x4 matrix instruction.  v_mfma_f32_4x4x4_16b_f16 multiplies 16 independent blocks;
// here a block is 4 neighbouring columns (A rows) x 4 activation rows (B columns) and the 16 blocks of a wave are 16
// different column quads of ONE quantisation group, so nothing is summed across lanes: lane (block q, j) ends with
// y[row j][its block's four columns].  A lane loads one 128-bit piece of one word row (the same word of four columns; a
// wave instruction covers 4 word rows x 256 contiguous bytes); the four lanes of a block then hold word rows 4g .. 4g + 3 of
// the same four columns, and a 4 x 4 transpose inside the lane quad (two exchange steps) leaves every lane with the
// four words, i.e. the whole group, of ONE column - the operand the NK few-row kernels load directly (gq_quadrow.hip),
// whose unpack, operand classes and offset term this kernel shares.  x of the workgroup's K slice sits in LDS in operand
// order; the 16 blocks read the same address (a broadcast).  A wave owns 64 columns and walks every group of the slice.
typedef uint32_t kn_u2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float4_t kn_mfma4(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, float4_t c) {
  const kn_u2 a = {a0, a1}, b = {b0, b1};
  return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, a), __builtin_bit_cast(half4_t, b), c, 0, 0, 0);
}
template <int CTRL>
__device__ __forceinline__ uint32_t kn_dpp(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xf, 0xf, true));
}
// lane i of a quad holds (m[i][0..3]); afterwards it holds (m[0..3][i])
__device__ __forceinline__ uint4 kn_quad_transpose(uint4 v, int lane) {
  const bool odd = (lane & 1) != 0, hi = (lane & 2) != 0;
  uint32_t r = kn_dpp<0xB1>(odd ? v.x : v.y);  // quad_perm [1,0,3,2]
  if (odd) v.x = r; else v.y = r;
  r = kn_dpp<0xB1>(odd ? v.z : v.w);
  if (odd) v.z = r; else v.w = r;
  r = kn_dpp<0x4E>(hi ? v.x : v.z);  // quad_perm [2,3,0,1]
  if (hi) v.x = r; else v.z = r;
  r = kn_dpp<0x4E>(hi ? v.y : v.w);
  if (hi) v.y = r; else v.w = r;
  return v;
}

// grid (column blocks of 256, K slices); NBQ batch quads (rows <= 4 * NBQ)
template <int BITS, int NBQ>
__global__ __launch_bounds__(256) void kn_quad_kernel(const KnParams p, int rows) {
  constexpr int G = GemvTraits<BITS>::G, CH = GemvTraits<BITS>::CH, HP = G / 2, U = 2;
  constexpr uint32_t kMagic = 0x64006400u;
  extern __shared__ uint4 smem[];  // x of the slice in operand order [4 NBQ][gps][4 words], then the offset terms
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 3, q = lane >> 2;
  const int g0 = blockIdx.y * p.gps;
  const int gcount = min(p.gps, p.ng - g0);
  float* const corr_lds = reinterpret_cast<float*>(smem + 4 * NBQ * p.gps * CH);

  // ---- the first items' loads go out ahead of the staging of x
  const int nq = blockIdx.x * 256 + wave * 64 + 4 * q;  // first column of this lane's quad
  const bool col_ok = nq < p.N;                       // (N % 4 == 0: a quad is all inside or all outside)
  const int nc = col_ok ? nq : 0;
  uint4 wa[U], wb[U];
  uint32_t sa[U], sb[U];
  auto issue = [&](int gl, uint4 (&wn)[U], uint32_t (&sn)[U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int g = g0 + min(gl + u, gcount - 1);
      wn[u] = *reinterpret_cast<const uint4*>(p.qw + static_cast<int64_t>(4 * g + li) * p.N + nc);
      sn[u] = p.qs[static_cast<int64_t>(g) * p.N + nc + li];
    }
  };
  issue(0, wa, sa);
  issue(U, wb, sb);

  // ---- stage this slice of x: one thread per (row, group); pair order, the odd fields' activations divided by 16 and
  //      the offset term formed from the divided values (as gq_quadrow.hip)
  for (int t = threadIdx.x; t < 4 * NBQ * gcount; t += 256) {
    const int b = t / gcount, gl = t - b * gcount;
    const int k0 = (g0 + gl) * G;
    uint32_t nat[HP], xr[HP];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int k = k0 + 8 * c;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (b < rows && k + 8 <= p.K) v = *reinterpret_cast<const uint4*>(p.x + static_cast<int64_t>(b) * p.K + k);
      nat[4 * c] = v.x; nat[4 * c + 1] = v.y; nat[4 * c + 2] = v.z; nat[4 * c + 3] = v.w;
    }
    permute_group<BITS>(nat, xr);
    const half2_t r16 = {static_cast<_Float16>(0.0625f), static_cast<_Float16>(0.0625f)};
    const half2_t r8 = {static_cast<_Float16>(0.125f), static_cast<_Float16>(0.125f)};
    const half2_t r64 = {static_cast<_Float16>(0.015625f), static_cast<_Float16>(0.015625f)};
    float corr = 0.f;
    if constexpr (BITS == 4) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        xr[4 * c + 1] = as_u32(as_half2(xr[4 * c + 1]) * r16);
        xr[4 * c + 3] = as_u32(as_half2(xr[4 * c + 3]) * r16);
        corr = dot2(xr[4 * c + 0], 0x64076407u /* (1031, 1031) */, corr);
        corr = dot2(xr[4 * c + 1], 0x64706470u /* (16 * 71, ..) */, corr);
        corr = dot2(xr[4 * c + 2], 0x64076407u, corr);
        corr = dot2(xr[4 * c + 3], 0x64706470u, corr);
        smem[(b * p.gps + gl) * CH + c] = make_uint4(xr[4 * c + 0], xr[4 * c + 2], xr[4 * c + 1], xr[4 * c + 3]);
      }
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        xr[5 * c + 1] = as_u32(as_half2(xr[5 * c + 1]) * r8);
        xr[5 * c + 4] = as_u32(as_half2(xr[5 * c + 4]) * r8);
        xr[5 * c + 2] = as_u32(as_half2(xr[5 * c + 2]) * r64);
        corr = dot2(xr[5 * c + 0], 0x64036403u /* (1027, 1027) */, corr);
        corr = dot2(xr[5 * c + 1], 0x64186418u /* (8 * 131, ..) */, corr);
        corr = dot2(xr[5 * c + 2], 0x64c064c0u /* (64 * 19, ..) */, corr);
        corr = dot2(xr[5 * c + 3], 0x64036403u, corr);
        corr = dot2(xr[5 * c + 4], 0x64186418u, corr);
        // word c: fields (0,5)(3,8) meet the x1 operands, (1,6)(4,9) the x8 operands
        smem[(b * p.gps + gl) * CH + c] = make_uint4(xr[5 * c + 0], xr[5 * c + 3], xr[5 * c + 1], xr[5 * c + 4]);
      }
      // fields (2,7) of all four words, the x64 class, share the fifth word
      smem[(b * p.gps + gl) * CH + 4] = make_uint4(xr[2], xr[7], xr[12], xr[17]);
    }
    corr_lds[b * p.gps + gl] = -corr;
  }
  __builtin_amdgcn_s_waitcnt(0);  // (the path around the staging loop would otherwise make the walk's first waits conservative)
  __syncthreads();

  float4_t acc[NBQ];
#pragma unroll
  for (int bq = 0; bq < NBQ; ++bq) acc[bq] = float4_t{0.f, 0.f, 0.f, 0.f};
  auto compute = [&](int gl, const uint4 (&wc)[U], const uint32_t (&sc)[U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bool live = gl + u < gcount;  // (uniform)
      const int g = min(gl + u, gcount - 1);
      const uint4 wt = kn_quad_transpose(wc[u], lane);  // the group's four words of column nq + li
      const uint32_t w[4] = {wt.x, wt.y, wt.z, wt.w};
      uint32_t lo[4][2], hi[4][2], a64[2][2];
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        if constexpr (BITS == 4) {
          const uint32_t w8 = w[d] >> 8;
          lo[d][0] = and_or_c(w[d], 0x000f000fu, kMagic);
          lo[d][1] = and_or_c(w8, 0x000f000fu, kMagic);
          hi[d][0] = and_or_c(w[d], 0x00f000f0u, kMagic);
          hi[d][1] = and_or_c(w8, 0x00f000f0u, kMagic);
        } else {
          // low half keeps fields 0-4, high half gets fields 5-9 aligned to bit 16
          const uint32_t tt = (w[d] & 0x0000ffffu) | ((w[d] << 1) & 0xffff0000u);
          const uint32_t t9 = tt >> 9;
          lo[d][0] = and_or_c(tt, 0x00070007u, kMagic);   // fields (0,5)
          lo[d][1] = and_or_c(t9, 0x00070007u, kMagic);   // fields (3,8)
          hi[d][0] = and_or_c(tt, 0x00380038u, kMagic);   // fields (1,6) x 8
          hi[d][1] = and_or_c(t9, 0x00380038u, kMagic);   // fields (4,9) x 8
          a64[d >> 1][d & 1] = and_or_c(tt, 0x01c001c0u, kMagic);  // fields (2,7) x 64
        }
      }
      // the four columns' scales of this block: lane 4q + i holds column i's (a group past the slice adds nothing)
      const uint32_t s32 = live ? __builtin_bit_cast(uint32_t, h2f(static_cast<uint16_t>(sc[u]))) : 0u;
      float sv[4];
      sv[0] = __builtin_bit_cast(float, kn_dpp<0x00>(s32));
      sv[1] = __builtin_bit_cast(float, kn_dpp<0x55>(s32));
      sv[2] = __builtin_bit_cast(float, kn_dpp<0xAA>(s32));
      sv[3] = __builtin_bit_cast(float, kn_dpp<0xFF>(s32));
#pragma unroll
      for (int bq = 0; bq < NBQ; ++bq) {
        const int e = (4 * bq + li) * p.gps + g;  // (activation row 4 bq + li, group): the same in every block
        const float c = corr_lds[e];
        float4_t tacc = {c, c, c, c};
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const uint4 xv = smem[e * CH + d];
          tacc = kn_mfma4(lo[d][0], lo[d][1], xv.x, xv.y, tacc);
          tacc = kn_mfma4(hi[d][0], hi[d][1], xv.z, xv.w, tacc);
        }
        if constexpr (BITS == 3) {
          const uint4 xv = smem[e * CH + 4];
          tacc = kn_mfma4(a64[0][0], a64[0][1], xv.x, xv.y, tacc);
          tacc = kn_mfma4(a64[1][0], a64[1][1], xv.z, xv.w, tacc);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[bq][i] = fmaf(sv[i], tacc[i], acc[bq][i]);
      }
    }
  };
  for (int gl = 0; gl < gcount; gl += 2 * U) {
    compute(gl, wa, sa);
    issue(gl + 2 * U, wa, sa);
    __builtin_amdgcn_sched_barrier(0);
    compute(gl + U, wb, sb);  // past the slice: scale 0, adds nothing
    issue(gl + 3 * U, wb, sb);
    __builtin_amdgcn_sched_barrier(0);
  }

  // lane (q, li): results of activation row 4 bq + li for the quad's four columns
  if (!col_ok) return;
#pragma unroll
  for (int bq = 0; bq < NBQ; ++bq) {
    const int b = 4 * bq + li;
    if (b >= rows) continue;
    float v[4] = {acc[bq][0], acc[bq][1], acc[bq][2], acc[bq][3]};
    if (p.slices > 1) {  // fp32 partial sums [slice][row][N]; the reduction adds the bias
      *reinterpret_cast<float4*>(static_cast<float*>(p.y) + (static_cast<int64_t>(blockIdx.y) * rows + b) * p.N + nq) =
          make_float4(v[0], v[1], v[2], v[3]);
      continue;
    }
    if (p.bias != nullptr) {
      const uint2 bb = *reinterpret_cast<const uint2*>(p.bias + nq);
      v[0] += h2f(static_cast<uint16_t>(bb.x & 0xffffu)); v[1] += h2f(static_cast<uint16_t>(bb.x >> 16));
      v[2] += h2f(static_cast<uint16_t>(bb.y & 0xffffu)); v[3] += h2f(static_cast<uint16_t>(bb.y >> 16));
    }
    const int64_t oi = static_cast<int64_t>(b) * p.N + nq;
    if (p.out_f32) {
      *reinterpret_cast<float4*>(static_cast<float*>(p.y) + oi) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
      uint2 o;
      o.x = static_cast<uint32_t>(f2h(v[0])) | (static_cast<uint32_t>(f2h(v[1])) << 16);
      o.y = static_cast<uint32_t>(f2h(v[2])) | (static_cast<uint32_t>(f2h(v[3])) << 16);
      *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.y) + oi) = o;
    }
  }
}

// y[i] = sum over slices of part[s][i] (+ bias), cast; i over M * N
__global__ __launch_bounds__(256) void kn_reduce_kernel(const float* __restrict__ part, int slices, int64_t count, int N,
                                                        const uint16_t* __restrict__ bias, void* y, int out_f32) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= count) return;
  float v = 0.f;
  for (int s = 0; s < slices; ++s) v += part[s * count + i];
  if (bias != nullptr) v += h2f(bias[i % N]);
  if (out_f32) static_cast<float*>(y)[i] = v;
  else static_cast<uint16_t*>(y)[i] = f2h(v);
}

// K slices for a shape: enough workgroups to cover the chip a few times over, whole groups, at most 64 per slice's x in LDS
int kn_slices(int64_t M, int64_t N, int ng) {
  const int64_t colblocks = (N + 255) / 256;
  int64_t slices = (512 + colblocks - 1) / colblocks;
  if (slices > (ng + 3) / 4) slices = (ng + 3) / 4;  // every wave keeps at least one group
  if (slices < 1) slices = 1;
  // x of a slice must fit LDS next to the sums: 48 KiB for x
  const int64_t per_group = M * (20 * 4 + 4);
  const int64_t gmax = (48 * 1024) / per_group;
  const int64_t need = (ng + gmax - 1) / gmax;
  if (slices < need) slices = need;
  return static_cast<int>(slices);
}

// the matrix-instruction form above: 16-byte aligned rows of x, 1..8 rows (a single row too: 4096 x 4096 7.8 us against
// 8.6 for the GEMV below, 4096 x 14336 15.8 / 19.1, 28672 x 4096 18.0 / 18.3, 6144 x 4096 9.3 / 9.1); tuning override
// gemv_variant 0: never
template <int BITS>
hipError_t launch_kn_quad(const KnParams& p0, int M, void* workspace, int64_t workspace_bytes, void* y,
                          const uint16_t* bias, hipStream_t s) {
  constexpr int kRowGroup = GemvTraits<BITS>::CH * 16 + 4;  // bytes of LDS per (activation row, group)
  const int gv = options().gemv_variant;
  if (!p0.x_vec || gv == 0) return hipErrorNotSupported;
  // (a single row of q3 over a large matrix: the GEMV's dot products are ahead, 4096 x 14336 12.1 us against 13.0,
  //  28672 x 4096 16.9 / 17.9; below that and from two rows on this form, 4096 x 4096 7.7 against 8.2, four rows of
  //  28672 x 4096 17.2 against 25.8, eight 21.0 / 38.9)
  if (BITS == 3 && M == 1 && gv < 0 && static_cast<int64_t>(p0.N) * p0.K >= (40ll << 20)) return hipErrorNotSupported;
  const int nbq = M <= 4 ? 1 : 2;
  KnParams p = p0;
  // K slices: about 512 workgroups, whole groups, the slice's x (68 bytes per row and group) within 48 KiB of LDS
  const int64_t colblocks = (p.N + 255) / 256;
  // (measured at 4 rows, graph replay over rotating weights: 4096 x 4096 at 8 / 16 / 32 slices 8.1 / 7.8 / 9.7 us, 6144 x 4096
  //  at 6 / 8 / 11 / 22 slices 10.4 / 9.0 / 9.3 / 11.1, 4096 x 14336 at 8 / 16 / 32 19.2 / 16.0 / 20.3, 28672 x 4096 at 2 / 3 / 4 / 7
  //  19.9 / 19.0 / 17.7 / 20.7: about one workgroup per CU, a little more where the column blocks alone are a third of that)
  const int64_t want = options().gemv_waves > 0 ? options().gemv_waves / 4 : (colblocks >= 64 ? 448 : 256);
  int64_t slices = (want + colblocks - 1) / colblocks;
  if (slices > (p.ng + 3) / 4) slices = (p.ng + 3) / 4;
  if (slices < 1) slices = 1;
  const int64_t gmax = (48 * 1024) / (4 * nbq * kRowGroup);
  if (slices < (p.ng + gmax - 1) / gmax) slices = (p.ng + gmax - 1) / gmax;
  const int64_t part_bytes = slices * M * p.N * 4;
  if (slices > 1 && (workspace == nullptr || workspace_bytes < part_bytes)) {
    if (p.ng > gmax) return hipErrorNotSupported;
    slices = 1;
  }
  p.gps = static_cast<int>((p.ng + slices - 1) / slices);
  p.slices = (p.ng + p.gps - 1) / p.gps;
  p.y = p.slices > 1 ? workspace : y;
  p.bias = p.slices > 1 ? nullptr : bias;
  const size_t lds = static_cast<size_t>(4 * nbq) * p.gps * kRowGroup;
  const dim3 grid(static_cast<unsigned>(colblocks), static_cast<unsigned>(p.slices));
  note_kernel("gq::kn_quad_kernel<%d,%d> slices=%d", BITS, nbq, p.slices);
  if (nbq == 1) hipLaunchKernelGGL((kn_quad_kernel<BITS, 1>), grid, dim3(256), lds, s, p, M);
  else hipLaunchKernelGGL((kn_quad_kernel<BITS, 2>), grid, dim3(256), lds, s, p, M);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || p.slices == 1) return e;
  const int64_t count = static_cast<int64_t>(M) * p.N;
  hipLaunchKernelGGL(kn_reduce_kernel, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, s,
                     static_cast<const float*>(workspace), p.slices, count, p.N, bias, y, p.out_f32);
  return hipGetLastError();
}

template <int BITS>
hipError_t launch_gemv_kn_bits(const KnParams& p0, int M, void* workspace, int64_t workspace_bytes, void* y,
                               const uint16_t* bias, hipStream_t s) {
  constexpr int CH = GemvTraits<BITS>::CH;
  {
    const hipError_t e = launch_kn_quad<BITS>(p0, M, workspace, workspace_bytes, y, bias, s);
    if (e != hipErrorNotSupported) return e;
  }
  KnParams p = p0;
  int slices = kn_slices(M, p.N, p.ng);
  const int64_t part_bytes = static_cast<int64_t>(slices) * M * p.N * 4;
  if (slices > 1 && (workspace == nullptr || workspace_bytes < part_bytes)) {
    // no room for partial sums: one slice per column block if x fits LDS whole, else decline
    if (static_cast<int64_t>(p.ng) * M * (CH * 16 + 4) > 48 * 1024) return hipErrorNotSupported;
    slices = 1;
  }
  p.slices = slices;
  p.gps = (p.ng + slices - 1) / slices;
  p.slices = (p.ng + p.gps - 1) / p.gps;
  p.y = p.slices > 1 ? workspace : y;
  p.bias = p.slices > 1 ? nullptr : bias;
  const size_t lds = static_cast<size_t>(M) * p.gps * (CH * 16) + static_cast<size_t>((M * p.gps + 3) & ~3) * 4 +
                     static_cast<size_t>(4) * M * 64 * 16;
  const dim3 grid(static_cast<unsigned>((p.N + 255) / 256), static_cast<unsigned>(p.slices));
  note_kernel("gq::gemv_kn_kernel<%d,%d> slices=%d", BITS, M, p.slices);
#define GQ_KN_CASE(NB_) \
  case NB_: hipLaunchKernelGGL((gemv_kn_kernel<BITS, NB_>), grid, dim3(256), lds, s, p); break;
  switch (M) {
    GQ_KN_CASE(1) GQ_KN_CASE(2) GQ_KN_CASE(3) GQ_KN_CASE(4) GQ_KN_CASE(5) GQ_KN_CASE(6) GQ_KN_CASE(7) GQ_KN_CASE(8)
    default: return hipErrorNotSupported;
  }
#undef GQ_KN_CASE
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || p.slices == 1) return e;
  const int64_t count = static_cast<int64_t>(M) * p.N;
  hipLaunchKernelGGL(kn_reduce_kernel, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, s,
                     static_cast<const float*>(workspace), p.slices, count, p.N, bias, y, p.out_f32);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_kn_transpose(const uint32_t* qw_src, const uint16_t* qs_src, int64_t src_rows_w, int64_t src_rows_s,
                               int64_t src_cols, uint32_t* qw_dst, uint16_t* qs_dst, hipStream_t s) {
  hipError_t e = launch_transpose<uint32_t>(qw_src, src_rows_w, src_cols, qw_dst, s);
  if (e != hipSuccess) return e;
  return launch_transpose<uint16_t>(qs_src, src_rows_s, src_cols, qs_dst, s);
}

hipError_t launch_dequantize_kn(const uint32_t* qw, const uint16_t* qs, int64_t N, int64_t K, int bits, uint16_t* out,
                                hipStream_t s) {
  const int G = bits == 4 ? 32 : 40;
  const int ng = static_cast<int>((K + G - 1) / G), nw = 4 * ng;
  const int64_t total = static_cast<int64_t>(nw) * N;
  if (total == 0) return hipSuccess;
  const dim3 grid(static_cast<unsigned>((total + 255) / 256));
  if (bits == 4) hipLaunchKernelGGL(dequantize_kn_kernel<4>, grid, dim3(256), 0, s, qw, qs, static_cast<int>(N), static_cast<int>(K), nw, out);
  else hipLaunchKernelGGL(dequantize_kn_kernel<3>, grid, dim3(256), 0, s, qw, qs, static_cast<int>(N), static_cast<int>(K), nw, out);
  return hipGetLastError();
}

int64_t gemv_kn_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits) {
  const int G = bits == 4 ? 32 : 40;
  const int ng = static_cast<int>((K + G - 1) / G);
  if (M < 1 || M > 8 || ng == 0) return 0;
  int64_t slices = kn_slices(M, N, ng);
  if (M >= 1) {  // the matrix-instruction form's split (launch_kn_quad)
    const int nbq = M <= 4 ? 1 : 2;
    const int64_t row_group = (bits == 4 ? 4 : 5) * 16 + 4;
    const int64_t colblocks = (N + 255) / 256;
    int64_t sq = ((colblocks >= 64 ? 448 : 256) + colblocks - 1) / colblocks;
    if (sq > (ng + 3) / 4) sq = (ng + 3) / 4;
    if (sq < 1) sq = 1;
    const int64_t gmax = (48 * 1024) / (4 * nbq * row_group);
    if (sq < (ng + gmax - 1) / gmax) sq = (ng + gmax - 1) / gmax;
    if (sq > slices) slices = sq;
  }
  return slices > 1 ? slices * M * N * 4 : 0;
}

// M <= 8 float16 rows, N % 4 == 0; hipErrorNotSupported otherwise (the caller transposes and runs the NK kernels)
hipError_t launch_gemv_kn(const uint16_t* x, const uint32_t* qw, const uint16_t* qs, const uint16_t* bias, int64_t M,
                          int64_t N, int64_t K, int bits, int out_f32, void* y, void* workspace, int64_t workspace_bytes,
                          hipStream_t s) {
  if (M < 1 || M > 8 || (N & 3) != 0 || K < 1) return hipErrorNotSupported;
  if ((reinterpret_cast<uintptr_t>(qw) & 15) != 0 || (reinterpret_cast<uintptr_t>(qs) & 7) != 0 ||
      (reinterpret_cast<uintptr_t>(y) & 15) != 0 || (reinterpret_cast<uintptr_t>(bias) & 7) != 0 ||
      (reinterpret_cast<uintptr_t>(workspace) & 15) != 0)
    return hipErrorNotSupported;
  const int G = bits == 4 ? 32 : 40;
  KnParams p{};
  p.x = x; p.qw = qw; p.qs = qs; p.bias = bias; p.y = y;
  p.N = static_cast<int>(N); p.K = static_cast<int>(K); p.ng = static_cast<int>((K + G - 1) / G);
  p.out_f32 = out_f32;
  p.x_vec = (K & 7) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
  if (bits == 4) return launch_gemv_kn_bits<4>(p, static_cast<int>(M), workspace, workspace_bytes, y, bias, s);
  return launch_gemv_kn_bits<3>(p, static_cast<int>(M), workspace, workspace_bytes, y, bias, s);
}

}  // namespace gq
