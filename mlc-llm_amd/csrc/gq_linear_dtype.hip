// Linear for the model dtypes other than float16 (q4f32_1, q4bf16_*): the dequantize-fused matmul
// of GroupQuantizeLinear.forward / lm_head_forward (group_quantization.py:390-437, 524-556) with
// x, q_scale and bias in float32 or bfloat16.
//
// A first form of the two regimes of the float16 path:
//  * up to 8 activation rows: a persistent-wave GEMV with x resident in LDS in the model dtype
//    (fp32 FMAs for float32, v_dot2_f32_bf16 on bf16 pairs for bfloat16);
//  * more rows: a 128 x 128 tile GEMM on v_mfma_f32_32x32x2_f32 with both operands in LDS as
//    float32 (bfloat16 operands are widened on the way in; their products are exact either way).
// Weights are dequantised exactly as GroupQuantize._dequantize does, (q - m) * scale rounded to the
// model dtype, before they meet x; accumulation is fp32.
// The same two kernels serve GroupQuantizeMixtralExperts.forward (group_quantization.py:619-660) over
// stacked expert weights: a workgroup row is then an expert segment (see Segment below).
#include <type_traits>

#include "gq_common.hpp"
#include "gq_internal.hpp"

namespace gq {

namespace {

template <int DT>
struct LinT;
template <>
struct LinT<MODEL_F32> {
  static __device__ __forceinline__ float load(const void* p, int64_t i) { return static_cast<const float*>(p)[i]; }
  static __device__ __forceinline__ float rnd(float v) { return v; }
};
template <>
struct LinT<MODEL_BF16> {
  static __device__ __forceinline__ float load(const void* p, int64_t i) {
    return __builtin_bit_cast(float, static_cast<uint32_t>(static_cast<const uint16_t*>(p)[i]) << 16);
  }
  static __device__ __forceinline__ float rnd(float v) {  // nearest-even bfloat16 (finite inputs)
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    return __builtin_bit_cast(float, (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u);
  }
};

__device__ __forceinline__ uint16_t bf16_bits(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
  return static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// out_kind: 1 float32, 2 bfloat16
__device__ __forceinline__ void store_out(void* y, int64_t i, float v, int out_kind) {
  if (out_kind == MODEL_F32) static_cast<float*>(y)[i] = v;
  else static_cast<uint16_t*>(y)[i] = bf16_bits(v);
}

struct LinParams {
  const void* x;
  const uint32_t* qw;
  const void* qs;
  const void* bias;
  const void* residual;  // [M, N] in the model dtype, added to the result, or null (may be y itself)
  void* y;
  int M, N, K, ng, nw;
  int out_kind;
  // expert stacks (q_weight [experts, N, nw], q_scale [experts, N, ng]); both null: a plain linear
  const int32_t* ids;   // dequantize_gemv: M output rows, row i uses expert ids[i]
  const void* indptr;   // dequantize_group_gemm: rows indptr[e] .. indptr[e + 1] of x use expert e
  int indptr_i64, num_experts;
  int x_one_row;        // with ids: every output row reads row 0 of x
};

// The activation rows one workgroup serves and where their weights start.
struct Segment {
  int64_t w_row0;  // first row of the expert's matrix in the stacked q_weight / q_scale
  int64_t x_row0, y_row0;
  int rows;
};

__device__ __forceinline__ Segment segment_of(const LinParams& p, int seg) {
  Segment sg{0, 0, 0, p.M};
  if (p.ids != nullptr) {
    const int e = min(max(p.ids[seg], 0), p.num_experts - 1);
    sg.w_row0 = static_cast<int64_t>(e) * p.N;
    sg.x_row0 = p.x_one_row ? 0 : seg;
    sg.y_row0 = seg;
    sg.rows = 1;
  } else if (p.indptr != nullptr) {
    int64_t lo, hi;
    if (p.indptr_i64) {
      lo = static_cast<const int64_t*>(p.indptr)[seg];
      hi = static_cast<const int64_t*>(p.indptr)[seg + 1];
    } else {
      lo = static_cast<const int32_t*>(p.indptr)[seg];
      hi = static_cast<const int32_t*>(p.indptr)[seg + 1];
    }
    lo = lo < 0 ? 0 : (lo > p.M ? p.M : lo);  // a corrupt indptr must not leave the tensors
    hi = hi < lo ? lo : (hi > p.M ? p.M : hi);
    sg.w_row0 = static_cast<int64_t>(seg) * p.N;
    sg.x_row0 = sg.y_row0 = lo;
    sg.rows = static_cast<int>(hi - lo);
  }
  return sg;
}

// ---------------------------------------------------------------- up to 8 rows

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));

// Persistent waves, two weight rows per step, the loads of the next two steps in flight (the
// structure of the float16 register GEMV); x lives in LDS in the model dtype, zero beyond K, and is
// read once per group for both rows.  Lane l owns groups l + 64 * it, it < ITERS.
//  * float32: one FMA per weight and activation row on the integer field itself; the group's sum is scaled
//    and offset once (s * (sum x q - m sum x)), as the float16 kernels do;
//  * bfloat16: (q - m) * s is exact in float32 (4 x 8 significant bits), v_cvt_pk_bf16_f32 rounds
//    two of them to the bf16 pair _dequantize would hold, and v_dot2_f32_bf16 multiplies the pair
//    with the matching pair of x (exact products, fp32 accumulation).
constexpr int gemv_dt_group_stride(int bits, int dt) {
  // float32: 16 bytes of padding (strides of 144 / 176 bytes); bfloat16: 80 / 88 bytes
  return dt == MODEL_F32 ? (bits == 4 ? 36 : 44) : (bits == 4 ? 40 : 44);
}

// SEG: expert stacks (a plain linear is compiled without the segment lookup and the pass loop, which cost
// its two-row float32 form a third of its speed).
template <int BITS, int DT, int NB, int ITERS, bool SEG>
__global__ __launch_bounds__(256) void gemv_dt_kernel(const LinParams p, int nsets) {
  using S = Scheme<BITS>;
  using T = LinT<DT>;
  constexpr int E = S::kElem;
  constexpr int G = 4 * E;
  constexpr bool BF = DT == MODEL_BF16;
  extern __shared__ uint32_t xs_raw[];
  float* xs = reinterpret_cast<float*>(xs_raw);         // float32: [NB][kpad]
  uint16_t* xh = reinterpret_cast<uint16_t*>(xs_raw);   // bfloat16: [NB][kpad]
  // a group of x is padded to GS elements so that the lanes of a wave, one group apart each, read
  // different LDS banks (unpadded, a group is 64 / 128 / 160 bytes and every lane lands on the same ones)
  constexpr int GS = gemv_dt_group_stride(BITS, DT);
  const int kpad = p.ng * GS;
  // blockIdx.y: the expert segment (one for a plain linear); a segment with more than NB rows is
  // served in passes over the expert's weights
  const Segment sg = SEG ? segment_of(p, blockIdx.y) : Segment{0, 0, 0, p.M};
  for (int m0 = 0; m0 < (SEG ? sg.rows : 1); m0 += NB) {
    if (m0 > 0) __syncthreads();  // the previous pass has finished reading x
    for (int i = threadIdx.x; i < NB * p.ng * G; i += 256) {
      const int b = i / (p.ng * G), k = i - b * (p.ng * G);
      const bool ok = m0 + b < sg.rows && k < p.K;
      const int at = b * kpad + (k / G) * GS + k % G;
      const int64_t src = (sg.x_row0 + m0 + b) * p.K + k;
      if (BF) xh[at] = ok ? static_cast<const uint16_t*>(p.x)[src] : uint16_t(0);
      else xs[at] = ok ? static_cast<const float*>(p.x)[src] : 0.0f;
    }

    const int lane = threadIdx.x & 63;
    const int gw = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int nwaves = gridDim.x * 4;
    int gidx[ITERS];
    bool gok[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      gok[it] = it * 64 + lane < p.ng;
      gidx[it] = gok[it] ? it * 64 + lane : p.ng - 1;
    }
    // branch-free loads: a set past the end reads valid addresses and is dropped at the store
    uint4 wa[2][ITERS], wb[2][ITERS];
    float sa[2][ITERS], sb[2][ITERS];
    auto issue = [&](int set, uint4 (&wn)[2][ITERS], float (&sn)[2][ITERS]) {
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int64_t row = sg.w_row0 + min(set * 2 + r, p.N - 1);
        const uint32_t* wr = p.qw + row * p.nw;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          wn[r][it] = *reinterpret_cast<const uint4*>(wr + 4 * gidx[it]);
          sn[r][it] = T::load(p.qs, row * p.ng + gidx[it]);
        }
      }
    };
    int set_a = gw, set_b = gw + nwaves;
    issue(set_a, wa, sa);
    issue(set_b, wb, sb);
    __syncthreads();

    const float m = static_cast<float>(S::kMaxInt);
    // float32: sum of x over each of this lane's groups, for the offset term of the scaled group sums below
    float xsum[BF ? 1 : NB][BF ? 1 : ITERS];
    if constexpr (!BF) {
#pragma unroll
      for (int it = 0; it < ITERS; ++it)
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          float t = 0.0f;
#pragma unroll
          for (int i = 0; i < G; ++i) t += xs[b * kpad + gidx[it] * GS + i];
          xsum[b][it] = t;
        }
    }
    auto reduce = [&](int set, const uint4 (&wc)[2][ITERS], const float (&sc)[2][ITERS]) {
      float acc[2][NB];
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[r][b] = 0.0f;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        float s[2], ms[2];
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          s[r] = gok[it] ? sc[r][it] : 0.0f;  // lanes past the last group add nothing
          ms[r] = -m * s[r];
        }
        float gacc[2][NB];  // float32: sum of x * q over the group, scaled once below
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
          for (int b = 0; b < NB; ++b) gacc[r][b] = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // the word's E values of x for every activation row, read once for both weight rows
          float xf[BF ? 1 : NB][BF ? 1 : E];
          uint32_t xp[BF ? NB : 1][BF ? E / 2 : 1];
          const int k0 = gidx[it] * GS + j * E;
#pragma unroll
          for (int b = 0; b < NB; ++b) {
            if constexpr (BF) {
              if constexpr (E == 8) {  // 8 bf16 = one 16-byte read
                const uint4 v4 = *reinterpret_cast<const uint4*>(xh + b * kpad + k0);
                xp[b][0] = v4.x; xp[b][1] = v4.y; xp[b][2] = v4.z; xp[b][3] = v4.w;
              } else {
#pragma unroll
                for (int i = 0; i < E / 2; ++i) xp[b][i] = reinterpret_cast<const uint32_t*>(xh + b * kpad + k0)[i];
              }
            } else if constexpr (E == 8) {  // k0 is a multiple of 8 floats: two 16-byte reads
              const float4 lo = *reinterpret_cast<const float4*>(xs + b * kpad + k0);
              const float4 hi = *reinterpret_cast<const float4*>(xs + b * kpad + k0 + 4);
              xf[b][0] = lo.x; xf[b][1] = lo.y; xf[b][2] = lo.z; xf[b][3] = lo.w;
              xf[b][4] = hi.x; xf[b][5] = hi.y; xf[b][6] = hi.z; xf[b][7] = hi.w;
            } else {                        // q3: k0 is a multiple of 10 floats: 8-byte reads
#pragma unroll
              for (int i = 0; i < E; i += 2) {
                const float2 v2 = *reinterpret_cast<const float2*>(xs + b * kpad + k0 + i);
                xf[b][i] = v2.x; xf[b][i + 1] = v2.y;
              }
            }
          }
#pragma unroll
          for (int r = 0; r < 2; ++r) {
            const uint32_t w = j == 0 ? wc[r][it].x : (j == 1 ? wc[r][it].y : (j == 2 ? wc[r][it].z : wc[r][it].w));
            float q[E];
            if constexpr (BITS == 4) {
              // even / odd fields spread one per byte: each conversion is then a single v_cvt_f32_ubyteN
              const uint32_t t0 = w & 0x0f0f0f0fu, t1 = (w >> 4) & 0x0f0f0f0fu;
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                q[2 * i] = static_cast<float>((t0 >> (8 * i)) & 0xffu);
                q[2 * i + 1] = static_cast<float>((t1 >> (8 * i)) & 0xffu);
              }
            } else {
#pragma unroll
              for (int i = 0; i < E; ++i) q[i] = static_cast<float>((w >> (i * BITS)) & S::kMask);
            }
            if constexpr (BF) {
#pragma unroll
              for (int i = 0; i < E / 2; ++i) {
                const float2_t pr = {fmaf(q[2 * i], s[r], ms[r]), fmaf(q[2 * i + 1], s[r], ms[r])};  // exact
                const bf16x2_t wp = __builtin_convertvector(pr, bf16x2_t);                            // _dequantize's rounding
#pragma unroll
                for (int b = 0; b < NB; ++b)
                  acc[r][b] = __builtin_amdgcn_fdot2_f32_bf16(wp, __builtin_bit_cast(bf16x2_t, xp[b][i]), acc[r][b], false);
              }
            } else {
#pragma unroll
              for (int i = 0; i < E; ++i)
#pragma unroll
                for (int b = 0; b < NB; ++b) gacc[r][b] = fmaf(q[i], xf[b][i], gacc[r][b]);
            }
          }
        }
        if constexpr (!BF) {
          // s * sum x (q - m): differs from the sum of x * round((q - m) * s) by 2^-24 per weight, the size of the
          // fp32 accumulation's own rounding
#pragma unroll
          for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int b = 0; b < NB; ++b) acc[r][b] = fmaf(s[r], fmaf(-m, xsum[b][it], gacc[r][b]), acc[r][b]);
        }
      }
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int row = set * 2 + r;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          const float t = wave_sum(acc[r][b]);
          if (lane == 0 && m0 + b < sg.rows && row < p.N) {
            const float bias = p.bias != nullptr ? T::load(p.bias, row) : 0.0f;
            const int64_t oi = (sg.y_row0 + m0 + b) * p.N + row;
            const float res = p.residual != nullptr ? T::load(p.residual, oi) : 0.0f;
            store_out(p.y, oi, t + bias + res, p.out_kind);
          }
        }
      }
    };
    while (set_a < nsets) {
      reduce(set_a, wa, sa);
      set_a += 2 * nwaves;
      issue(set_a, wa, sa);
      reduce(set_b, wb, sb);  // past the end: rows >= N, nothing is stored
      set_b += 2 * nwaves;
      issue(set_b, wb, sb);
    }
  }
}

// ---------------------------------------------------------------- more rows: fp32 MFMA GEMM

typedef float float16v __attribute__((ext_vector_type(16)));

// 128 x 128 tile, 4 waves of 64 x 64 (2 x 2 accumulators of 32 x 32), K tile = one group.
// LDS rows are G + 1 floats long: consecutive rows fall into consecutive banks, so the 32 rows a
// fragment read touches hit 32 different banks.
template <int BITS, int DT>
__global__ __launch_bounds__(256) void gemm_dt_kernel(const LinParams p) {
  using S = Scheme<BITS>;
  using T = LinT<DT>;
  constexpr int E = S::kElem;
  constexpr int G = 4 * E;      // K tile: 32 | 40
  constexpr int LD = G + 1;
  constexpr int BM = 128, BN = 128;
  constexpr int A_PER = BM * G / 256;  // x values per thread and tile: 16 | 20
  extern __shared__ float lds[];
  auto a_tile = [&](int s) { return lds + s * (BM + BN) * LD; };
  auto w_tile = [&](int s) { return lds + s * (BM + BN) * LD + BM * LD; };

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
  // blockIdx.y: the row tile; with expert stacks, the tiles of the segments one after another (a
  // segment of r rows owns ceil(r / BM) of them; python/mlc_llm/op/moe_matmul.py:653-679 of the
  // reference walks indptr per tile the same way)
  Segment sg = segment_of(p, 0);
  int mt = blockIdx.y;
  if (p.ids != nullptr) {
    sg = segment_of(p, mt);
    mt = 0;
  } else if (p.indptr != nullptr) {
    bool found = false;
    for (int e = 0; e < p.num_experts && !found; ++e) {
      sg = segment_of(p, e);
      const int tiles = (sg.rows + BM - 1) / BM;
      if (mt < tiles) found = true;
      else mt -= tiles;
    }
    if (!found) return;
  }
  const int m0 = mt * BM, n0 = blockIdx.x * BN;  // rows are counted inside the segment
  if (m0 >= sg.rows) return;
  const float m = static_cast<float>(S::kMaxInt);

  // this thread's share of a tile: x values (row ar, k offsets ak .. ak + A_PER) and two storage
  // words of weight row wrow
  const int ar = tid >> 1, ak = (tid & 1) * A_PER;
  const int64_t wrow = sg.w_row0 + min(n0 + (tid >> 1), p.N - 1);  // rows past N are computed and dropped
  const int whalf = tid & 1;
  float areg[A_PER];
  uint32_t wreg[2];
  float sreg = 0.0f;
  // rows of x that start 16-byte aligned (float32, K % 4 == 0) are read four values at a time
  const bool a_vec = DT == MODEL_F32 && (p.K & 3) == 0 && (reinterpret_cast<uintptr_t>(p.x) & 15) == 0;
  auto load_tile = [&](int kt) {
    const int64_t row = m0 + ar;
    if (a_vec) {
      const int64_t rc = sg.x_row0 + (row < sg.rows ? row : sg.rows - 1);  // a valid row; its values are dropped below
#pragma unroll
      for (int i = 0; i < A_PER; i += 4) {
        const int k = kt * G + ak + i;  // a multiple of 4, so the four values are inside K together
        const bool ok = row < sg.rows && k < p.K;
        const float4 v = *reinterpret_cast<const float4*>(static_cast<const float*>(p.x) + rc * p.K + (k < p.K ? k : 0));
        areg[i] = ok ? v.x : 0.0f; areg[i + 1] = ok ? v.y : 0.0f;
        areg[i + 2] = ok ? v.z : 0.0f; areg[i + 3] = ok ? v.w : 0.0f;
      }
    } else {
#pragma unroll
      for (int i = 0; i < A_PER; ++i) {
        const int k = kt * G + ak + i;
        areg[i] = (row < sg.rows && k < p.K) ? T::load(p.x, (sg.x_row0 + row) * p.K + k) : 0.0f;
      }
    }
    const uint32_t* wr = p.qw + wrow * p.nw + 4 * kt + 2 * whalf;
    wreg[0] = wr[0];
    wreg[1] = wr[1];
    sreg = T::load(p.qs, wrow * p.ng + kt);
  };
  auto store_tile = [&](int s) {
    float* at = a_tile(s) + ar * LD + ak;
#pragma unroll
    for (int i = 0; i < A_PER; ++i) at[i] = areg[i];
    float* wt = w_tile(s) + (tid >> 1) * LD + whalf * 2 * E;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const float q = static_cast<float>((wreg[j] >> (i * BITS)) & S::kMask);
        wt[j * E + i] = T::rnd((q - m) * sreg);
      }
  };

  float16v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int frow = lane & 31, fk = lane >> 5;  // fragment: lane supplies element (row, k = 2 * step + fk)
  const int nk = p.ng;
  load_tile(0);
  store_tile(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int s = kt & 1;
    if (kt + 1 < nk) load_tile(kt + 1);
    const float* at = a_tile(s) + (wm0 + frow) * LD + fk;
    const float* wt = w_tile(s) + (wn0 + frow) * LD + fk;
#pragma unroll
    for (int ks = 0; ks < G / 2; ++ks) {
      float a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) a[i] = at[i * 32 * LD + 2 * ks];
#pragma unroll
      for (int j = 0; j < 2; ++j) b[j] = wt[j * 32 * LD + 2 * ks];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) store_tile(s ^ 1);  // the other stage: nobody reads it during this tile
    __syncthreads();
  }

  // D[r][c] of a 32 x 32 accumulator: lane c + 32 * ((r / 4) % 2), register 4 * (r / 8) + r % 4
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn0 + j * 32 + (lane & 31);
      const float bias = (p.bias != nullptr && col < p.N) ? T::load(p.bias, col) : 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm0 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (row < sg.rows && col < p.N) {
          const int64_t oi = (sg.y_row0 + row) * p.N + col;
          const float res = p.residual != nullptr ? T::load(p.residual, oi) : 0.0f;
          store_out(p.y, oi, acc[i][j][r] + bias + res, p.out_kind);
        }
      }
    }
}

template <int BITS, int DT>
hipError_t launch_dt(const LinParams& p, hipStream_t s) {
  constexpr int G = 4 * Scheme<BITS>::kElem;
  const int iters = (p.ng + 63) / 64;
  const bool stacks = p.ids != nullptr || p.indptr != nullptr;
  const int segments = p.ids != nullptr ? p.M : (p.indptr != nullptr ? p.num_experts : 1);
  // up to 8 rows of a plain linear, the one-row segments of dequantize_gemv, and grouped problems of
  // few rows in total (every expert then streams its weights for a handful of rows)
  const bool few = p.ids != nullptr || (p.indptr != nullptr ? p.M <= 32 : p.M <= 8);
  if (few && iters <= 4) {
    // few activation rows per pass: the kernel's registers grow with rows x groups per lane (374 for
    // four float32 rows at K = 4096, one wave per SIMD), so more rows run as more passes over the
    // weights: measured faster from 3 rows (float32) / 5 rows (bfloat16) on
    const int cap = DT == MODEL_F32 ? 2 : 4;
    // a plain linear is cut into passes here; a segment's passes are the kernel's own loop
    const int seg_rows = p.ids != nullptr ? 1 : p.M;
    const int passes = stacks ? 1 : (seg_rows + cap - 1) / cap;
    const int per_pass = stacks ? (seg_rows < cap ? seg_rows : cap) : (seg_rows + passes - 1) / passes;
    const int nb = per_pass <= 1 ? 1 : (per_pass <= 2 ? 2 : 4);
    const size_t lds = static_cast<size_t>(nb) * p.ng * gemv_dt_group_stride(BITS, DT) * (DT == MODEL_BF16 ? 2 : 4);
    if (lds <= 150 * 1024) {
      const int nsets = (p.N + 1) / 2;
      int waves = nsets / 2;  // about two sets per wave, a few waves per SIMD
      waves = waves < 4 ? 4 : (waves > 2048 ? 2048 : waves);
      int blocks = (waves + 3) / 4;
      // expert stacks: every segment gets a grid of its own, so keep the total near two rounds of workgroups
      if (stacks && blocks * segments > 2048) blocks = 2048 / segments < 64 ? 64 : 2048 / segments;
      const size_t x_el = DT == MODEL_BF16 ? 2 : 4, y_el = p.out_kind == MODEL_BF16 ? 2 : 4;
      for (int m0 = 0; m0 < (stacks ? 1 : p.M); m0 += per_pass) {
        LinParams q = p;
        if (!stacks) {
          q.x = static_cast<const char*>(p.x) + static_cast<size_t>(m0) * p.K * x_el;
          q.y = static_cast<char*>(p.y) + static_cast<size_t>(m0) * p.N * y_el;
          if (p.residual != nullptr)
            q.residual = static_cast<const char*>(p.residual) + static_cast<size_t>(m0) * p.N * x_el;
          q.M = p.M - m0 < per_pass ? p.M - m0 : per_pass;
        }
        auto go = [&](auto kern) -> hipError_t {
          if (lds > 65536) {
            const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kern));
            if (e != hipSuccess) return e;
          }
          hipLaunchKernelGGL(kern, dim3(blocks, segments), dim3(256), lds, s, q, nsets);
          return hipGetLastError();
        };
        auto by_iters = [&](auto nbc) -> hipError_t {
          constexpr int NBC = decltype(nbc)::value;
          if (stacks) {
            if (iters == 1) return go(gemv_dt_kernel<BITS, DT, NBC, 1, true>);
            if (iters == 2) return go(gemv_dt_kernel<BITS, DT, NBC, 2, true>);
            return go(gemv_dt_kernel<BITS, DT, NBC, 4, true>);
          }
          if (iters == 1) return go(gemv_dt_kernel<BITS, DT, NBC, 1, false>);
          if (iters == 2) return go(gemv_dt_kernel<BITS, DT, NBC, 2, false>);
          return go(gemv_dt_kernel<BITS, DT, NBC, 4, false>);
        };
        const hipError_t e = nb == 1 ? by_iters(std::integral_constant<int, 1>{})
                                     : (nb == 2 ? by_iters(std::integral_constant<int, 2>{})
                                                : by_iters(std::integral_constant<int, 4>{}));
        if (e != hipSuccess) return e;
      }
      return hipSuccess;
    }
  }
  constexpr size_t lds = size_t(2) * 256 * (G + 1) * sizeof(float);
  auto kern = gemm_dt_kernel<BITS, DT>;
  const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kern));
  if (e != hipSuccess) return e;
  // row tiles: one per one-row segment; grouped, every expert may add a partly filled one
  const int m_tiles = p.ids != nullptr ? p.M : (p.M + 127) / 128 + (p.indptr != nullptr ? p.num_experts : 0);
  if (m_tiles > 65535) return hipErrorNotSupported;
  hipLaunchKernelGGL(kern, dim3((p.N + 127) / 128, m_tiles), dim3(256), lds, s, p);
  return hipGetLastError();
}

}  // namespace

template <typename Fill>
static hipError_t launch_dt_any(int64_t M, int64_t N, int64_t K, int bits, int group_size, int model_dtype,
                                int out_kind, hipStream_t s, Fill fill) {
  LinParams p{};
  p.M = static_cast<int>(M); p.N = static_cast<int>(N); p.K = static_cast<int>(K);
  p.ng = static_cast<int>((K + group_size - 1) / group_size);
  p.nw = 4 * p.ng;
  p.out_kind = out_kind;
  fill(p);
  if (model_dtype == MODEL_F32) return bits == 4 ? launch_dt<4, MODEL_F32>(p, s) : launch_dt<3, MODEL_F32>(p, s);
  if (model_dtype == MODEL_BF16) return bits == 4 ? launch_dt<4, MODEL_BF16>(p, s) : launch_dt<3, MODEL_BF16>(p, s);
  return hipErrorInvalidValue;
}

hipError_t launch_linear_dt(const void* x, const uint32_t* qw, const void* qs, const void* bias, const void* residual,
                            int64_t M, int64_t N, int64_t K, int bits, int group_size, int model_dtype, int out_kind,
                            void* y, hipStream_t s) {
  return launch_dt_any(M, N, K, bits, group_size, model_dtype, out_kind, s, [&](LinParams& p) {
    p.x = x; p.qw = qw; p.qs = qs; p.bias = bias; p.residual = residual; p.y = y;
  });
}

hipError_t launch_moe_gemv_dt(const void* x, bool x_one_row, const uint32_t* qw, const void* qs, const int32_t* ids,
                              int64_t slots, int64_t num_experts, int64_t N, int64_t K, int bits, int group_size,
                              int model_dtype, void* y, hipStream_t s) {
  return launch_dt_any(slots, N, K, bits, group_size, model_dtype, model_dtype, s, [&](LinParams& p) {
    p.x = x; p.qw = qw; p.qs = qs; p.y = y;
    p.ids = ids; p.x_one_row = x_one_row; p.num_experts = static_cast<int>(num_experts);
  });
}

hipError_t launch_moe_group_gemm_dt(const void* x, const uint32_t* qw, const void* qs, const void* indptr,
                                    bool indptr_i64, int64_t rows, int64_t num_experts, int64_t N, int64_t K,
                                    int bits, int group_size, int model_dtype, void* y, hipStream_t s) {
  return launch_dt_any(rows, N, K, bits, group_size, model_dtype, model_dtype, s, [&](LinParams& p) {
    p.x = x; p.qw = qw; p.qs = qs; p.y = y;
    p.indptr = indptr; p.indptr_i64 = indptr_i64; p.num_experts = static_cast<int>(num_experts);
  });
}

}  // namespace gq
