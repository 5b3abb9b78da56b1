// Few-row matmul for q4f16_1 / q3f16_1 on the 16-block 4x4x4 matrix instruction: 3..8 activation rows
// against streamed weights, with the memory access pattern of the batch-1 GEMV.
//
// Covers the same callers as gq_skinny.hip (the low-batch buckets of
// python/mlc_llm/compiler_pass/low_batch_specialization.py:22-57 and the few-tokens-per-expert
// case of python/mlc_llm/op/moe_matmul.py:562-768) whenever the activations fit LDS whole.
//
// v_mfma_f32_4x4x4_16b_f16 multiplies 16 independent 4x4x4 blocks: in block b (lanes 4b..4b+3)
// lane 4b+i supplies 4 k of A row i, lane 4b+j supplies the same 4 k of B column j, and lane 4b+j
// receives D[0..3][j].  Here A rows are 4 consecutive weight rows (a "quad"), B columns are 4
// activation rows, and the 16 blocks are 16 different quantisation groups of those rows:
//  * a lane loads ONE 128-bit group of ONE weight row per step, so a wave load covers 4 rows x
//    256 contiguous bytes (the 16x16x32 layout of gq_skinny.hip touches 16 rows x 64 bytes);
//  * the four storage words of the group unpack with the (field | 0x6400) trick into eight A
//    operands (even fields, and odd fields times 16), none of which leaves its lane: no LDS
//    transpose, no cross-lane move between the load and the matrix core;
//  * all 8 products of a group land in one accumulator pair, so the group's scale and the
//    (1024 + m) offset are applied once per group in fp32, as in the GEMV kernels (q3f16_1: ten
//    operands per group in three classes - fields that come out of the masks times 1, 8 and 64 -
//    and three accumulators);
//  * x is staged once per workgroup in LDS, already in operand order ([k step][word][lane] so
//    that every ds_read_b128 of a wave is one contiguous KiB), with the offset term of every
//    (activation row, group) beside it;
//  * waves are persistent and walk (quad, k step) items with the loads of the next two items
//    in flight, U KiB per item;
//  * when x does not fit LDS whole (8 rows of a 14336-wide layer), K is walked in phases: each
//    phase stages its slice of x and visits every quad, partial sums wait in LDS in between, so
//    the weights are still read exactly once.
// The 16 blocks are summed across lanes once per quad.
#include "gq_gemv_common.hpp"

namespace gq {

struct QuadParams {
  const uint16_t* x;
  const uint32_t* qw;
  const uint16_t* qs;
  const uint16_t* bias;
  const uint16_t* residual;  // [rows, N] or null
  void* y;
  const void* indptr;  // null: one segment [0, rows)
  int64_t expert_w_stride, expert_s_stride;
  int rows, N, K, ng, nw;
  int nquads;       // N / 4
  int nsets;        // quad sets (QP consecutive quads share every read of x): ceil(nquads / QP)
  int nsteps;       // k steps per quad and phase; a step is U iterations of 16 groups
  int steps_total;  // k steps per quad over all phases
  int nphases;      // passes over K, each with its slice of x in LDS
  int rounds;       // most quad sets any wave walks
  int indptr_i64, out_f32;
  int paired;       // fused gate/up form: y is [rows, N / 2] fp16
  const int32_t* x_rows;  // null, or the row of x each activation row reads (int32 [rows])
  int x_src_rows;         // rows of x when x_rows is set
  int bf16;               // x, scales, bias, residual and a 16-bit y are bfloat16
  int kw_log2 = 0;        // log2 of the waves that share a quad set's K range (launcher: one phase, one round)
};

// The kernel's ten leading arguments (14 dwords) arrive in scalar registers with the wave: x, qw, qs, y, rows, N, K and three
// packed words (below); ng, nw, nquads and nsets follow from them.  A plain linear reads nothing else, so it starts its
// loads without a memory read for its own arguments (about 0.4 us per launch, measured on the batch-1 kernel); the
// launch dimensions, which would sit in one more 64-byte line of the argument block, are not read by any form.
// QuadTail holds what the other forms add and is only read when kQuadHasTail is set.
struct QuadTail {
  const void* indptr;
  const int32_t* x_rows;
  int64_t expert_w_stride, expert_s_stride;
  const uint16_t* bias;
  const uint16_t* residual;
  int x_src_rows;
};
// packed words: w0 = nsteps | steps_total << 16, w1 = rounds | nwaves << 16,
// w2 = nphases | flags << 16 | log2(waves that share a quad set) << 20 | waves per workgroup << 24
constexpr uint32_t kQuadOutF32 = 1u << 16, kQuadIndptrI64 = 1u << 17, kQuadHasTail = 1u << 18;

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u(uint32_t v) {
  return static_cast<uint32_t>(
      __builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xf, 0xf, true));
}

__device__ __forceinline__ float4_t mfma4(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1,
                                          float4_t c) {
  typedef uint32_t u2 __attribute__((ext_vector_type(2)));
  const u2 a = {a0, a1}, b = {b0, b1};
  return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, a),
                                            __builtin_bit_cast(half4_t, b), c, 0, 0, 0);
}

// the same blocks on bfloat16 operands (v_mfma_f32_4x4x4_16b_bf16)
__device__ __forceinline__ float4_t mfma4_bf16(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, float4_t c) {
  typedef uint32_t u2 __attribute__((ext_vector_type(2)));
  typedef short short4_t __attribute__((ext_vector_type(4)));
  const u2 a = {a0, a1}, b = {b0, b1};
  return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(short4_t, a), __builtin_bit_cast(short4_t, b), c, 0,
                                                0, 0);
}

// NBQ: activation rows / 4 (rows past the segment are zero); U: iterations per item
// MODE 1: a bias or residual operand exists (template flag: their loads are extra memory
// instructions per item); MODE 2: fused gate/up form
// BF: bfloat16 model (x, scales, bias, residual and a 16-bit result are bfloat16).  0x4300 | q is the bfloat16
// 128 + q, so every field is shifted down to bit 0 of its half instead of being rescaled afterwards, and all
// operand classes share the offset 128 + m.
// QP: quads per item.  The x operands of an iteration are read from LDS once and meet the weights of QP
// consecutive quads, so the LDS bytes read per weight byte fall by that factor (a 4x4x4 block needs as many
// operand bytes of x as of weights: with 8 activation rows that is 8 LDS bytes per packed weight byte at QP = 1).
// KS: neighbouring waves may share the K range of a quad set (see kw_log2 below).  An instantiation of its own: with the
// split's bookkeeping the forms that run sixteen-wave workgroups no longer fit their 128 registers.
template <int BITS, int NBQ, int U, int MODE, bool BF = false, int QP = 1, bool KS = false>
// (sixteen-wave workgroups exist for the forms that fit 128 registers: 2 KiB items without the bias / residual loads;
//  with them the same bound forced spill reloads into the walk, and a reload waits for every weight load in flight)
__global__ __launch_bounds__((NBQ == 2 && U * QP <= 2 && MODE != 1 && !KS) ? 1024 : 512) void quad_kernel(const uint16_t* x_, const uint32_t* qw_, const uint16_t* qs_, void* y_, int rows_, int N_, int K_,
                 uint32_t w0, uint32_t w1, uint32_t w2, const QuadTail t) {
  QuadParams p;
  p.x = x_; p.qw = qw_; p.qs = qs_; p.y = y_;
  p.rows = rows_; p.N = N_; p.K = K_;
  p.ng = (K_ + GemvTraits<BITS>::G - 1) / GemvTraits<BITS>::G; p.nw = 4 * p.ng;
  p.nquads = N_ >> 2; p.nsets = (p.nquads + QP - 1) / QP;
  p.nsteps = w0 & 0xffffu; p.steps_total = w0 >> 16; p.rounds = w1 & 0xffffu; p.nphases = w2 & 0xffffu;
  p.out_f32 = (w2 & kQuadOutF32) != 0; p.indptr_i64 = (w2 & kQuadIndptrI64) != 0;
  p.indptr = nullptr; p.x_rows = nullptr; p.expert_w_stride = 0; p.expert_s_stride = 0;
  p.bias = nullptr; p.residual = nullptr; p.x_src_rows = 0;
  if (MODE == 1 || (w2 & kQuadHasTail) != 0) {
    p.indptr = t.indptr; p.x_rows = t.x_rows; p.expert_w_stride = t.expert_w_stride;
    p.expert_s_stride = t.expert_s_stride; p.bias = t.bias; p.residual = t.residual; p.x_src_rows = t.x_src_rows;
  }
  constexpr bool EXTRA = MODE == 1, PAIRED = MODE == 2;  // 2: fused gate/up form, quad = 2 (gate, up) pairs
  constexpr uint32_t kMagic = BF ? 0x43004300u : 0x64006400u;
  auto to_f32 = [](uint16_t bits) { return BF ? bf2f(bits) : h2f(bits); };
  auto to_out = [](float v) { return BF ? f2bf(v) : f2h(v); };
  auto mm = [](uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, float4_t c) {
    return BF ? mfma4_bf16(a0, a1, b0, b1, c) : mfma4(a0, a1, b0, b1, c);
  };
  constexpr int G = GemvTraits<BITS>::G;    // values per group: 32 | 40
  constexpr int CH = GemvTraits<BITS>::CH;  // 16-byte words of x per (activation row, group): 4 | 5
  constexpr int XB = BITS == 4 ? 4 : 3;     // (activation row, group) pairs a thread stages per round

  extern __shared__ uint4 smem[];

  const int tid = threadIdx.x, nthreads = static_cast<int>(w2 >> 24) << 6;
  const int lane = tid & 63;
  const int wpb = nthreads >> 6;
  const int gw = blockIdx.x * wpb + (tid >> 6);
  // K shared among neighbouring waves (matrices with few quads, where every wave has one quad set at most: a wave is
  // one dependent chain of loads, LDS reads and matrix instructions over its K range, and on such launches a SIMD hosts
  // a single wave, so nothing overlaps the chain): 2^kw_log2 consecutive waves of a workgroup take equal shares of the
  // steps of the same quad set, leave their sums in LDS, and the first of them adds the shares up after the walk.
  const int kw_log2 = KS ? static_cast<int>(w2 >> 20) & 3 : 0;
  const int ksub = gw & ((1 << kw_log2) - 1);
  const int gwq = gw >> kw_log2;
  const int nwaves = static_cast<int>(w1 >> 16) >> kw_log2;  // stride of the walk over quad sets
  const int li = lane & 3;   // weight row of the quad (A), activation row of the batch quad (B, D)
  const int ks = lane >> 2;  // block: group 16 * iteration + ks

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
  const int m0 = seg_lo + blockIdx.z * (4 * NBQ);
  if (m0 >= seg_hi) return;  // uniform: this expert has no (more) rows
  const int m_valid = min(4 * NBQ, seg_hi - m0);
  const uint32_t* qw = p.qw + expert * p.expert_w_stride;
  const uint16_t* qs = p.qs + expert * p.expert_s_stride;

  // LDS: x of one phase [NBQ][niter][CH words][64 lanes] uint4, its negated offset terms [NBQ][niter][64]
  // floats (what the group's accumulator starts from), then this workgroup's partial sums between phases
  // [wave][quad of the walk][NBQ][16]
  const int niter = p.nsteps * U;  // staged iterations per phase (groups past ng hold zeros)
  float* const corr_lds = reinterpret_cast<float*>(smem + static_cast<size_t>(NBQ) * niter * CH * 64);
  float* const part_lds = corr_lds + NBQ * niter * 64 + (tid >> 6) * (p.rounds * QP * NBQ * 16);

  uint4 wa[QP][U], wb[QP][U];
  uint32_t sa[QP][U], sb[QP][U];  // fp16 bits, 32 bits wide so that in-flight values are never re-packed
  uint2 ba[QP], bb[QP];
  uint2 ra[QP][NBQ], rb[QP][NBQ];  // residual of (activation row 4 * bq + lane, the quad's 4 weight rows), lanes 0..3
  float4_t acc[QP][NBQ];

  // K is walked in phases when x does not fit LDS whole: every phase stages its slice of x and
  // walks all of this wave's quads; partial sums wait in LDS for the last phase.
  for (int phase = 0; phase < p.nphases; ++phase) {
    const int nst_all = min(p.nsteps, p.steps_total - phase * p.nsteps);  // steps of this phase
    const int spw = (nst_all + (1 << kw_log2) - 1) >> kw_log2;            // ... per wave of a quad set
    const int step0 = ksub * spw;
    const int nst = max(0, min(spw, nst_all - step0));                    // ... of this wave (all of them unless K is shared)
    const int it0 = phase * niter;                                        // first iteration of the phase
    const int itw = step0 * U;                                            // ... of this wave inside the phase
    const bool last_phase = phase == p.nphases - 1;
#pragma unroll
    for (int qp = 0; qp < QP; ++qp)
#pragma unroll
      for (int bq = 0; bq < NBQ; ++bq) acc[qp][bq] = float4_t{0.f, 0.f, 0.f, 0.f};  // drops what an item past the end left

    // ---- weight / scale / bias loads of one item.  Branch-free: every path issues the same
    //      loads, so the wait counts let the other buffer's loads stay in flight across the loop;
    //      an item past the end reads one cached line instead.
    auto issue = [&](int qset, int step, uint4 (&wn)[QP][U], uint32_t (&sn)[QP][U], uint2 (&bn)[QP],
                     uint2 (&rn)[QP][NBQ]) {
#pragma unroll
      for (int qp = 0; qp < QP; ++qp) {
        const int quad = qset * QP + qp;
        const bool live = quad < p.nquads;
        int row = min(quad * 4 + li, p.N - 1);
        if (PAIRED) row = gate_up_row(row, p.N);
        const uint32_t* wr = qw + static_cast<int64_t>(row) * p.nw;
        const uint16_t* sr = qs + static_cast<int64_t>(row) * p.ng;
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int g = min((it0 + itw + step * U + u) * 16 + ks, p.ng - 1);
          wn[qp][u] = *reinterpret_cast<const uint4*>(live ? wr + 4 * g : qw);
          sn[qp][u] = *(live ? sr + g : qs);
        }
        // bias and residual ride along (at store time they would wait behind the next items' weights)
        if constexpr (EXTRA) {
          bn[qp] = *reinterpret_cast<const uint2*>(
              (live && p.bias != nullptr) ? p.bias + quad * 4 : reinterpret_cast<const uint16_t*>(qw));
#pragma unroll
          for (int bq = 0; bq < NBQ; ++bq) {
            const int b = min(4 * bq + (lane & 3), m_valid - 1);
            rn[qp][bq] = *reinterpret_cast<const uint2*>(
                (live && p.residual != nullptr) ? p.residual + static_cast<int64_t>(m0 + b) * p.N + quad * 4
                                                : reinterpret_cast<const uint16_t*>(qw));
          }
        }
      }
    };
    auto advance = [&](int& qset, int& step) {  // two items on
      step += 2;
      if (step >= nst) {
        step -= nst;
        qset += nwaves;
        if (step >= nst) {
          step -= nst;
          qset += nwaves;
        }
      }
    };
    const int q_first = nst > 0 ? gwq : p.nsets;  // (a wave whose share of the steps is empty has no quad set)
    int qa = q_first, sta = 0, qb = q_first, stb = 1;
    if (stb >= nst) {
      stb = 0;
      qb += nwaves;
    }
    issue(qa, sta, wa, sa, ba, ra);
    issue(qb, stb, wb, sb, bb, rb);

    // ---- stage x in operand order.  Pair q = (batch quad, iteration, lane') with lane' = 4 *
    //      block + activation row; its CH 16-byte words go to [q / 64][word][lane'].
    if (phase > 0) __syncthreads();  // the previous phase's x is still being read
    {
      const int npairs = NBQ * niter * 64;
      for (int q0 = tid; q0 < npairs; q0 += nthreads * XB) {
        uint4 raw[XB][CH];
        bool ok[XB][CH];
#pragma unroll
        for (int i = 0; i < XB; ++i) {
          const int q = q0 + i * nthreads;
          const int lp = q & 63, bi = q >> 6;  // bi = bq * niter + it
          const int bq = bi / niter, it = bi - bq * niter;
          const int b = 4 * bq + (lp & 3);
          const int g = 16 * (it0 + it) + (lp >> 2);
          const uint16_t* src = p.x + x_row(p.x_rows, p.x_src_rows, m0 + min(b, m_valid - 1)) * p.K;
#pragma unroll
          for (int c = 0; c < CH; ++c) {
            const int k = G * g + 8 * c;
            ok[i][c] = q < npairs && b < m_valid && g < p.ng && k + 8 <= p.K;
            raw[i][c] = *reinterpret_cast<const uint4*>(ok[i][c] ? src + k : p.x);
          }
        }
#pragma unroll
        for (int i = 0; i < XB; ++i) {
          const int q = q0 + i * nthreads;
          if (q < npairs) {
            uint32_t nat[G / 2], xr[G / 2];
#pragma unroll
            for (int c = 0; c < CH; ++c) {
              const uint4 r = ok[i][c] ? raw[i][c] : make_uint4(0, 0, 0, 0);
              nat[4 * c + 0] = r.x; nat[4 * c + 1] = r.y; nat[4 * c + 2] = r.z; nat[4 * c + 3] = r.w;
            }
            float corr = permute_group<BITS, BF>(nat, xr);
            const int lp = q & 63, bi = q >> 6;
            // The float16 unpack leaves the odd fields times 16 (q3: times 8 and times 64) in their operands.  Their
            // activations are divided by the same power of two here, once per workgroup, so that all of a group's
            // products can run through ONE accumulator.  The division is exact unless the quotient is subnormal
            // (|x| < 2^-10 for the x16 class, 2^-8 for x64).  The offset term is therefore formed from the divided
            // values (times 16 x 71, 8 x 131, 64 x 19: the same real numbers, so the same bits, wherever the division
            // was exact): what a rounded quotient adds to the products then cancels against it up to
            // 2^-25 * 16 * (q - m) per weight, instead of 2^-25 * 16 * (64 + q) with the offset taken from x itself.
            if constexpr (!BF) {
              const half2_t r16 = {static_cast<_Float16>(0.0625f), static_cast<_Float16>(0.0625f)};
              const half2_t r8 = {static_cast<_Float16>(0.125f), static_cast<_Float16>(0.125f)};
              const half2_t r64 = {static_cast<_Float16>(0.015625f), static_cast<_Float16>(0.015625f)};
              if constexpr (BITS == 4) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                  xr[4 * c + 1] = as_u32(as_half2(xr[4 * c + 1]) * r16);
                  xr[4 * c + 3] = as_u32(as_half2(xr[4 * c + 3]) * r16);
                }
              } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                  xr[5 * c + 1] = as_u32(as_half2(xr[5 * c + 1]) * r8);
                  xr[5 * c + 4] = as_u32(as_half2(xr[5 * c + 4]) * r8);
                  xr[5 * c + 2] = as_u32(as_half2(xr[5 * c + 2]) * r64);
                }
              }
              corr = 0.f;  // same order of accumulation as permute_group
              if constexpr (BITS == 4) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                  corr = dot2(xr[4 * c + 0], 0x64076407u /* (1031, 1031) */, corr);
                  corr = dot2(xr[4 * c + 1], 0x64706470u /* (16 * 71, ..) */, corr);
                  corr = dot2(xr[4 * c + 2], 0x64076407u, corr);
                  corr = dot2(xr[4 * c + 3], 0x64706470u, corr);
                }
              } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                  corr = dot2(xr[5 * c + 0], 0x64036403u /* (1027, 1027) */, corr);
                  corr = dot2(xr[5 * c + 1], 0x64186418u /* (8 * 131, ..) */, corr);
                  corr = dot2(xr[5 * c + 2], 0x64c064c0u /* (64 * 19, ..) */, corr);
                  corr = dot2(xr[5 * c + 3], 0x64036403u, corr);
                  corr = dot2(xr[5 * c + 4], 0x64186418u, corr);
                }
              }
            }
            if constexpr (BITS == 4) {
#pragma unroll
              for (int c = 0; c < 4; ++c)  // word c: (even fields: 2 pairs), (odd fields: 2 pairs)
                smem[(bi * CH + c) * 64 + lp] =
                    make_uint4(xr[4 * c + 0], xr[4 * c + 2], xr[4 * c + 1], xr[4 * c + 3]);
            } else {
              // word c: fields (0,5)(3,8) meet the x1 operands, (1,6)(4,9) the x8 operands;
              // fields (2,7) of all four words, the x64 class, share the fifth 16-byte word
#pragma unroll
              for (int c = 0; c < 4; ++c)
                smem[(bi * CH + c) * 64 + lp] =
                    make_uint4(xr[5 * c + 0], xr[5 * c + 3], xr[5 * c + 1], xr[5 * c + 4]);
              smem[(bi * CH + 4) * 64 + lp] = make_uint4(xr[2], xr[7], xr[12], xr[17]);
            }
            corr_lds[bi * 64 + lp] = -corr;
          }
        }
      }
    }
    // Every load above has been consumed by now, but on the path that skips the staging loop the
    // wait-count bookkeeping cannot see it and would make the walk's first waits conservative.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    // ---- persistent walk
    // the four results of (activation row m0 + b, quad) leave in the output's type
    auto put = [&](int quad, int b, const float (&v)[4]) {
      const int64_t oi = static_cast<int64_t>(m0 + b) * p.N + quad * 4;
      if constexpr (PAIRED) {
        *reinterpret_cast<uint32_t*>(static_cast<uint16_t*>(p.y) + (oi >> 1)) =
            static_cast<uint32_t>(silu_mul_t<BF>(v[0], v[1])) | (static_cast<uint32_t>(silu_mul_t<BF>(v[2], v[3])) << 16);
      } else if (p.out_f32) {
        *reinterpret_cast<float4*>(static_cast<float*>(p.y) + oi) = make_float4(v[0], v[1], v[2], v[3]);
      } else {
        uint2 o;
        o.x = static_cast<uint32_t>(to_out(v[0])) | (static_cast<uint32_t>(to_out(v[1])) << 16);
        o.y = static_cast<uint32_t>(to_out(v[2])) | (static_cast<uint32_t>(to_out(v[3])) << 16);
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.y) + oi) = o;
      }
    };
    int done = 0;  // quads this wave has completed in this phase
    auto compute = [&](int qset, int step, const uint4 (&wc)[QP][U], const uint32_t (&sc)[QP][U],
                       const uint2 (&bias_bits)[QP], const uint2 (&res_bits)[QP][NBQ]) {
      // One batch quad: every LDS read of the item goes out before the first matrix instruction.  Left to the compiler
      // each read is issued one ahead of its use, so a wave waits out most of an LDS round trip ten times per item, and
      // on the launches this form serves a SIMD often hosts a single wave.  (One instantiation, q3 with two quads per
      // item, once returned wrong sums for the first quad of every pair in this form.  The cause was the unpack's
      // v_and_or_b32 sitting in an asm statement, where the compiler cannot keep its distance to the matrix
      // instruction that reads the result: see and_or_c.)
      constexpr bool HOIST = NBQ == 1 && U <= 4;
      uint4 xh[HOIST ? U : 1][CH];
      float ch[HOIST ? U : 1];
      if constexpr (HOIST) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int bi = itw + step * U + u;
          ch[u] = corr_lds[bi * 64 + lane];
#pragma unroll
          for (int d = 0; d < CH; ++d) xh[u][d] = smem[(bi * CH + d) * 64 + lane];
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int it = itw + step * U + u;
        // A operands: q4 lo/hi = even / odd fields (x1, x16) of word d; q3 a1/a8 = the x1 / x8
        // fields of word d, a64 = the x64 field pairs of words (0,1) and (2,3)
        uint32_t lo[QP][4][2], hi[QP][4][2], a64[QP][2][2];
        float sv[QP][4];
#pragma unroll
        for (int qp = 0; qp < QP; ++qp) {
          const uint32_t w[4] = {wc[qp][u].x, wc[qp][u].y, wc[qp][u].z, wc[qp][u].w};
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            if constexpr (BITS == 4) {
              const uint32_t w8 = w[d] >> 8;
              lo[qp][d][0] = and_or_c(w[d], 0x000f000fu, kMagic);
              lo[qp][d][1] = and_or_c(w8, 0x000f000fu, kMagic);
              if constexpr (BF) {
                hi[qp][d][0] = and_or_c(w[d] >> 4, 0x000f000fu, kMagic);
                hi[qp][d][1] = and_or_c(w[d] >> 12, 0x000f000fu, kMagic);
              } else {
                hi[qp][d][0] = and_or_c(w[d], 0x00f000f0u, kMagic);
                hi[qp][d][1] = and_or_c(w8, 0x00f000f0u, kMagic);
              }
            } else {
              // low half keeps fields 0-4, high half gets fields 5-9 aligned to bit 16
              const uint32_t t = (w[d] & 0x0000ffffu) | ((w[d] << 1) & 0xffff0000u);
              const uint32_t t9 = t >> 9;
              lo[qp][d][0] = and_or_c(t, 0x00070007u, kMagic);   // fields (0,5)
              lo[qp][d][1] = and_or_c(t9, 0x00070007u, kMagic);  // fields (3,8)
              if constexpr (BF) {
                hi[qp][d][0] = and_or_c(t >> 3, 0x00070007u, kMagic);   // fields (1,6)
                hi[qp][d][1] = and_or_c(t >> 12, 0x00070007u, kMagic);  // fields (4,9)
                a64[qp][d >> 1][d & 1] = and_or_c(t >> 6, 0x00070007u, kMagic);  // fields (2,7)
              } else {
                hi[qp][d][0] = and_or_c(t, 0x00380038u, kMagic);   // fields (1,6) x 8
                hi[qp][d][1] = and_or_c(t9, 0x00380038u, kMagic);  // fields (4,9) x 8
                a64[qp][d >> 1][d & 1] = and_or_c(t, 0x01c001c0u, kMagic);  // fields (2,7) x 64
              }
            }
          }
          // the four rows' scales of this block: lane 4b+i holds row i's (converted once, then broadcast)
          const uint32_t s32 = __builtin_bit_cast(uint32_t, to_f32(static_cast<uint16_t>(sc[qp][u])));
          sv[qp][0] = __builtin_bit_cast(float, dpp_u<0x00>(s32));
          sv[qp][1] = __builtin_bit_cast(float, dpp_u<0x55>(s32));
          sv[qp][2] = __builtin_bit_cast(float, dpp_u<0xAA>(s32));
          sv[qp][3] = __builtin_bit_cast(float, dpp_u<0xFF>(s32));
        }
#pragma unroll
        for (int bq = 0; bq < NBQ; ++bq) {
          if (bq > 0 && 4 * bq >= m_valid) continue;  // uniform: this segment has no such rows
          const int bi = bq * niter + it;
          // one accumulator per group: it starts from minus the offset term and takes every operand class (the
          // activations of the scaled classes were divided when they were staged)
          float c;
          uint4 xv[CH];
          if constexpr (HOIST) {
            c = ch[u];
#pragma unroll
            for (int d = 0; d < CH; ++d) xv[d] = xh[u][d];
          } else {
            c = corr_lds[bi * 64 + lane];
#pragma unroll
            for (int d = 0; d < CH; ++d) xv[d] = smem[(bi * CH + d) * 64 + lane];
          }
#pragma unroll
          for (int qp = 0; qp < QP; ++qp) {
            float4_t t = {c, c, c, c};
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              t = mm(lo[qp][d][0], lo[qp][d][1], xv[d].x, xv[d].y, t);
              t = mm(hi[qp][d][0], hi[qp][d][1], xv[d].z, xv[d].w, t);
            }
            if constexpr (BITS == 3) {
              t = mm(a64[qp][0][0], a64[qp][0][1], xv[CH - 1].x, xv[CH - 1].y, t);
              t = mm(a64[qp][1][0], a64[qp][1][1], xv[CH - 1].z, xv[CH - 1].w, t);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[qp][bq][i] = fmaf(sv[qp][i], t[i], acc[qp][bq][i]);
          }
        }
      }
      if (step == nst - 1) {  // uniform: the quads' share of this phase is complete
#pragma unroll
        for (int qp = 0; qp < QP; ++qp) {
          const int quad = qset * QP + qp;
#pragma unroll
          for (int bq = 0; bq < NBQ; ++bq) {
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              float t = acc[qp][bq][i];
              t += dpp_f<0x124>(t);  // row_ror:4
              t += dpp_f<0x128>(t);  // row_ror:8: every lane holds the sum over its row of 16 lanes
              t += __shfl_xor(t, 16, kWave);
              t += __shfl_xor(t, 32, kWave);
              v[i] = t;
              acc[qp][bq][i] = 0.f;
            }
            const int b = 4 * bq + lane;  // lanes 0..3: one activation row each, 4 weight rows
            if (lane < 4 && b < m_valid && quad < p.nquads) {
              float4* part = reinterpret_cast<float4*>(part_lds) + ((done * QP + qp) * NBQ + bq) * 4 + lane;
              if (kw_log2 != 0) {  // (uniform) this wave's share of K: the shares meet after the walk
                *part = make_float4(v[0], v[1], v[2], v[3]);
                continue;
              }
              if (phase > 0) {
                const float4 pv = *part;
                v[0] += pv.x; v[1] += pv.y; v[2] += pv.z; v[3] += pv.w;
              }
              if (!last_phase) {
                *part = make_float4(v[0], v[1], v[2], v[3]);
              } else {
                if (EXTRA && p.bias != nullptr) {
                  v[0] += to_f32(static_cast<uint16_t>(bias_bits[qp].x & 0xffffu));
                  v[1] += to_f32(static_cast<uint16_t>(bias_bits[qp].x >> 16));
                  v[2] += to_f32(static_cast<uint16_t>(bias_bits[qp].y & 0xffffu));
                  v[3] += to_f32(static_cast<uint16_t>(bias_bits[qp].y >> 16));
                }
                if (EXTRA && p.residual != nullptr) {
                  v[0] += to_f32(static_cast<uint16_t>(res_bits[qp][bq].x & 0xffffu));
                  v[1] += to_f32(static_cast<uint16_t>(res_bits[qp][bq].x >> 16));
                  v[2] += to_f32(static_cast<uint16_t>(res_bits[qp][bq].y & 0xffffu));
                  v[3] += to_f32(static_cast<uint16_t>(res_bits[qp][bq].y >> 16));
                }
                put(quad, b, v);
              }
            }
          }
        }
        ++done;
      }
    };

    while (qa < p.nsets) {
      compute(qa, sta, wa, sa, ba, ra);
      advance(qa, sta);
      issue(qa, sta, wa, sa, ba, ra);
      __builtin_amdgcn_sched_barrier(0);  // keep the refill ahead of the next item's arithmetic
      compute(qb, stb, wb, sb, bb, rb);  // past the end: nothing is stored
      advance(qb, stb);
      issue(qb, stb, wb, sb, bb, rb);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (kw_log2 != 0) {  // (uniform over the launch; one phase, one quad set per group of waves: see the launcher)
      __syncthreads();
      if (ksub == 0 && gwq < p.nsets && lane < 4) {
        const int stride = p.rounds * QP * NBQ * 16;  // floats between the slots of consecutive waves
#pragma unroll
        for (int qp = 0; qp < QP; ++qp) {
          const int quad = gwq * QP + qp;
#pragma unroll
          for (int bq = 0; bq < NBQ; ++bq) {
            const int b = 4 * bq + lane;
            if (b < m_valid && quad < p.nquads) {
              float v[4] = {0.f, 0.f, 0.f, 0.f};
              for (int j = 0; j < (1 << kw_log2) && j * spw < nst_all; ++j) {  // in wave order, whatever finished first
                const float4 pv = reinterpret_cast<const float4*>(part_lds + j * stride)[(qp * NBQ + bq) * 4 + lane];
                v[0] += pv.x; v[1] += pv.y; v[2] += pv.z; v[3] += pv.w;
              }
              put(quad, b, v);
            }
          }
        }
      }
    }
  }
}

template <int BITS, int NBQ, int U, int MODE, bool BF = false, int QP = 1>
static hipError_t launch_quad_extra(const QuadParams& p, dim3 grid, int threads, size_t lds,
                                    hipStream_t s) {
  constexpr bool KS_OK = MODE != 1 && U * QP <= 2;  // the forms that exist with K shared between waves
  const bool ks = p.kw_log2 != 0;
  if (ks && !KS_OK) return hipErrorNotSupported;
  if (lds > 65536) {
    hipError_t e = hipSuccess;
    if constexpr (KS_OK) {
      if (ks) e = allow_large_lds(reinterpret_cast<const void*>(&quad_kernel<BITS, NBQ, U, MODE, BF, QP, true>));
    }
    if (!ks) e = allow_large_lds(reinterpret_cast<const void*>(&quad_kernel<BITS, NBQ, U, MODE, BF, QP>));
    if (e != hipSuccess) return e;
  }
  note_kernel("gq::quad_kernel<%d,%d,%d,%d,%s,%d%s>", BITS, NBQ, U, MODE, BF ? "true" : "false", QP, ks ? ",true" : "");
  const int nwaves = static_cast<int>(grid.x) * (threads >> 6);
  if (threads % 64 != 0 || threads > ((ks || NBQ != 2 || U * QP > 2 || MODE == 1) ? 512 : 1024) || p.nsteps > 0xffff || p.steps_total > 0xffff || p.rounds > 0xffff ||
      nwaves > 0xffff || p.nphases > 0xffff || p.nquads != p.N / 4 || p.nsets != (p.nquads + QP - 1) / QP ||
      p.kw_log2 < 0 || p.kw_log2 > 2 ||
      (p.kw_log2 != 0 && (p.nphases != 1 || p.rounds != 1 || MODE == 1 || (threads >> 6) % (1 << p.kw_log2) != 0 ||
                          (nwaves >> p.kw_log2) < p.nsets)))
    return hipErrorNotSupported;
  const bool tail = p.indptr != nullptr || p.x_rows != nullptr || p.bias != nullptr || p.residual != nullptr;
  const QuadTail t{p.indptr, p.x_rows, p.expert_w_stride, p.expert_s_stride, p.bias, p.residual, p.x_src_rows};
  const uint32_t w0 = static_cast<uint32_t>(p.nsteps) | static_cast<uint32_t>(p.steps_total) << 16;
  const uint32_t w1 = static_cast<uint32_t>(p.rounds) | static_cast<uint32_t>(nwaves) << 16;
  const uint32_t w2 = static_cast<uint32_t>(p.nphases) | (p.out_f32 ? kQuadOutF32 : 0u) |
                      (p.indptr_i64 ? kQuadIndptrI64 : 0u) | (tail ? kQuadHasTail : 0u) |
                      static_cast<uint32_t>(p.kw_log2) << 20 | static_cast<uint32_t>(threads >> 6) << 24;
  if constexpr (KS_OK) {
    if (ks) {
      hipLaunchKernelGGL((quad_kernel<BITS, NBQ, U, MODE, BF, QP, true>), grid, dim3(threads), lds, s,
                         p.x, p.qw, p.qs, p.y, p.rows, p.N, p.K, w0, w1, w2, t);
      return hipGetLastError();
    }
  }
  hipLaunchKernelGGL((quad_kernel<BITS, NBQ, U, MODE, BF, QP>), grid, dim3(threads), lds, s,
                     p.x, p.qw, p.qs, p.y, p.rows, p.N, p.K, w0, w1, w2, t);
  return hipGetLastError();
}

template <int BITS, int NBQ, int U, int QP = 1>
static hipError_t launch_quad_cfg(const QuadParams& p, dim3 grid, int threads, size_t lds,
                                  hipStream_t s) {
  if (p.bf16) {
    if constexpr (QP == 1) {
      if (p.paired) return launch_quad_extra<BITS, NBQ, U, 2, true>(p, grid, threads, lds, s);
      return (p.bias != nullptr || p.residual != nullptr)
                 ? launch_quad_extra<BITS, NBQ, U, 1, true>(p, grid, threads, lds, s)
                 : launch_quad_extra<BITS, NBQ, U, 0, true>(p, grid, threads, lds, s);
    } else {
      return hipErrorNotSupported;
    }
  }
  if (p.paired) return launch_quad_extra<BITS, NBQ, U, 2, false, QP>(p, grid, threads, lds, s);
  return (p.bias != nullptr || p.residual != nullptr)
             ? launch_quad_extra<BITS, NBQ, U, 1, false, QP>(p, grid, threads, lds, s)
             : launch_quad_extra<BITS, NBQ, U, 0, false, QP>(p, grid, threads, lds, s);
}

// hipErrorNotSupported when the shape does not fit (the caller falls back to its other kernels)
template <int BITS>
static hipError_t launch_quadrow_bits(const GemmArgs& a, int rows_max, hipStream_t s) {
  constexpr int G = GemvTraits<BITS>::G;
  constexpr int CH = GemvTraits<BITS>::CH;
  if (a.group_size != G) return hipErrorNotSupported;
  if (a.rows == 0 || a.N == 0) return hipSuccess;
  if ((a.N & 3) != 0 || (a.K & 7) != 0 || a.K == 0) return hipErrorNotSupported;
  if ((reinterpret_cast<uintptr_t>(a.x) & 15) != 0 || (reinterpret_cast<uintptr_t>(a.y) & 15) != 0 ||
      (reinterpret_cast<uintptr_t>(a.bias) & 7) != 0 || (reinterpret_cast<uintptr_t>(a.residual) & 7) != 0 ||
      (reinterpret_cast<uintptr_t>(a.q_weight) & 15) != 0)
    return hipErrorNotSupported;
  QuadParams p;
  p.x = a.x; p.qw = a.q_weight; p.qs = a.q_scale; p.bias = a.bias; p.residual = a.residual; p.y = a.y;
  p.indptr = a.indptr; p.indptr_i64 = a.indptr_i64; p.paired = a.paired;
  p.x_rows = a.x_rows; p.x_src_rows = static_cast<int>(a.x_src_rows);
  p.bf16 = a.bf16;
  p.rows = static_cast<int>(a.rows); p.N = static_cast<int>(a.N); p.K = static_cast<int>(a.K);
  p.ng = static_cast<int>((a.K + G - 1) / G);
  p.nw = 4 * p.ng;
  p.nquads = p.N / 4;
  p.expert_w_stride = a.N * p.nw;
  p.expert_s_stride = a.N * p.ng;
  p.out_f32 = a.out_f32;
  const int experts = a.indptr ? static_cast<int>(a.num_experts) : 1;

  // LDS per iteration (16 groups) and batch quad: x in operand order and the offset terms
  constexpr size_t kLdsIter = CH * 1024 + 256;
  const int niter = (p.ng + 15) / 16;
  const int opt_u = options().gemv_rows_per_wave;  // tuning override (1: 2 KiB items and sixteen waves per workgroup)
  const int mode = options().gemv_variant;
  // measured: 4 KiB items pay off only on matrices large enough to run long (gate_up, lm_head)
  const bool large = niter >= 4 && static_cast<int64_t>(a.N) * a.K * experts >= (100ll << 20);
  // ... except with two batch quads (5..8 rows) of a plain linear: there sixteen waves per workgroup (four per
  // SIMD, one copy of x between them) on 2 KiB items and twice the waves are ahead (gate_up 28672 x 4096 at 8
  // rows: 24.9 -> 22.2 us, lm_head 74.3 -> 72.0; slower everywhere else, 4 rows included)
  // quads per item (tuning override; float16 only)
  // Quads per item: two where the 8-row form runs long (float16; measured on 28672 x 4096 at 8 rows 21.5 -> 20.5 us,
  // 128256 x 4096 68.6 -> 67.0, Mixtral's expert layer at 16 tokens 197 -> 180 us; 4-row forms within 1.5 % either
  // way, small matrices 5-25 % slower: half as many items to spread over the waves; four quads per item no better)
  const int opt_qp = options().quad_pairs;
  int QP = 1;
  bool big_wg = opt_u == 1 || (opt_u < 0 && large && rows_max > 4 && a.indptr == nullptr && mode != 8 &&
                               options().gemv_waves <= 0);
  int U = 0, nbq = 0;
  for (int attempt = 0; attempt < 2; ++attempt) {
    U = (opt_u == 2 || opt_u == 4 || opt_u == 8) ? opt_u : (big_wg ? 2 : (large ? 4 : 2));
    p.steps_total = (niter + U - 1) / U;
    // More than 4 rows: 8 per pass when their x fits LDS whole.  Otherwise a plain linear runs
    // two concurrent 4-row passes (the second pass's weight reads hit the last-level cache, and
    // the grid doubles), a grouped matmul walks K in phases (experts already fill the grid).
    // Tuning overrides: gemv_variant 7 prefers phases, 8 prefers 4-row passes.
    nbq = rows_max <= 4 ? 1 : 2;
    if (nbq == 2) {
      const size_t whole = static_cast<size_t>(p.steps_total) * U * 2 * kLdsIter;
      const bool phases = mode == 7 || (mode != 8 && a.indptr != nullptr);
      if (mode == 8 || (whole > 150 * 1024 && !phases)) nbq = 1;
    }
    if (!big_wg || nbq == 2) break;
    big_wg = false;  // x of 8 rows does not fit: the concurrent 4-row passes keep their own launch shape
  }
  QP = a.bf16 ? 1 : ((opt_qp == 1 || opt_qp == 2) ? opt_qp : ((large && nbq == 2) ? 2 : 1));
  if (QP == 2) {
    U = U >= 4 ? 2 : 1;  // the same bytes per item
    p.steps_total = (niter + U - 1) / U;
  }
  const int mtiles = (rows_max + 4 * nbq - 1) / (4 * nbq);
  if (mtiles > 4 && a.indptr == nullptr) return hipErrorNotSupported;

  // About one quad per wave up to 2048 waves (measured over the projection shapes of 7B..70B models: 13 to 30 %
  // faster than 1024 waves of two to four quads each at 2..8 rows); concurrent passes over the same weights
  // already multiply the grid, and there 1024 measured better (down_proj 8192 x 28672 at 8 rows: 48 vs 66 us).
  int waves = options().gemv_waves > 0 ? options().gemv_waves
                                       : (big_wg ? 4096 : (a.indptr != nullptr || mtiles == 1 ? 2048 : 1024));
  // workgroups of experts without rows leave at once: share the waves among those that can have rows
  const int busy = p.rows < experts ? p.rows : experts;
  waves = (waves + busy - 1) / busy;
  p.nsets = (p.nquads + QP - 1) / QP;
  if (waves > p.nsets) waves = p.nsets;
  p.rounds = (p.nsets + waves - 1) / waves;

  // per wave: the partial sums of its quads.  Phases share K evenly.
  const size_t lds_cap = 150 * 1024;
  const size_t lds_step = static_cast<size_t>(U) * nbq * kLdsIter;
  const size_t lds_part = static_cast<size_t>(8) * p.rounds * QP * nbq * 64;  // up to 8 waves
  if (lds_part + lds_step > lds_cap) return hipErrorNotSupported;
  const int steps_fit = static_cast<int>((lds_cap - lds_part) / lds_step);
  p.nphases = (p.steps_total + steps_fit - 1) / steps_fit;
  p.nsteps = (p.steps_total + p.nphases - 1) / p.nphases;
  const size_t lds_x = lds_step * p.nsteps;
  // two waves per SIMD: 512-thread workgroups when only one workgroup fits a CU's LDS
  // ... unless that leaves CUs without a workgroup (down_proj with 4 rows: 1024 quads = 128 workgroups
  // of 8 waves): then 4 waves per workgroup and twice the workgroups
  // ... and for a plain linear in general: every workgroup stages all of x, so eight waves sharing one copy
  // halve that traffic (qkv 6144 x 4096 at 8 rows 11.4 -> 9.9 us, gate_up 24.3 -> 22.6; never slower)
  // K shared among 2 neighbouring waves: a plain linear whose waves have one quad set at most, on a long K (every wave
  // keeps five steps or more) and while the launch stays within two waves per SIMD.  Measured at 4 rows: 4096 x 14336
  // 15.7 -> 14.0 us, 4096 x 11008 12.7 -> 11.6; with four steps per wave to share (K = 4096) the meeting of the shares costs
  // more than the shorter chains return (o_proj 6.5 -> 7.1 us), past two waves per SIMD it loses outright (6144 x 4096:
  // 8.0 -> 12.4), and so do four waves per quad set (14.5 -> 19.6).
  // Tuning override: quad_ksplit 0 | 1 | 2.
  p.kw_log2 = 0;
  if (a.indptr == nullptr && p.nphases == 1 && p.rounds == 1 && a.bias == nullptr && a.residual == nullptr &&
      U * QP <= 2 && !big_wg) {
    const int opt_kw = options().quad_ksplit > 2 ? 2 : options().quad_ksplit;
    const int want = opt_kw >= 0 ? opt_kw : 1;
    while (p.kw_log2 < want && p.kw_log2 < 2 && (p.steps_total >> (p.kw_log2 + 1)) >= (opt_kw >= 0 ? 1 : 5) &&
           (static_cast<int64_t>(p.nsets) * mtiles << (p.kw_log2 + 1)) <= (opt_kw >= 0 ? 4096 : 2048))
      ++p.kw_log2;
  }
  const int sets_w = ((p.nsets + p.rounds - 1) / p.rounds) << p.kw_log2;  // waves of one grid row that have work
  int threads = (lds_x > 76 * 1024 || a.indptr == nullptr) ? 512 : 256;
  if (threads == 512) {
    const int64_t wgs = static_cast<int64_t>((sets_w + 7) / 8) * busy * mtiles;
    if (2 * wgs <= 256) threads = 256;  // (the doubled count must still be one round of workgroups)
  }
  // four waves per SIMD share one copy of x (the instances that fit 128 registers: 2 KiB items without bias / residual loads)
  if (big_wg && nbq == 2 && p.nphases == 1 && U * QP <= 2 && a.bias == nullptr && a.residual == nullptr) threads = 1024;
  const int wpb = threads / 64;
  const size_t lds = lds_x + ((p.nphases > 1 || p.kw_log2 != 0) ? static_cast<size_t>(wpb) * p.rounds * QP * nbq * 64 : 0);
  const int blocks = (sets_w + wpb - 1) / wpb;
  const dim3 grid(blocks, experts, mtiles);
#define GQ_QUAD_CASE(NBQ_, U_) \
  if (nbq == NBQ_ && U == U_) return launch_quad_cfg<BITS, NBQ_, U_>(p, grid, threads, lds, s);
  if (QP == 1) {
    GQ_QUAD_CASE(1, 2) GQ_QUAD_CASE(1, 4) GQ_QUAD_CASE(1, 8)
    GQ_QUAD_CASE(2, 2) GQ_QUAD_CASE(2, 4) GQ_QUAD_CASE(2, 8)
  }
#undef GQ_QUAD_CASE
#define GQ_QUAD_CASE(NBQ_, U_) \
  if (nbq == NBQ_ && U == U_) return launch_quad_cfg<BITS, NBQ_, U_, 2>(p, grid, threads, lds, s);
  if (QP == 2) {
    GQ_QUAD_CASE(1, 1) GQ_QUAD_CASE(1, 2)
    GQ_QUAD_CASE(2, 1) GQ_QUAD_CASE(2, 2)
  }
#undef GQ_QUAD_CASE
  return hipErrorNotSupported;
}

hipError_t launch_quadrow(const GemmArgs& a, int rows_max, hipStream_t s) {
  if (a.bits == 4) return launch_quadrow_bits<4>(a, rows_max, s);
  if (a.bits == 3) return launch_quadrow_bits<3>(a, rows_max, s);
  return hipErrorNotSupported;
}

}  // namespace gq
