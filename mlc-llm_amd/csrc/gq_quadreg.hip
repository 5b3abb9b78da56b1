// Few-row matmul (up to 8 activation rows) for q4f16_1 / q3f16_1 with the activations RESIDENT IN REGISTERS.
//
// Same callers and the same arithmetic as gq_quadrow.hip (the low-batch buckets of
// python/mlc_llm/compiler_pass/low_batch_specialization.py:22-57 under GroupQuantizeLinear.forward,
// python/mlc_llm/quantization/group_quantization.py:390-437): v_mfma_f32_4x4x4_16b_f16 multiplies 16 independent 4x4x4
// blocks, A rows = 4 consecutive weight rows (a "quad"), B columns = 4 activation rows, the 16 blocks = 16 quantisation
// groups; a lane loads ONE 128-bit group of ONE weight row per iteration, so a wave's load instruction covers 4 rows x 256
// contiguous bytes, and the unpacked operands never leave their lane.
//
// What differs is where x lives.  There, every workgroup stages all of x in LDS (64 KiB at 8 rows of K = 4096) and every
// item re-reads its operands from LDS; on the small projections that staging and its barrier, and the LDS round trips in
// front of the matrix instructions, cost as much as streaming the weights.  Here:
//  * KW = 1, 2, 4 or 8 neighbouring waves share the K range of a quad; a wave owns U consecutive iterations (U x 256 B of
//    every weight row) and keeps the matching slice of x - U x 64 bytes per activation row and lane, already in operand
//    order, with the offset terms - in VGPRs for the whole kernel.  It reads that slice from global memory (L2) once, with
//    row-contiguous 16-byte loads (a wave instruction covers whole 128-byte lines), and turns it into the per-lane operand
//    order through an LDS tile of its own (4 rows x 1 KiB; no other wave touches it, so no barrier): there is no shared
//    staging, no barrier in front of the walk and no LDS read inside it;
//  * persistent waves walk quads with two quads of loads in flight (register ping-pong, branch-free issue);
//  * results leave after the walk: a wave's partial sums wait in LDS (64 bytes per quad, batch quad and wave), one
//    barrier, then the first wave of each group adds the shares in wave order and stores.  Bias and residual are read
//    there as well, after the weight stream, so they never queue in front of it.
#include "gq_gemv_common.hpp"

namespace gq {

namespace {

template <int CTRL>
__device__ __forceinline__ uint32_t qr_dpp_u(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xf, 0xf, true));
}

__device__ __forceinline__ float4_t qr_mfma4(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, float4_t c) {
  typedef uint32_t u2 __attribute__((ext_vector_type(2)));
  const u2 a = {a0, a1}, b = {b0, b1};
  return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, a), __builtin_bit_cast(half4_t, b), c, 0, 0, 0);
}

// the same blocks on bfloat16 operands (v_mfma_f32_4x4x4_16b_bf16)
__device__ __forceinline__ float4_t qr_mfma4_bf16(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, float4_t c) {
  typedef uint32_t u2 __attribute__((ext_vector_type(2)));
  typedef short short4_t __attribute__((ext_vector_type(4)));
  const u2 a = {a0, a1}, b = {b0, b1};
  return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(short4_t, a), __builtin_bit_cast(short4_t, b), c, 0,
                                                0, 0);
}

struct QuadRegTail {
  const uint16_t* bias;      // [N] or null
  const uint16_t* residual;  // [rows, N] or null
};

constexpr uint32_t kQrOutF32 = 1u;

// NBQ: batch quads (rows <= 4 * NBQ); U: iterations (of 16 groups) a wave owns; KWL: log2 of the waves that share a quad;
// MODE 0: plain, 1: bias / residual, 2: fused gate/up form (y is [rows, N / 2]).
// BF: bfloat16 model (x, scales, bias, residual and the 16-bit result are bfloat16): the unpack shifts every field down to
// the low bits (a bfloat16 has no room for the x16 trick), every field carries the offset 128 + m, x is not rescaled.
// The eleven leading arguments (13 dwords) arrive in scalar registers with the wave.
template <int BITS, int NBQ, int U, int KWL, int MODE, bool BF = false>
__global__ __launch_bounds__(KWL == 3 ? 512 : 256) void quadreg_kernel(const uint16_t* x, const uint32_t* qw,
                                                                        const uint16_t* qs, void* y, int rows, int N, int K,
                                                                        uint32_t w0, uint32_t flags, const QuadRegTail t) {
  constexpr int G = GemvTraits<BITS>::G;
  constexpr int CH = GemvTraits<BITS>::CH;
  constexpr int KW = 1 << KWL;
  constexpr int WPB = KWL == 3 ? 8 : 4;
  constexpr bool EXTRA = MODE == 1, PAIRED = MODE == 2;
  constexpr uint32_t kMagic = BF ? 0x43004300u : 0x64006400u;
  auto to_f32 = [](uint16_t bits) { return BF ? bf2f(bits) : h2f(bits); };
  auto to_out = [](float v) { return BF ? f2bf(v) : f2h(v); };
  auto mm = [](uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, float4_t c) {
    return BF ? qr_mfma4_bf16(a0, a1, b0, b1, c) : qr_mfma4(a0, a1, b0, b1, c);
  };

  extern __shared__ float4 part_lds[];  // [wave][round][batch quad][4 lanes]

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int gw = blockIdx.x * WPB + wave;
  const int ksub = gw & (KW - 1);
  const int walker = gw >> KWL;
  const int nwalkers = static_cast<int>(w0 & 0xffffu), rounds = static_cast<int>(w0 >> 16);
  const int ng = (K + G - 1) / G, nw = 4 * ng, nquads = N >> 2;
  const int li = lane & 3;   // weight row of the quad (A), activation row of the batch quad (B, D)
  const int ks = lane >> 2;  // block: group 16 * iteration + ks
  const bool out_f32 = (flags & kQrOutF32) != 0;

  // ---- this wave's slice of x goes out first (it is needed first, and loads retire in issue order).  Tile (bq, u) is
  //      4 activation rows x the 16 groups of iteration ksub * U + u: CPR 16-byte chunks per row, contiguous in memory;
  //      load i of a lane is chunk (64 * i + lane) of the tile in row-major order
  constexpr int CPR = 16 * CH;          // chunks per row of a tile
  constexpr int RB = CPR * 16 + 16;     // bytes between the rows of a tile in LDS (padded: conflict-free operand reads)
  uint4 xo[NBQ][U][CH];
  float cneg[NBQ][U];
#pragma unroll
  for (int bq = 0; bq < NBQ; ++bq)
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k0 = (ksub * U + u) * 16 * G;
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        const int f = 64 * i + lane;
        const int r = f / CPR, ch = f - r * CPR;
        const int b = 4 * bq + r, k = k0 + 8 * ch;
        const bool ok = b < rows && k + 8 <= K;
        // (an aligned, valid address either way: the base of x where the chunk lies outside; zeroed)
        xo[bq][u][i] = *reinterpret_cast<const uint4*>(ok ? x + static_cast<int64_t>(b) * K + k : x);
        if (!ok) xo[bq][u][i] = make_uint4(0, 0, 0, 0);
      }
    }

  // ---- weight / scale loads of one quad.  Branch-free: every path issues the same loads, so the wait counts let the
  //      other buffer's loads stay in flight across the loop; a quad past the end reads one cached line instead.
  uint4 wa[U], wb[U];
  uint32_t sa[U], sb[U];  // fp16 bits, 32 bits wide so that in-flight values are never re-packed
  auto issue = [&](int quad, uint4 (&wn)[U], uint32_t (&sn)[U]) {
    const bool live = quad < nquads;
    int row = min(quad * 4 + li, N - 1);
    if (PAIRED) row = gate_up_row(row, N);
    const uint32_t* wr = qw + static_cast<int64_t>(row) * nw;
    const uint16_t* sr = qs + static_cast<int64_t>(row) * ng;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int g = min((ksub * U + u) * 16 + ks, ng - 1);
      wn[u] = *reinterpret_cast<const uint4*>(live ? wr + 4 * g : qw);
      sn[u] = *(live ? sr + g : qs);
    }
  };
  const int q_first = walker < nwalkers ? walker : nquads;  // (waves past the last walker have no quads)
  int qa = q_first, qb = q_first + nwalkers;
  issue(qa, wa, sa);
  issue(qb, wb, sb);

  // ---- x into operand order, in place: pairs as the unpack masks produce them; the activations of the scaled operand
  //      classes divided by their power of two (so that one accumulator takes every class), and minus the offset term
  //      formed from the divided values (see gq_quadrow.hip)
  char* const xtile = reinterpret_cast<char*>(part_lds) + WPB * rounds * NBQ * 64 + wave * (4 * RB);
#pragma unroll
  for (int bq = 0; bq < NBQ; ++bq)
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // through this wave's LDS tile: written as loaded (row-major), read back as (row li, group ks).  A wave's LDS
      // instructions execute in order, so the reads see the writes and the next tile's writes come after these reads.
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        const int f = 64 * i + lane;
        const int r = f / CPR, ch = f - r * CPR;
        *reinterpret_cast<uint4*>(xtile + r * RB + ch * 16) = xo[bq][u][i];
      }
      __builtin_amdgcn_wave_barrier();
      uint32_t nat[G / 2], xr[G / 2];
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const uint4 v = *reinterpret_cast<const uint4*>(xtile + li * RB + ks * (2 * G) + c * 16);
        nat[4 * c + 0] = v.x; nat[4 * c + 1] = v.y; nat[4 * c + 2] = v.z; nat[4 * c + 3] = v.w;
      }
      __builtin_amdgcn_wave_barrier();
      float corr = permute_group<BITS, BF>(nat, xr);
      const half2_t r16 = {static_cast<_Float16>(0.0625f), static_cast<_Float16>(0.0625f)};
      const half2_t r8 = {static_cast<_Float16>(0.125f), static_cast<_Float16>(0.125f)};
      const half2_t r64 = {static_cast<_Float16>(0.015625f), static_cast<_Float16>(0.015625f)};
      if constexpr (BF) {
        // (no rescaling: every field was shifted down to the low bits, the offset term is permute_group's)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          if constexpr (BITS == 4) xo[bq][u][c] = make_uint4(xr[4 * c + 0], xr[4 * c + 2], xr[4 * c + 1], xr[4 * c + 3]);
          else xo[bq][u][c] = make_uint4(xr[5 * c + 0], xr[5 * c + 3], xr[5 * c + 1], xr[5 * c + 4]);
        }
        if constexpr (BITS == 3) xo[bq][u][CH - 1] = make_uint4(xr[2], xr[7], xr[12], xr[17]);
      } else if constexpr (BITS == 4) {
        corr = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          xr[4 * c + 1] = as_u32(as_half2(xr[4 * c + 1]) * r16);
          xr[4 * c + 3] = as_u32(as_half2(xr[4 * c + 3]) * r16);
          corr = dot2(xr[4 * c + 0], 0x64076407u /* (1031, 1031) */, corr);
          corr = dot2(xr[4 * c + 1], 0x64706470u /* (16 * 71, ..) */, corr);
          corr = dot2(xr[4 * c + 2], 0x64076407u, corr);
          corr = dot2(xr[4 * c + 3], 0x64706470u, corr);
          xo[bq][u][c] = make_uint4(xr[4 * c + 0], xr[4 * c + 2], xr[4 * c + 1], xr[4 * c + 3]);
        }
      } else {
        corr = 0.f;
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
          xo[bq][u][c] = make_uint4(xr[5 * c + 0], xr[5 * c + 3], xr[5 * c + 1], xr[5 * c + 4]);
        }
        // fields (2,7) of all four words, the x64 class, share the fifth word
        xo[bq][u][CH - 1] = make_uint4(xr[2], xr[7], xr[12], xr[17]);
      }
      cneg[bq][u] = -corr;
    }

  // the four results of (activation row b, quad) leave in the output's type
  auto put = [&](int quad, int b, float (&v)[4]) {
    const int64_t oi = static_cast<int64_t>(b) * N + quad * 4;
    if constexpr (EXTRA) {
      if (t.bias != nullptr) {
        const uint2 bb = *reinterpret_cast<const uint2*>(t.bias + quad * 4);
        v[0] += to_f32(static_cast<uint16_t>(bb.x & 0xffffu)); v[1] += to_f32(static_cast<uint16_t>(bb.x >> 16));
        v[2] += to_f32(static_cast<uint16_t>(bb.y & 0xffffu)); v[3] += to_f32(static_cast<uint16_t>(bb.y >> 16));
      }
      if (t.residual != nullptr) {
        const uint2 rr = *reinterpret_cast<const uint2*>(t.residual + oi);
        v[0] += to_f32(static_cast<uint16_t>(rr.x & 0xffffu)); v[1] += to_f32(static_cast<uint16_t>(rr.x >> 16));
        v[2] += to_f32(static_cast<uint16_t>(rr.y & 0xffffu)); v[3] += to_f32(static_cast<uint16_t>(rr.y >> 16));
      }
    }
    if constexpr (PAIRED) {
      *reinterpret_cast<uint32_t*>(static_cast<uint16_t*>(y) + (oi >> 1)) =
          static_cast<uint32_t>(silu_mul_t<BF>(v[0], v[1])) | (static_cast<uint32_t>(silu_mul_t<BF>(v[2], v[3])) << 16);
    } else if (out_f32) {
      *reinterpret_cast<float4*>(static_cast<float*>(y) + oi) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
      uint2 o;
      o.x = static_cast<uint32_t>(to_out(v[0])) | (static_cast<uint32_t>(to_out(v[1])) << 16);
      o.y = static_cast<uint32_t>(to_out(v[2])) | (static_cast<uint32_t>(to_out(v[3])) << 16);
      *reinterpret_cast<uint2*>(static_cast<uint16_t*>(y) + oi) = o;
    }
  };

  // ---- persistent walk
  int done = 0;  // quads this wave has been through
  auto compute = [&](int quad, const uint4 (&wc)[U], const uint32_t (&sc)[U]) {
    float4_t acc[NBQ];
#pragma unroll
    for (int bq = 0; bq < NBQ; ++bq) acc[bq] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // A operands: q4 lo/hi = even / odd fields (x1, x16) of word d; q3 lo/hi = the x1 / x8 fields of word d,
      // a64 = the x64 field pairs of words (0,1) and (2,3)
      uint32_t lo[4][2], hi[4][2], a64[2][2];
      const uint32_t w[4] = {wc[u].x, wc[u].y, wc[u].z, wc[u].w};
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        if constexpr (BITS == 4) {
          const uint32_t w8 = w[d] >> 8;
          lo[d][0] = and_or_c(w[d], 0x000f000fu, kMagic);
          lo[d][1] = and_or_c(w8, 0x000f000fu, kMagic);
          if constexpr (BF) {
            hi[d][0] = and_or_c(w[d] >> 4, 0x000f000fu, kMagic);
            hi[d][1] = and_or_c(w[d] >> 12, 0x000f000fu, kMagic);
          } else {
            hi[d][0] = and_or_c(w[d], 0x00f000f0u, kMagic);
            hi[d][1] = and_or_c(w8, 0x00f000f0u, kMagic);
          }
        } else {
          // low half keeps fields 0-4, high half gets fields 5-9 aligned to bit 16
          const uint32_t tt = (w[d] & 0x0000ffffu) | ((w[d] << 1) & 0xffff0000u);
          const uint32_t t9 = tt >> 9;
          lo[d][0] = and_or_c(tt, 0x00070007u, kMagic);   // fields (0,5)
          lo[d][1] = and_or_c(t9, 0x00070007u, kMagic);   // fields (3,8)
          if constexpr (BF) {
            hi[d][0] = and_or_c(tt >> 3, 0x00070007u, kMagic);   // fields (1,6)
            hi[d][1] = and_or_c(tt >> 12, 0x00070007u, kMagic);  // fields (4,9)
            a64[d >> 1][d & 1] = and_or_c(tt >> 6, 0x00070007u, kMagic);  // fields (2,7)
          } else {
            hi[d][0] = and_or_c(tt, 0x00380038u, kMagic);   // fields (1,6) x 8
            hi[d][1] = and_or_c(t9, 0x00380038u, kMagic);   // fields (4,9) x 8
            a64[d >> 1][d & 1] = and_or_c(tt, 0x01c001c0u, kMagic);  // fields (2,7) x 64
          }
        }
      }
      // the four rows' scales of this block: lane 4b+i holds row i's (converted once, then broadcast)
      const uint32_t s32 = __builtin_bit_cast(uint32_t, to_f32(static_cast<uint16_t>(sc[u])));
      float sv[4];
      sv[0] = __builtin_bit_cast(float, qr_dpp_u<0x00>(s32));
      sv[1] = __builtin_bit_cast(float, qr_dpp_u<0x55>(s32));
      sv[2] = __builtin_bit_cast(float, qr_dpp_u<0xAA>(s32));
      sv[3] = __builtin_bit_cast(float, qr_dpp_u<0xFF>(s32));
#pragma unroll
      for (int bq = 0; bq < NBQ; ++bq) {
        // one accumulator per group: it starts from minus the offset term and takes every operand class
        const float c = cneg[bq][u];
        float4_t tacc = {c, c, c, c};
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          tacc = mm(lo[d][0], lo[d][1], xo[bq][u][d].x, xo[bq][u][d].y, tacc);
          tacc = mm(hi[d][0], hi[d][1], xo[bq][u][d].z, xo[bq][u][d].w, tacc);
        }
        if constexpr (BITS == 3) {
          tacc = mm(a64[0][0], a64[0][1], xo[bq][u][CH - 1].x, xo[bq][u][CH - 1].y, tacc);
          tacc = mm(a64[1][0], a64[1][1], xo[bq][u][CH - 1].z, xo[bq][u][CH - 1].w, tacc);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[bq][i] = fmaf(sv[i], tacc[i], acc[bq][i]);
      }
    }
    // The 16 blocks of this wave's share, summed across lanes.  Two rotations inside each row of 16 lanes leave the
    // row's sum of value i in all four lanes of a batch row; lane (li, j = block % 4) then keeps value j alone, so the
    // two steps across rows run on one register instead of four, and lanes 0..15 end with the 4 x 4 results of the quad.
    const int jsel = ks & 3;
#pragma unroll
    for (int bq = 0; bq < NBQ; ++bq) {
      float sr[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float s = acc[bq][i];
        // (rotation by 8 first: it pairs lanes l and l ^ 8, so both hold the same bits; the rotation by 4 then adds the
        //  two pair sums, in either order: all four lanes of a batch row end with the same bits, and a row's result
        //  does not depend on its position in the quad - which differs between the plain and the gate/up walk)
        s += dpp_f<0x128>(s);  // row_ror:8
        s += dpp_f<0x124>(s);  // row_ror:4: every lane holds the sum over its row of 16 lanes
        sr[i] = s;
      }
      float w = jsel == 0 ? sr[0] : (jsel == 1 ? sr[1] : (jsel == 2 ? sr[2] : sr[3]));
      w += __shfl_xor(w, 16, kWave);
      w += __shfl_xor(w, 32, kWave);
      // (weight row jsel of the quad, activation row 4 * bq + li); waits in LDS as [activation row][weight row]
      if (lane < 16 && 4 * bq + li < rows && quad < nquads)
        reinterpret_cast<float*>(part_lds)[((wave * rounds + done) * NBQ + bq) * 16 + li * 4 + jsel] = w;
    }
    ++done;
  };

  // (the scheduling barriers keep each refill ahead of the next quad's arithmetic)
  while (qa < nquads) {
    compute(qa, wa, sa);
    qa += 2 * nwalkers;
    issue(qa, wa, sa);
    __builtin_amdgcn_sched_barrier(0);
    compute(qb, wb, sb);  // past the end: nothing is kept
    qb += 2 * nwalkers;
    issue(qb, wb, sb);
    __builtin_amdgcn_sched_barrier(0);
  }

  {
    // the shares meet: the first wave of each group adds them in wave order, 16 quads per pass (lane = 4 * quad + row)
    __syncthreads();
    if (ksub == 0 && walker < nwalkers) {
      for (int r = lane >> 2; r < rounds; r += 16) {
        const int quad = walker + r * nwalkers;
        if (quad >= nquads) break;
#pragma unroll
        for (int bq = 0; bq < NBQ; ++bq) {
          const int b = 4 * bq + li;
          if (b < rows) {
            float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < KW; ++j) {
              const float4 pv = part_lds[(((wave + j) * rounds + r) * NBQ + bq) * 4 + li];
              v[0] += pv.x; v[1] += pv.y; v[2] += pv.z; v[3] += pv.w;
            }
            put(quad, b, v);
          }
        }
      }
    }
  }
}

template <int BITS, int NBQ, int U, int KWL, bool BF>
hipError_t launch_mode(const GemmArgs& a, int nwalkers, int rounds, hipStream_t s) {
  constexpr int WPB = KWL == 3 ? 8 : 4;
  const int mode = a.paired ? 2 : ((a.bias != nullptr || a.residual != nullptr) ? 1 : 0);
  constexpr int kTile = 4 * (16 * GemvTraits<BITS>::CH * 16 + 16);  // a wave's tile of x
  const size_t lds = static_cast<size_t>(WPB) * rounds * NBQ * 64 + static_cast<size_t>(WPB) * kTile;
  if (lds > 64 * 1024 || nwalkers > 0xffff || rounds > 0xffff) return hipErrorNotSupported;
  const int waves = nwalkers << KWL;
  const dim3 grid((waves + WPB - 1) / WPB), block(WPB * 64);
  const uint32_t w0 = static_cast<uint32_t>(nwalkers) | static_cast<uint32_t>(rounds) << 16;
  const uint32_t flags = a.out_f32 ? kQrOutF32 : 0u;
  const QuadRegTail t{a.bias, a.residual};
  note_kernel("gq::quadreg_kernel<%d,%d,%d,%d,%d%s>", BITS, NBQ, U, KWL, mode, BF ? ",true" : "");
  const int rows = static_cast<int>(a.rows), N = static_cast<int>(a.N), K = static_cast<int>(a.K);
#define GQ_QR_LAUNCH(MODE_) \
  hipLaunchKernelGGL((quadreg_kernel<BITS, NBQ, U, KWL, MODE_, BF>), grid, block, lds, s, a.x, a.q_weight, a.q_scale, a.y, \
                     rows, N, K, w0, flags, t)
  if (mode == 2) GQ_QR_LAUNCH(2);
  else if (mode == 1) GQ_QR_LAUNCH(1);
  else GQ_QR_LAUNCH(0);
#undef GQ_QR_LAUNCH
  return hipGetLastError();
}

template <int BITS, int NBQ, bool BF = false>
hipError_t launch_shape(const GemmArgs& a, int U, int kwl, int nwalkers, int rounds, hipStream_t s) {
#define GQ_QR_CASE(U_, KWL_) \
  if (U == U_ && kwl == KWL_) return launch_mode<BITS, NBQ, U_, KWL_, BF>(a, nwalkers, rounds, s);
  GQ_QR_CASE(1, 0) GQ_QR_CASE(2, 0) GQ_QR_CASE(1, 1) GQ_QR_CASE(2, 1)
  GQ_QR_CASE(1, 2) GQ_QR_CASE(2, 2) GQ_QR_CASE(1, 3) GQ_QR_CASE(2, 3)
  if constexpr (NBQ == 1) {  // (two batch quads stop at two iterations per wave)
    GQ_QR_CASE(3, 0) GQ_QR_CASE(4, 0) GQ_QR_CASE(3, 1) GQ_QR_CASE(4, 1)
    GQ_QR_CASE(3, 2) GQ_QR_CASE(4, 2) GQ_QR_CASE(3, 3) GQ_QR_CASE(4, 3)
  }
#undef GQ_QR_CASE
  return hipErrorNotSupported;
}

}  // namespace

// Plain linears (no expert segments, no gather) of up to 8 float16 (q4: also bfloat16) activation rows with N % 4 == 0 and K % 8 == 0
// and K of at most 16 iterations of 16 groups (q4: K <= 8192; q3: K <= 10240); hipErrorNotSupported otherwise.
// Tuning overrides: quad_ksplit (log2 of the waves per quad), gemv_waves (waves in all).
hipError_t launch_quadreg(const GemmArgs& a, int rows_max, hipStream_t s) {
  if (a.bits != 4 && a.bits != 3) return hipErrorNotSupported;
  const int G = a.bits == 4 ? 32 : 40;
  if (a.group_size != G || a.indptr != nullptr || a.x_rows != nullptr) return hipErrorNotSupported;
  if (a.bf16 && a.bits != 4) return hipErrorNotSupported;  // (the bfloat16 instances: q4bf16_*)
  if (a.rows == 0 || a.N == 0) return hipSuccess;
  if (rows_max > 8 || a.rows > 8 || (a.N & 3) != 0 || (a.K & 7) != 0 || a.K == 0) return hipErrorNotSupported;
  if ((reinterpret_cast<uintptr_t>(a.x) & 15) != 0 || (reinterpret_cast<uintptr_t>(a.y) & 15) != 0 ||
      (reinterpret_cast<uintptr_t>(a.bias) & 7) != 0 || (reinterpret_cast<uintptr_t>(a.residual) & 7) != 0 ||
      (reinterpret_cast<uintptr_t>(a.q_weight) & 15) != 0)
    return hipErrorNotSupported;
  const int nbq = a.rows <= 4 ? 1 : 2;
  const int ng = static_cast<int>((a.K + G - 1) / G);
  const int niter = (ng + 15) / 16;
  // Long K (q4: beyond 8192) stays with the kernel that stages x once per workgroup: every group of waves here reads
  // all of x for itself, and at 4 rows of K = 14336 that is as many bytes as the weights (measured equal at best).
  if (niter > 16) return hipErrorNotSupported;
  // q3f16_1 (ten matrix instructions and five words of x per group): ahead only on the smallest projections (4096 x 4096
  // at 4 / 8 rows 6.2 / 8.3 us against 6.5 / 8.9; 12288 x 4096 equal at 4 rows and behind at 8, 22016 x 4096 behind)
  if (a.bits == 3 && a.N > 4096 && options().gemv_variant != 9) return hipErrorNotSupported;
  // iterations per wave: the registers of x are NBQ * U * (4 * CH + 1); two batch quads at four iterations would leave
  // one wave per SIMD, so they stop at 2
  const int umax = nbq == 2 ? 2 : 4;
  const int nquads = static_cast<int>(a.N / 4);
  int kwl = 0;
  const int opt = options().quad_ksplit;
  if (opt >= 0) {
    if (opt > 3) return hipErrorNotSupported;
    kwl = opt;
  } else {
    // Measured on the Llama-3-8B projections (graph replay over rotating weights, 4 / 8 rows): few quads want the
    // shortest chains (8 waves per quad: 4096 x 4096 4.8 / 5.9 us against 5.3 / 6.6 with 4, 6144 x 4096 5.8 / 7.1 against
    // 6.2 / 8.0), 28672 x 4096 wants 4 (13.9 / 18.0 us; 8 waves 14.0 / 19.7), 128256 x 4096 at 4 rows wants 2 on 1024
    // waves (49.5 us against 52.6)
    kwl = nquads <= 2048 ? 3 : ((nquads <= 16384 || nbq == 2) ? 2 : 1);
    while (kwl < 3 && (niter + (1 << kwl) - 1) / (1 << kwl) > umax) ++kwl;
    while (kwl > 0 && niter < (1 << kwl)) --kwl;  // (every wave keeps at least one iteration)
  }
  const int U = (niter + (1 << kwl) - 1) / (1 << kwl);
  if (U > umax || U < 1) return hipErrorNotSupported;
  int waves = options().gemv_waves > 0 ? options().gemv_waves : ((nquads > 16384 && nbq == 1) ? 1024 : 2048);
  int nwalkers = waves >> kwl;
  if (nwalkers < 1) nwalkers = 1;
  if (nwalkers > nquads) nwalkers = nquads;
  const int rounds = (nquads + nwalkers - 1) / nwalkers;
  nwalkers = (nquads + rounds - 1) / rounds;  // even share of quads per walker
  if (a.bf16) return nbq == 1 ? launch_shape<4, 1, true>(a, U, kwl, nwalkers, rounds, s) : launch_shape<4, 2, true>(a, U, kwl, nwalkers, rounds, s);
  if (a.bits == 4) return nbq == 1 ? launch_shape<4, 1>(a, U, kwl, nwalkers, rounds, s) : launch_shape<4, 2>(a, U, kwl, nwalkers, rounds, s);
  return nbq == 1 ? launch_shape<3, 1>(a, U, kwl, nwalkers, rounds, s) : launch_shape<3, 2>(a, U, kwl, nwalkers, rounds, s);
}

}  // namespace gq
