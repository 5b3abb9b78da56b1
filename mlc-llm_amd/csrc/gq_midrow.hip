// Matmul for 9..64 activation rows against streamed q4f16_1 (q4bf16_1) weights (batched decode, short prefill chunks):
// v_mfma_f32_16x16x32_f16 on UNSCALED weight operands, the group's scale applied to the matrix instruction's result,
// the activations resident in registers.
//
// Same callers as the few-row tiles of gq_gemm_pipe.hip and as gq_skinny.hip (GroupQuantizeLinear.forward,
// python/mlc_llm/quantization/group_quantization.py:390-437, for the batch buckets above the low-batch GEMV of
// python/mlc_llm/compiler_pass/low_batch_specialization.py:22-57).
//
// Those kernels materialise fp16 weights (q - 7) * s for the matrix core: unpack, subtract, multiply, and for the
// tiles that go through LDS a byte permute into natural k order, 3.4 to 5 vector instructions per weight and lane,
// which is what bounds them in this regime (the weight stream itself would take half their time).  Here the matrix
// instruction multiplies x by the integers 1024 + q (q4 fields OR-ed into the mantissa of 1024.0: one v_and_or per
// field pair, odd fields come out times 16 and meet activations divided by 16), one instruction per quantisation
// group, so that the group's scale multiplies four accumulator values per lane afterwards and the offset
// -(1024 + 7) * sum(x) of the group enters as the instruction's C operand: the arithmetic of the 4x4x4 kernels
// (gq_quadrow.hip), about ten vector instructions per group of 512 weights and wave at 16 rows.
//
// B operand of instruction g = group g of 16 weight rows (a "tile"): lane (c = lane % 16, j = lane / 16) supplies the
// 8 k of storage word j of row c.  A lane LOADS a whole group (128 bits: lane (c, j) group 4 * step + j of row c, so a
// wave instruction covers 16 rows x 64 contiguous bytes); a 4 x 4 transpose across the four 16-lane rows
// (v_permlane32_swap, v_permlane16_swap: four instructions) then leaves register m of lane (c, j) with word j of group
// 4 * step + m.  A operand = 16 activation rows x the same 32 k: lane (i, j) holds x[i][32 g + 8 j ..] in the pair
// order of the unpack masks, the odd fields' activations divided by 16; it reads those 16 bytes straight from global
// memory once and keeps them.  The offset term needs no cross-lane sum either: the same matrix instruction on a
// constant B operand (-1031 for the even fields, -16 * 71 for the odd ones) leaves -(offset) of rows 4 j .. 4 j + 3 in
// lane (c, j), which is where the C operand wants it.  D: lane (c, j) receives rows 4 j .. 4 j + 3 of column c, four
// values of the lane's own weight row: its scale of the group multiplies them into the fp32 accumulators.
//
// A wave owns U consecutive groups of K (its x: 4 registers per group and batch tile, the offsets as many where they are
// kept) and walks tiles with RT tiles of loads in flight.  The 16 waves of a workgroup are KW neighbouring K shares x
// 16 / KW tiles side by side; results wait in LDS until the walk is over (a store inside the walk would turn every wait
// for a load into a wait for all of them), then the K shares are added and leave.  K beyond a workgroup's KW * U groups
// is walked in phases: each phase loads its share of x and visits every tile again (its own K range of it: the weights
// are still read once), adding to the sums in LDS.  Expert segments (moe_matmul.dequantize_group_gemm,
// python/mlc_llm/op/moe_matmul.py:562-768): grid row = expert, rows from indptr, more rows than the batch tiles hold in
// passes.  The fused gate/up form walks a gate tile and its up tile in consecutive rounds and folds silu(gate) * up into
// the step that adds the K shares.
#include "gq_gemm_common.hpp"
#include "gq_gemv_common.hpp"

namespace gq {

namespace {

struct MidParams {
  const uint16_t* x;
  const uint32_t* qw;
  const uint16_t* qs;
  const uint16_t* bias;
  const uint16_t* residual;
  void* y;
  const void* indptr;      // null: one segment [0, rows)
  const int32_t* x_rows;   // null, or the row of x each activation row reads
  int64_t expert_w_stride, expert_s_stride;
  int rows, N, K, ng, nw;
  int ntiles;              // tiles of 16 weight rows a walk visits: ceil(N / 16); the fused gate/up form: N / 32 pairs
  int rounds;              // tiles a wave walks per chunk (a multiple of the tiles in flight; the fused form: even)
  int chunks;              // chunks of rounds (1 when K takes phases)
  int phases;              // passes over K (a workgroup covers KW * U groups per phase)
  int slices;              // workgroups along K (plain linears with a workspace: grid z; each covers one phase's worth of
                           // K and leaves fp32 partial sums [slice][rows][N] in y for the reduction kernel)
  int kw_log2;             // log2 of the waves that share a tile's K
  int out_f32, paired, indptr_i64, x_src_rows;
};

// T[j][m] (register m of the lanes 16 j .. 16 j + 15) -> T[m][j]
__device__ __forceinline__ void mid_transpose(uint32_t& r0, uint32_t& r1, uint32_t& r2, uint32_t& r3) {
  auto a = __builtin_amdgcn_permlane32_swap(r0, r2, false, false);  // upper half of r0 <-> lower half of r2
  auto b = __builtin_amdgcn_permlane32_swap(r1, r3, false, false);
  auto c = __builtin_amdgcn_permlane16_swap(a[0], b[0], false, false);  // odd rows of the first <-> even rows of the second
  auto d = __builtin_amdgcn_permlane16_swap(a[1], b[1], false, false);
  r0 = c[0]; r1 = c[1]; r2 = d[0]; r3 = d[1];
}

typedef uint32_t mid_u4 __attribute__((ext_vector_type(4)));

template <bool BF>
__device__ __forceinline__ float4_t mid_mfma(const mid_u4 a, const mid_u4 b, const float4_t c) {
  if constexpr (BF) {
    typedef __bf16 mid_bf8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mid_bf8, a), __builtin_bit_cast(mid_bf8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
  }
}

// NBT: batch tiles of 16 rows; U: groups of K a wave owns (4 or 8); RT: tiles of loads in flight per wave;
// BF: bfloat16 model (x, scales, bias, residual and the 16-bit result are bfloat16): 0x4300 | q is the bfloat16 128 + q, so
// every field is shifted down to bit 0 of its half (no x16 trick, x is not rescaled) and all carry the offset 128 + 7;
// KEEP_C: the offset terms stay in registers (else the constant-operand instruction runs again in front of each group);
// PHASED: K takes more than one phase (the sums of all of a wave's rounds stay in LDS between phases: one chunk of rounds);
// else a wave's rounds come in chunks of p.rounds, each followed by the step that adds the K shares and stores, with x
// and the ring of loads carried across
template <int NBT, int U, int RT, bool KEEP_C, bool PHASED, bool BF = false>
__global__ __launch_bounds__(1024) void midrow_kernel(const MidParams p) {
  constexpr int STEPS = U / 4;
  constexpr uint32_t kMagic = BF ? 0x43004300u : 0x64006400u;
  auto to_f32 = [](uint16_t bits) { return BF ? bf2f(bits) : h2f(bits); };
  extern __shared__ float4 res_lds[];  // [round][wave][NBT][64 lanes]

  // (the wave index in a scalar register: everything derived from it - K share, tiles, the loads' scalar offsets - is
  //  then uniform for the compiler as well, which would otherwise wrap every buffer load in a loop over lanes)
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, j = lane >> 4;
  const int kw = 1 << p.kw_log2, tw = 16 >> p.kw_log2;
  const int ks = wave & (kw - 1), ti = wave >> p.kw_log2;
  const int tstride = gridDim.x * tw;
  const int base = blockIdx.x * tw + ti;  // this wave's first tile (the fused form: its first gate / up pair)
  const int half_tiles = p.N >> 5;        // (the fused form: tiles of gate rows)

  // ---- this workgroup's expert and rows
  const int expert = blockIdx.y;
  int seg_lo = 0, seg_hi = p.rows;
  if (p.indptr != nullptr) {
    if (p.indptr_i64) {
      seg_lo = static_cast<int>(static_cast<const int64_t*>(p.indptr)[expert]);
      seg_hi = static_cast<int>(static_cast<const int64_t*>(p.indptr)[expert + 1]);
    } else {
      seg_lo = static_cast<const int32_t*>(p.indptr)[expert];
      seg_hi = static_cast<const int32_t*>(p.indptr)[expert + 1];
    }
    seg_lo = max(seg_lo, 0);
    seg_hi = min(seg_hi, p.rows);
  }
  if (seg_hi <= seg_lo) return;  // (uniform: before any barrier)

  // ---- weight / scale loads of one tile, through buffer descriptors: the tensor in scalar registers, the tile as the
  //      scalar offset, one 32-bit lane offset for all tiles.  The descriptors carry the tensors' sizes: rows past N read
  //      zeros, and a tile past the end (a wave's last rounds issue for tiles that do not exist) gets the tensor's size
  //      as its offset, which puts every lane out of range: zeros, and no memory traffic.  Nothing of either is kept.
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  const uint32_t w_bytes = static_cast<uint32_t>(p.N) * static_cast<uint32_t>(p.nw) * 4u;
  const uint32_t s_bytes = static_cast<uint32_t>(p.N) * static_cast<uint32_t>(p.ng) * 2u;
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint32_t*>(p.qw + expert * p.expert_w_stride), short(0), static_cast<int>(w_bytes), 0x00020000);
  const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(p.qs + expert * p.expert_s_stride), short(0), static_cast<int>(s_bytes), 0x00020000);
  const uint32_t w_tile = 16u * static_cast<uint32_t>(p.nw) * 4u, s_tile = 16u * static_cast<uint32_t>(p.ng) * 2u;
  // round r of this wave -> tile (the fused form: rounds 2 i, 2 i + 1 = gate tile, up tile of pair i); -1 past the end.
  // Straight-line scalar arithmetic: a branch here would sit inside the walk, where every join makes the wait for one
  // tile's loads a wait for all of them.
  const int pair_shift = p.paired ? 1 : 0;
  const int up_tiles = p.paired ? half_tiles : 0;
  auto tile_of = [&](int r) -> int {
    const int item = base + (r >> pair_shift) * tstride;
    const int t = item + (r & pair_shift) * up_tiles;
    return item < p.ntiles ? t : -1;
  };

  constexpr uint32_t kLoLo = 0x05040100u, kHiHi = 0x07060302u;
  const half2_t r16 = {static_cast<_Float16>(0.0625f), static_cast<_Float16>(0.0625f)};
  const mid_u4 neg_off = BF ? mid_u4{0xc307c307u /* -135 */, 0xc307c307u, 0xc307c307u, 0xc307c307u}
                            : mid_u4{0xe407e407u /* -1031 */, 0xe407e407u, 0xe470e470u /* -16 * 71 */, 0xe470e470u};

  for (int pass_lo = seg_lo; pass_lo < seg_hi; pass_lo += 16 * NBT) {
    for (int ph = 0; ph < (PHASED ? p.phases : 1); ++ph) {
      const int ga_raw = ((static_cast<int>(blockIdx.z) + ph) * kw + ks) * U;  // (slices > 1: one phase each)
      const bool k_live = ga_raw < p.ng;  // (uniform; ng % U == 0: a share is whole or empty)
      const int ga = k_live ? ga_raw : p.ng - U;
      const int w_lane = (c * p.nw + 4 * (ga + j)) * 4, s_lane = (c * p.ng + ga) * 2;
      u32x4 w[RT][STEPS];  // (kept as whole register tuples until the point of use, see walk_tile)
      uint32_t sc[RT][U / 2];  // the U scales of this lane's row (two per register)
      auto issue = [&](int r, u32x4 (&wv)[STEPS], uint32_t (&sv)[U / 2]) {
        const int tile = tile_of(r);
        const int w_off = static_cast<int>(tile >= 0 ? static_cast<uint32_t>(tile) * w_tile : w_bytes);
        const int s_off = static_cast<int>(tile >= 0 ? static_cast<uint32_t>(tile) * s_tile : s_bytes);
#pragma unroll
        for (int st = 0; st < STEPS; ++st) {
          wv[st] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, w_lane + 64 * st, w_off, 0);
        }
        if constexpr (U == 8) {
          const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(s_rsrc, s_lane, s_off, 0);
          sv[0] = v.x; sv[1] = v.y; sv[2] = v.z; sv[3] = v.w;
        } else {
          const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(s_rsrc, s_lane, s_off, 0);
          sv[0] = v.x; sv[1] = v.y;
        }
      };
      // ---- this wave's share of x goes out first (it is needed first, and loads retire in issue order): lane (i = c, j)
      //      of batch tile bt reads x[row 16 bt + i][32 g + 8 j .. + 7]
      uint4 xraw[NBT][U];
      bool x_ok[NBT];
#pragma unroll
      for (int bt = 0; bt < NBT; ++bt) {
        const int b = pass_lo + 16 * bt + c;
        x_ok[bt] = k_live && b < seg_hi;
        const uint16_t* xrow = p.x + x_row(p.x_rows, p.x_src_rows, x_ok[bt] ? b : seg_lo) * p.K + ga * 32 + 8 * j;
#pragma unroll
        for (int u = 0; u < U; ++u) xraw[bt][u] = *reinterpret_cast<const uint4*>(xrow + u * 32);
      }
#pragma unroll
      for (int r = 0; r < RT; ++r) issue(r, w[r], sc[r]);

      // ---- x in operand order, (x0, x4) (x2, x6) (x1, x5) / 16 (x3, x7) / 16, and the offset terms
      mid_u4 xa[NBT][U];
      float4_t cc[KEEP_C ? NBT : 1][KEEP_C ? U : 1];
#pragma unroll
      for (int bt = 0; bt < NBT; ++bt) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          uint4 v = xraw[bt][u];
          if (!x_ok[bt]) v = make_uint4(0, 0, 0, 0);
          xa[bt][u][0] = __builtin_amdgcn_perm(v.z, v.x, kLoLo);
          xa[bt][u][1] = __builtin_amdgcn_perm(v.w, v.y, kLoLo);
          xa[bt][u][2] = __builtin_amdgcn_perm(v.z, v.x, kHiHi);
          xa[bt][u][3] = __builtin_amdgcn_perm(v.w, v.y, kHiHi);
          if constexpr (!BF) {
            xa[bt][u][2] = as_u32(as_half2(xa[bt][u][2]) * r16);
            xa[bt][u][3] = as_u32(as_half2(xa[bt][u][3]) * r16);
          }
          if constexpr (KEEP_C) cc[bt][u] = mid_mfma<BF>(xa[bt][u], neg_off, float4_t{0.f, 0.f, 0.f, 0.f});
        }
      }

      // one tile from a ring slot; round `next` goes into the registers it leaves
      auto walk_tile = [&](int next, u32x4 (&wv)[STEPS], uint32_t (&sv)[U / 2], float4_t (&acc)[NBT]) __attribute__((always_inline)) {
#pragma unroll
        for (int bt = 0; bt < NBT; ++bt) acc[bt] = float4_t{0.f, 0.f, 0.f, 0.f};
        // (a zero the compiler cannot see through: the offset instruction would otherwise be hoisted out of the walk,
        //  into the registers this form is there to save)
        float zero = 0.f;
        asm volatile("" : "+v"(zero));
        const float4_t zero4 = {zero, zero, zero, zero};
#pragma unroll
        for (int st = 0; st < STEPS; ++st) {
          // (the loaded tuple becomes a new value HERE and is taken apart after that: the in-place lane swaps below
          //  otherwise make the compiler copy parts of a load into other registers right behind the load itself, and
          //  that copy waits for the load)
          u32x4 t = wv[st];
          asm volatile("" : "+v"(t));
          uint32_t r[4] = {t.x, t.y, t.z, t.w};
          mid_transpose(r[0], r[1], r[2], r[3]);
#pragma unroll
          for (int m = 0; m < 4; ++m) {
            const int u = 4 * st + m;
            const uint32_t w8 = r[m] >> 8;
            const mid_u4 bw = BF ? mid_u4{and_or_c(r[m], 0x000f000fu, kMagic), and_or_c(w8, 0x000f000fu, kMagic),
                                          and_or_c(r[m] >> 4, 0x000f000fu, kMagic), and_or_c(r[m] >> 12, 0x000f000fu, kMagic)}
                                 : mid_u4{and_or_c(r[m], 0x000f000fu, kMagic), and_or_c(w8, 0x000f000fu, kMagic),
                                          and_or_c(r[m], 0x00f000f0u, kMagic), and_or_c(w8, 0x00f000f0u, kMagic)};
            const float s = to_f32(static_cast<uint16_t>((u & 1) ? sv[u >> 1] >> 16 : sv[u >> 1] & 0xffffu));
            // (float16 without the kept offsets: the offsets come off the weight operand instead, exactly - 1024 + q - 1031
            //  and 1024 + 16 q - 16 * 71 are small integers -, four packed adds per group whatever the batch tiles, in place
            //  of one more matrix instruction per group and batch tile)
            constexpr bool SUB = !KEEP_C && !BF;
            mid_u4 bo = bw;
            if constexpr (SUB) {
              const half2_t o_lo = {static_cast<_Float16>(-1031.f), static_cast<_Float16>(-1031.f)};
              const half2_t o_hi = {static_cast<_Float16>(-1136.f), static_cast<_Float16>(-1136.f)};
              bo[0] = as_u32(as_half2(bw[0]) + o_lo); bo[1] = as_u32(as_half2(bw[1]) + o_lo);
              bo[2] = as_u32(as_half2(bw[2]) + o_hi); bo[3] = as_u32(as_half2(bw[3]) + o_hi);
            }
#pragma unroll
            for (int bt = 0; bt < NBT; ++bt) {
              float4_t c0;
              if constexpr (KEEP_C) c0 = cc[bt][u];
              else if constexpr (SUB) c0 = float4_t{0.f, 0.f, 0.f, 0.f};
              else c0 = mid_mfma<BF>(xa[bt][u], neg_off, zero4);
              const float4_t d = mid_mfma<BF>(xa[bt][u], SUB ? bo : bw, c0);
#pragma unroll
              for (int q = 0; q < 4; ++q) acc[bt][q] = fmaf(s, d[q], acc[bt][q]);
            }
          }
        }
        // (after the arithmetic: the loads then land in the very registers the tile has left, with no copies whose
        //  wait would drain the queue)
        issue(next, wv, sv);
      };

      // ---- the K shares of a tile meet: 256 values per (round, tile lane, batch tile); thread (jq, cq) takes row
      //      16 bt + jq of column cq, so that 16 neighbouring threads store 16 neighbouring columns
      auto finish = [&](int r0) __attribute__((always_inline)) {
        const float* const res = reinterpret_cast<const float*>(res_lds);
        const int sub = threadIdx.x & 255, cq = sub & 15, jq = sub >> 4;
        const int at = (((jq >> 2) * 16 + cq) << 2) + (jq & 3);  // lane (cq, jq / 4), value jq % 4
        auto share_sum = [&](int round, int tl, int bt) {
          float v = 0.f;
          for (int k = 0; k < kw; ++k) v += res[(((round * 16 + (tl << p.kw_log2) + k) * NBT + bt) << 8) + at];
          return v;
        };
        if (p.paired) {
          const int items = (p.rounds >> 1) * tw * NBT;
          const int half = p.N >> 1;
          for (int it = threadIdx.x >> 8; it < items; it += 4) {
            const int bt = it % NBT, rest = it / NBT, tl = rest % tw, pr = rest / tw;
            const int pair = blockIdx.x * tw + tl + ((r0 >> 1) + pr) * tstride;
            const int col = pair * 16 + cq, b = pass_lo + 16 * bt + jq;
            if (pair >= p.ntiles || b >= seg_hi) continue;
            const float gate = share_sum(2 * pr, tl, bt), up = share_sum(2 * pr + 1, tl, bt);
            static_cast<uint16_t*>(p.y)[static_cast<int64_t>(b) * half + col] = silu_mul_t<BF>(gate, up);
          }
        } else {
          const int items = p.rounds * tw * NBT;
          for (int it = threadIdx.x >> 8; it < items; it += 4) {
            const int bt = it % NBT, rest = it / NBT, tl = rest % tw, round = rest / tw;
            const int t = blockIdx.x * tw + tl + (r0 + round) * tstride;
            const int col = t * 16 + cq, b = pass_lo + 16 * bt + jq;
            if (t >= p.ntiles || col >= p.N || b >= seg_hi) continue;
            float v = share_sum(round, tl, bt);
            const int64_t oi = static_cast<int64_t>(b) * p.N + col;
            if (p.slices > 1) {  // (bias, residual and the cast belong to the reduction)
              static_cast<float*>(p.y)[static_cast<int64_t>(blockIdx.z) * p.rows * p.N + oi] = v;
              continue;
            }
            if (p.bias != nullptr) v += to_f32(p.bias[col]);
            if (p.residual != nullptr) v += to_f32(p.residual[oi]);
            if (p.out_f32) static_cast<float*>(p.y)[oi] = v;
            else static_cast<uint16_t*>(p.y)[oi] = BF ? f2bf(v) : f2h(v);
          }
        }
      };

      // ---- the walk: p.rounds is a multiple of RT (rounds past the last tile read nothing and leave zeros in LDS slots
      //      that nobody reads).  Later phases add to what the earlier ones left (the read is unconditional and the
      //      first phase drops it: no branch inside the walk).
      for (int chunk = 0; chunk < p.chunks; ++chunk) {
        const int r0 = chunk * p.rounds;
        for (int round = 0; round < p.rounds; round += RT) {
#pragma unroll
          for (int slot = 0; slot < RT; ++slot) {
            float4_t acc[NBT];
            walk_tile(r0 + round + slot + RT, w[slot], sc[slot], acc);
#pragma unroll
            for (int bt = 0; bt < NBT; ++bt) {
              float4* const at = res_lds + (((round + slot) * 16 + wave) * NBT + bt) * 64 + lane;
              if constexpr (PHASED) {
                const float4 old = *at;
                const bool add = ph > 0;
                *at = make_float4(acc[bt][0] + (add ? old.x : 0.f), acc[bt][1] + (add ? old.y : 0.f),
                                  acc[bt][2] + (add ? old.z : 0.f), acc[bt][3] + (add ? old.w : 0.f));
              } else {
                *at = make_float4(acc[bt][0], acc[bt][1], acc[bt][2], acc[bt][3]);
              }
            }
            __builtin_amdgcn_sched_barrier(0);  // (each refill stays ahead of the next tile's arithmetic)
          }
        }
        if (!PHASED || ph + 1 == p.phases) {  // (uniform)
          __syncthreads();
          finish(r0);
          __syncthreads();  // (the next chunk, or the next pass, writes the same LDS slots)
        }
      }
    }
  }
}

// y[b][j] = silu(sum over slices of part[s][b][j]) * (sum over slices of part[s][b][N / 2 + j]), in the model dtype
__global__ __launch_bounds__(256) void mid_reduce_silu_kernel(const float* __restrict__ part, int slices, int64_t rows, int N,
                                                              uint16_t* __restrict__ y, int bf16) {
  const int half = N >> 1;
  const int64_t count = rows * N, outs = rows * half;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < outs; i += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t b = i / half;
    const int64_t at = b * N + (i - b * half);
    float g = 0.f, u = 0.f;
    for (int sl = 0; sl < slices; ++sl) {
      g += part[sl * count + at];
      u += part[sl * count + at + half];
    }
    y[i] = bf16 ? silu_mul_bf(g, u) : silu_mul_h(g, u);
  }
}

template <int NBT, int U, int RT, bool KEEP_C, bool PHASED, bool BF = false>
hipError_t launch_mid(const MidParams& p, int wgx, int experts, hipStream_t s) {
  const size_t lds = static_cast<size_t>(p.rounds) * 16 * NBT * 1024;
  if (lds > 160 * 1024) return hipErrorNotSupported;
  if (lds > 64 * 1024) {
    static bool raised = false;  // (idempotent; a race sets the same attribute twice)
    if (!raised) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&midrow_kernel<NBT, U, RT, KEEP_C, PHASED, BF>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      if (e != hipSuccess) return e;
      raised = true;
    }
  }
  note_kernel("gq::midrow_kernel<%d,%d,%d,%d,%d%s> rounds=%d chunks=%d phases=%d slices=%d kw=%d", NBT, U, RT, int(KEEP_C),
              int(PHASED), BF ? ",true" : "", p.rounds, p.chunks, p.phases, p.slices, 1 << p.kw_log2);
  hipLaunchKernelGGL((midrow_kernel<NBT, U, RT, KEEP_C, PHASED, BF>), dim3(wgx, experts, p.slices), dim3(1024), lds, s, p);
  return hipGetLastError();
}

}  // namespace

// q4f16_1 / q4bf16_1 (float16 / bfloat16 activations, scales and results), K % 256 == 0 (a wave's eight groups: 16-byte runs of scales), N % 16 == 0 for expert
// segments and N % 32 == 0 for the fused gate/up form; any number of rows (more than the batch tiles hold: passes that read
// the weights again, so callers keep it to few rows per segment).  hipErrorNotSupported otherwise.  Tuning overrides:
// quad_ksplit (log2 of the waves that share a tile's K, minus one), gemv_waves (workgroups per expert x 16),
// gemv_rows_per_wave (1, 2: other one-batch-tile instances).
hipError_t launch_midrow(const GemmArgs& a, int rows_max, hipStream_t s) {
  if (a.bits != 4 || a.group_size != 32) return hipErrorNotSupported;
  if (a.rows < 1 || a.N < 16 || (a.K & 255) != 0 || a.K == 0) return hipErrorNotSupported;
  const bool grouped = a.indptr != nullptr;
  if (grouped && (a.N & 15) != 0) return hipErrorNotSupported;  // (an expert's tensor ends where the next begins)
  if (a.paired && ((a.N & 31) != 0 || a.bias != nullptr || a.residual != nullptr || a.out_f32)) return hipErrorNotSupported;
  if ((reinterpret_cast<uintptr_t>(a.x) & 15) != 0 || (reinterpret_cast<uintptr_t>(a.q_weight) & 15) != 0 ||
      (reinterpret_cast<uintptr_t>(a.q_scale) & 15) != 0)
    return hipErrorNotSupported;
  if (a.N * (a.K / 8) >= (int64_t(1) << 29)) return hipErrorNotSupported;  // (32-bit byte offsets with room to add)
  const int experts = grouped ? static_cast<int>(a.num_experts) : 1;
  if (experts < 1 || experts > 65535) return hipErrorNotSupported;
  MidParams p{};
  p.x = a.x; p.qw = a.q_weight; p.qs = a.q_scale; p.bias = a.bias; p.residual = a.residual; p.y = a.y;
  p.indptr = a.indptr; p.indptr_i64 = a.indptr_i64; p.x_rows = a.x_rows; p.x_src_rows = static_cast<int>(a.x_src_rows);
  p.rows = static_cast<int>(a.rows); p.N = static_cast<int>(a.N); p.K = static_cast<int>(a.K);
  p.ng = p.K / 32; p.nw = 4 * p.ng;
  p.expert_w_stride = static_cast<int64_t>(p.N) * p.nw;
  p.expert_s_stride = static_cast<int64_t>(p.N) * p.ng;
  p.paired = a.paired;
  p.ntiles = a.paired ? p.N / 32 : (p.N + 15) / 16;
  p.out_f32 = a.out_f32;
  // batch tiles per pass: one for up to 16 rows per segment, else two (more rows: passes)
  const int nbt = rows_max <= 16 ? 1 : 2;
  constexpr int U = 8;
  // waves that share a tile's K: the power of two that covers K's shares of U groups, at most 16 (a wave whose share lies
  // past K idles: one phase with 14 of 16 waves at work is ahead of two phases of 8)
  int kwl = 0;
  while (kwl < 4 && (1 << kwl) < p.ng / U) ++kwl;
  if (options().quad_ksplit >= 0) kwl = options().quad_ksplit + 1;  // (tuning override: 2, 4, 8 or 16 waves)
  p.kw_log2 = kwl;
  const int phase_groups = (1 << kwl) * U;
  p.phases = (p.ng + phase_groups - 1) / phase_groups;
  // A plain linear whose K takes several phases and whose caller brings the scratch: one workgroup row per phase's worth of
  // K instead (x stays in registers for all of a workgroup's tiles, the walk comes in chunks), fp32 partial sums in the
  // workspace and a second, small launch that adds them; the fused gate/up form then runs as a plain one and the reduction
  // folds the activation in.  Tuning override: gemv_ksplit 0 keeps the phases.
  p.slices = 1;
  bool fold_silu = false;
  if (p.phases > 1 && !grouped && p.phases <= 64 && options().gemv_ksplit != 0 && a.workspace != nullptr &&
      a.workspace_bytes >= static_cast<int64_t>(p.phases) * p.rows * p.N * 4 &&
      (reinterpret_cast<uintptr_t>(a.workspace) & 15) == 0) {
    p.slices = p.phases;
    p.phases = 1;
    p.y = a.workspace;
    p.bias = nullptr; p.residual = nullptr; p.out_f32 = 1;
    if (p.paired) {
      fold_silu = true;
      p.paired = 0;
      p.ntiles = (p.N + 15) / 16;
    }
  }
  const bool paired_walk = p.paired != 0;
  const int tw = 16 >> kwl;
  const int form = options().gemv_rows_per_wave;  // (tuning override: which one-batch-tile instance)
  const int rt = form == 2 ? 4 : (form == 4 ? 3 : 2);
  // workgroups in all: one per CU (sixteen waves of up to 128 registers fill it), each with at most 128 KiB of sums in LDS
  const int want_wg = options().gemv_waves > 0 ? options().gemv_waves / 16 : 256;
  int wgx = want_wg / (experts * p.slices);
  if (wgx < 1) wgx = 1;
  const int per_round = paired_walk ? 2 : 1;           // rounds per walked item
  const int sets = (p.ntiles + tw - 1) / tw;        // items per tile lane
  if (wgx > sets) wgx = sets;
  const int unit = paired_walk ? (rt % 2 == 0 ? rt : 2 * rt) : rt;  // rounds come in whole rings (and whole pairs)
  const int max_rounds = (128 / (16 * nbt)) / unit * unit;
  if (max_rounds < unit) return hipErrorNotSupported;
  int items = (sets + wgx - 1) / wgx;               // items per wave
  if (p.phases > 1 && items * per_round > max_rounds) {  // (one chunk: more workgroups instead)
    items = max_rounds / per_round;
    wgx = (sets + items - 1) / items;
  }
  wgx = (sets + items - 1) / items;
  int rounds = (items * per_round + unit - 1) / unit * unit;
  p.chunks = (rounds + max_rounds - 1) / max_rounds;
  p.rounds = ((rounds + p.chunks - 1) / p.chunks + unit - 1) / unit * unit;
  auto run = [&]() -> hipError_t {
    if (a.bf16) {  // (the bfloat16 instances: q4bf16_*)
      if (p.phases > 1)
        return nbt == 2 ? launch_mid<2, 8, 2, false, true, true>(p, wgx, experts, s)
                        : launch_mid<1, 8, 2, true, true, true>(p, wgx, experts, s);
      return nbt == 2 ? launch_mid<2, 8, 2, false, false, true>(p, wgx, experts, s)
                      : launch_mid<1, 8, 2, true, false, true>(p, wgx, experts, s);
    }
    if (p.phases > 1) {
      if (form == 2) return hipErrorNotSupported;
      if (nbt == 2) return launch_mid<2, 8, 2, false, true>(p, wgx, experts, s);
      return launch_mid<1, 8, 2, true, true>(p, wgx, experts, s);
    }
    if (nbt == 2) return launch_mid<2, 8, 2, false, false>(p, wgx, experts, s);
    if (form == 2) return launch_mid<1, 8, 4, false, false>(p, wgx, experts, s);
    if (form == 4) return launch_mid<1, 8, 3, true, false>(p, wgx, experts, s);
    return launch_mid<1, 8, 2, true, false>(p, wgx, experts, s);
  };
  const hipError_t e = run();
  if (e != hipSuccess || p.slices == 1) return e;
  const int64_t count = static_cast<int64_t>(p.rows) * p.N;
  if (fold_silu) {
    const int64_t outs = count / 2;
    hipLaunchKernelGGL(mid_reduce_silu_kernel, dim3(static_cast<unsigned>((outs + 255) / 256 > 4096 ? 4096 : (outs + 255) / 256)),
                       dim3(256), 0, s, static_cast<const float*>(a.workspace), p.slices, static_cast<int64_t>(p.rows), p.N,
                       static_cast<uint16_t*>(a.y), a.bf16);
  } else {
    const int64_t blocks = ((p.N & 3) == 0 ? (count / 4 + 255) / 256 : (count + 255) / 256);
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3(static_cast<unsigned>(blocks > 4096 ? 4096 : blocks)), dim3(256), 0, s,
                       static_cast<const float*>(a.workspace), p.slices, count, p.N, a.bias, a.residual, a.y, a.out_f32, a.bf16);
  }
  return hipGetLastError();
}

// scratch for the K slices of a plain linear (0: K is one phase)
int64_t midrow_workspace_bytes(int64_t rows, int64_t N, int64_t K) {
  if (rows < 1 || N < 16 || K <= 0 || (K & 255) != 0) return 0;
  const int64_t phases = (K / 32 + 127) / 128;
  return phases > 1 ? phases * rows * N * 4 : 0;
}

}  // namespace gq
