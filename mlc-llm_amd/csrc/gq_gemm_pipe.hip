// Prefill GEMM / MoE grouped GEMM, software-pipelined form (the one that normally runs).
//
// Same tiling and LDS layout as gq_gemm.hip; what differs is how latency is hidden:
//  * global loads run TWO K tiles ahead of the MFMAs (register ping-pong), because one tile of
//    MFMA work (~0.4 us) is shorter than a trip to L2 / HBM;
//  * every load is branch-free (addresses are clamped, out-of-range data is zeroed when it is
//    written to LDS) so that the compiler's wait-count insertion can leave the newest loads in
//    flight instead of draining the queue at every join;
//  * the MFMA fragments of k-step s+1 are read from LDS before the MFMAs of step s are issued.
// Requires K % 8 == 0 (16-byte aligned activation rows); other K take the kernel in gq_gemm.hip.
#include <type_traits>

#include "gq_gemm_common.hpp"

namespace gq {

// DEPTH: K tiles of global loads in flight (register stages); even, 2 for the large tiles, more
// for few-row tiles whose MFMA work per tile is far shorter than a trip to memory
// BF: bfloat16 model (operands and 16-bit outputs are bf16; see dequant_word4_bf16)
// SKIP: waves leave out the 32-row blocks of their sub-tile that lie past the segment's last row
// WX: extra register stages for the weights alone.  Loads return in issue order, so each iteration issues its
// activation loads first and the weight loads (WX tiles further ahead) after them: waiting for the activations of
// the next tile then leaves the newer weight loads in flight.  For matmuls whose weights are read once and come
// straight from HBM (grouped, one row tile per expert) while the activations come from L2.
// FAST: K is whole K tiles and whole rounds of the register rings, and every byte offset is below 4 GiB (checked by the
// launcher).  The K loop then has no zero-selects and no clamps, and loads through buffer descriptors (tensor in scalar
// registers, K tile as the scalar offset, one 32-bit lane offset): 122 -> 62 VALU instructions per wave and K tile.  Rows
// past the segment and columns past N need no zeros: their loads are clamped to valid rows when the offsets are set up, a
// row of x or of W only ever reaches its own row or column of the result, and the epilogue drops those; only k past K
// would reach live results: q4 runs this form only when there is none; q3f16_1, whose 80-wide K tiles divide no power of two
// (K = 4096 is 51.2 tiles), masks the activation chunks at k >= K and gives a group past the last one scale 0 (one AND per
// chunk word, one select per group), and its descriptors carry the tensors' sizes, so that the last row's overrun reads
// zeros instead of the bytes behind the tensor.  A separate instantiation rather than a branch: the general
// form's addresses and flags would otherwise stay in registers next to this one's, and the large tile has none to spare
// (a spill reload inside the loop waits for every global load in flight).
// q4 in that form also reads its scales in bulk: the two lanes of a weight row load the row's 16 bytes of scales for FOUR
// K tiles at once (one request: both lanes name the same address) instead of 2 bytes per lane and K tile.  A 2-byte load
// costs the memory pipeline what a 16-byte one does (a wave's instruction touches 32 rows = 32 cache lines either way),
// and those loads alone were 9 % of the plain 256 x 256 GEMM, 18 % of down_proj's and a third of a grouped GEMM with few
// rows per expert (timing-only builds without them).  Needs K in whole blocks of four K tiles and 16-byte aligned scale
// rows (checked by the launcher).
template <int BITS, int BM, int BN, int WM, int WN, int DEPTH = 2, bool BF = false, bool SKIP = false, int WX = 0,
          bool FAST = false>
__global__ __launch_bounds__(64 * (BM / WM) * (BN / WN)) void gemm_pipe_kernel(const GemmParams p) {
  using T = GemmTraits<BITS>;
  constexpr int G = T::G;
  constexpr int BK = 2 * G;        // 64 | 80
  constexpr int KSTEPS = BK / 16;  // MFMA k = 16
  constexpr int CPR = BK / 8;      // 16-byte chunks per tile row
  constexpr int LDA = BK + 8;      // padded row, in halves
  constexpr int WAVES_N = BN / WN;
  constexpr int NT = 64 * (BM / WM) * (BN / WN);
  static_assert(NT == 256 || NT == 512, "4 or 8 waves per workgroup");
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int A_CHUNKS = (BM * CPR + NT - 1) / NT;  // the last round may cover part of the threads only
  constexpr bool A_EXACT = BM * CPR % NT == 0;
  // groups of W per thread and K tile; a tile with fewer groups than threads (256 x 128) leaves the upper waves
  // without any (W_ALL false: a wave-uniform test, every SIMD still hosts one wave that dequantises)
  constexpr int W_GROUPS = BN * 2 >= NT ? BN * 2 / NT : 1;
  constexpr bool W_ALL = BN * 2 >= NT;
  static_assert(BN * 2 % NT == 0 || BN * 2 * 2 == NT, "tile / thread mismatch");
  constexpr bool SCV = FAST && BITS == 4;  // scales of four K tiles per load

  extern __shared__ uint4 smem[];
  uint16_t* lds = reinterpret_cast<uint16_t*>(smem);
  // [A stage 0][A stage 1][W stage 0][W stage 1]: the two stages of an operand lie less than 64 KiB apart, so a
  // stage is an immediate offset of the LDS instruction and both share one address register
  auto a_tile = [&](int s) { return lds + s * BM * LDA; };
  auto w_tile = [&](int s) { return lds + 2 * BM * LDA + s * BN * LDA; };

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
  const bool w_active = W_ALL || tid < BN * 2;  // (wave-uniform)

  int seg_lo, seg_hi, mt, expert;
  if (!locate_tile<BM>(p, blockIdx.y, seg_lo, seg_hi, mt, expert)) return;  // uniform
  const int m0 = seg_lo + mt * BM;
  // 32-row blocks of this wave that hold rows of the segment: the others are skipped by the matrix core
  // (SKIP; a ragged expert segment or a last row tile leaves most of a tall tile empty)
  const int live = SKIP ? min(TM, max(0, (seg_hi - (m0 + wm0) + 31) / 32)) : TM;
  const int n0 = p.n_begin + blockIdx.x * BN;
  const uint32_t* qw = p.qw + expert * p.expert_w_stride;
  const uint16_t* qs = p.qs + expert * p.expert_s_stride;

  // ---- per-thread load slots: where each 16-byte chunk of x / each group of W comes from
  const uint16_t* a_src[A_CHUNKS];  // chunk address at K tile 0 (row clamped into the segment)
  bool a_row_ok[A_CHUNKS];
  bool a_in_tile[A_CHUNKS];         // false: this thread has no chunk in round i (loads a valid address, stores nothing)
  int a_k[A_CHUNKS];                // k offset of the chunk inside a tile
  int a_dst[A_CHUNKS];              // offset (halves) inside the LDS tile
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) {
    const int idx_raw = tid + NT * i;
    a_in_tile[i] = A_EXACT || idx_raw < BM * CPR;
    const int idx = a_in_tile[i] ? idx_raw : 0;
    // (q4: a thread's chunks sit NT / CPR rows apart in the same column, written out so that their LDS addresses
    //  become one register plus constants instead of a register each)
    constexpr bool AFFINE = A_EXACT && NT % CPR == 0;
    const int r = AFFINE ? tid / CPR + i * (NT / CPR) : idx / CPR;
    const int c = AFFINE ? tid % CPR : idx - r * CPR;
    a_row_ok[i] = m0 + r < seg_hi;
    a_k[i] = 8 * c;
    a_src[i] = p.x + x_row(p.x_rows, p.x_src_rows, a_row_ok[i] ? m0 + r : m0) * p.K + 8 * c;
    a_dst[i] = r * LDA + 8 * c;
  }
  const uint32_t* w_src[W_GROUPS];
  const uint16_t* s_src[W_GROUPS];
  int w_g[W_GROUPS];  // group index at K tile 0
  int w_dst[W_GROUPS];
#pragma unroll
  for (int i = 0; i < W_GROUPS; ++i) {
    const int idx = w_active ? tid + NT * i : 0;
    const int r = idx >> 1, gsel = idx & 1;
    int row = min(n0 + r, p.N - 1);  // rows past N are computed and dropped
    if (p.paired) row = gate_up_row_blk<(TN % 2 == 0) ? 32 : 16>(n0 + r, p.N);
    w_src[i] = qw + static_cast<int64_t>(row) * p.nw;
    s_src[i] = qs + static_cast<int64_t>(row) * p.ng;
    w_g[i] = gsel;
    // (offset from the start of LDS, made opaque: left to itself the compiler folds the W region's 72 KiB into the
    //  constants, finds them past the 64 KiB an LDS instruction's immediate holds, and keeps a register per store)
    w_dst[i] = 2 * BM * LDA + r * LDA + gsel * G;
    asm volatile("" : "+v"(w_dst[i]));
  }

  uint32_t a_off[A_CHUNKS], w_off[W_GROUPS], s_off[W_GROUPS];
  uint32_t sc_shift[W_GROUPS];  // (SCV) bit position of this lane's group inside a K tile's word of two scales
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i)
    a_off[i] = static_cast<uint32_t>(reinterpret_cast<const char*>(a_src[i]) - reinterpret_cast<const char*>(p.x));
#pragma unroll
  for (int i = 0; i < W_GROUPS; ++i) {
    w_off[i] = static_cast<uint32_t>(reinterpret_cast<const char*>(w_src[i] + 4 * w_g[i]) - reinterpret_cast<const char*>(qw));
    s_off[i] = static_cast<uint32_t>(reinterpret_cast<const char*>(s_src[i] + (SCV ? 0 : w_g[i])) - reinterpret_cast<const char*>(qs));
    sc_shift[i] = 16u * static_cast<uint32_t>(w_g[i]);
  }

  // this workgroup's share of K (all of it unless the launch splits K)
  const int nk = (p.ng + 1) / 2;
  const int kt0 = blockIdx.z * p.kt_per_split;
  const int kt1 = min(nk, kt0 + p.kt_per_split);
  const int k_lim = min(p.K, kt1 * BK);  // k and groups from here on contribute nothing
  const int g_lim = min(p.ng, 2 * kt1);

  struct StageA {
    uint4 a[A_CHUNKS];
  };
  struct StageW {
    uint4 w[W_GROUPS];
    uint32_t s[W_GROUPS];  // fp16 scale bits (32 bits wide on purpose: in flight, never re-packed)
  };
  static_assert(DEPTH >= 2 && DEPTH % 2 == 0, "register stages pair up with the two LDS stages");
  constexpr int WD = DEPTH + WX;
  static_assert(WD % DEPTH == 0, "the unrolled loop walks whole rounds of both register rings");
  StageA ra[DEPTH];
  StageW rw[WD];

  // K tile kt into registers.  Always valid addresses; validity is re-derived at store time.
  // (buffer loads: the descriptor of each tensor sits in scalar registers, the K tile is the scalar offset and the lane
  //  offset one 32-bit register, so no 64-bit address is formed or kept per load)
  constexpr bool KTAIL = FAST && BITS == 3;  // the last K tile may reach past K
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(p.x), short(0), KTAIL ? static_cast<int>(p.x_bytes) : -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint32_t*>(qw), short(0), KTAIL ? static_cast<int>(static_cast<uint32_t>(p.N) * static_cast<uint32_t>(p.nw) * 4u) : -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(qs), short(0), KTAIL ? static_cast<int>(static_cast<uint32_t>(p.N) * static_cast<uint32_t>(p.ng) * 2u) : -1, 0x00020000);
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  auto load_a_fast = [&](int kt, StageA& st) {  // (tiles past the end re-read the last one: never multiplied)
    const int soff = min(kt, kt1 - 1) * (BK * 2);
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, static_cast<int>(a_off[i]), soff, 0);
      st.a[i] = make_uint4(v.x, v.y, v.z, v.w);
    }
  };
  auto load_w_fast = [&](int kt, StageW& st) {
    if (w_active) {
      const int ktc = min(kt, kt1 - 1);
#pragma unroll
      for (int i = 0; i < W_GROUPS; ++i) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, static_cast<int>(w_off[i]), ktc * 32, 0);
        st.w[i] = make_uint4(v.x, v.y, v.z, v.w);
        if constexpr (!SCV) st.s[i] = __builtin_amdgcn_raw_buffer_load_b16(s_rsrc, static_cast<int>(s_off[i]), ktc * 4, 0);
      }
    }
  };
  // (SCV) the scales of K tiles kt0 + 4 blk .. + 3 of this lane's weight row: word c = the two groups of tile c
  struct ScaleBlock {
    uint4 v[W_GROUPS];
  };
  auto load_scales = [&](int blk, ScaleBlock& sb) {
    if (w_active) {
      const int t = min(kt0 + 4 * blk, kt1 - 4);
#pragma unroll
      for (int i = 0; i < W_GROUPS; ++i) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(s_rsrc, static_cast<int>(s_off[i]), t * 4, 0);
        sb.v[i] = make_uint4(v.x, v.y, v.z, v.w);
      }
    }
  };
  auto scale_of = [&](const ScaleBlock& sb, int i, int c) -> uint32_t {  // c: K tile inside the block (compile-time)
    const uint32_t word = c == 0 ? sb.v[i].x : (c == 1 ? sb.v[i].y : (c == 2 ? sb.v[i].z : sb.v[i].w));
    return (word >> sc_shift[i]) & 0xffffu;
  };
  auto load_a = [&](int kt, StageA& st) {
    if constexpr (FAST) {
      load_a_fast(kt, st);
      return;
    }
    const int k_base = kt * BK;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const bool ok = k_base + a_k[i] < k_lim;  // K % 8 == 0: a chunk is entirely inside or outside
      st.a[i] = *reinterpret_cast<const uint4*>(ok ? a_src[i] + k_base : a_src[i]);
    }
  };
  auto load_w = [&](int kt, StageW& st) {
    if constexpr (FAST) {
      load_w_fast(kt, st);
      return;
    }
    if (w_active) {
#pragma unroll
      for (int i = 0; i < W_GROUPS; ++i) {
        const int g = 2 * kt + w_g[i];
        const int gc = g < p.ng ? g : 0;
        st.w[i] = *reinterpret_cast<const uint4*>(w_src[i] + 4 * gc);
        st.s[i] = s_src[i][gc];
      }
    }
  };
  // One of KSTEPS slices of "tile kt: registers -> LDS stage s".  The slices are issued between the
  // MFMA k-steps of the tile being multiplied, so that dequantisation (VALU) and the LDS stores
  // run in the shadow of the matrix pipe instead of after it.
  auto store_part = [&](int kt, const StageA& sa, const StageW& st, int s, int part, const ScaleBlock& scb, int sc_c) {
    uint16_t* at = a_tile(s);
    uint16_t* wt = lds + s * BN * LDA;  // (w_dst holds the offset of the W region)
    const int k_base = kt * BK;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      if (i % KSTEPS != part) continue;
      // (the zero for rows past the segment and k past K as an AND with a lane mask: written as a select of the four
      //  words it becomes a branch around four moves, and control flow inside the loop makes the wait-count insertion
      //  drain every load in flight at the loop header)
      const bool kept = KTAIL ? k_base + a_k[i] < p.K : (FAST || (a_row_ok[i] && (k_base + a_k[i] < k_lim)));
      const uint32_t keep = kept ? 0xffffffffu : 0u;
      if (A_EXACT || a_in_tile[i])
        *reinterpret_cast<uint4*>(at + a_dst[i]) =
            (FAST && !KTAIL) ? sa.a[i] : make_uint4(sa.a[i].x & keep, sa.a[i].y & keep, sa.a[i].z & keep, sa.a[i].w & keep);
    }
    if (!w_active) return;
#pragma unroll
    for (int i = 0; i < W_GROUPS; ++i) {
      const bool ok = KTAIL ? 2 * kt + w_g[i] < p.ng : (FAST || 2 * kt + w_g[i] < g_lim);
      // a group past the end gets scale +0.0: every value becomes (q - m) * 0 = +-0
      const uint16_t sb = SCV ? static_cast<uint16_t>(scale_of(scb, i, sc_c)) : (ok ? static_cast<uint16_t>(st.s[i]) : uint16_t(0));
      uint4* dst = reinterpret_cast<uint4*>(wt + w_dst[i]);
      if (BITS == 4) {
        // word `part` of the group -> 8 halves = one 16-byte chunk
        const uint32_t w4[4] = {st.w[i].x, st.w[i].y, st.w[i].z, st.w[i].w};
        uint32_t d[4];
        if constexpr (BF) dequant_word4_bf16(w4[part], sb, d);
        else dequant_word4(w4[part], sb, d);
        dst[part] = make_uint4(d[0], d[1], d[2], d[3]);
      } else if constexpr (!BF) {
        // q3: 16-byte chunk `part` of the group (5 chunks, 5 k-steps)
        uint32_t d[4];
        dequant_chunk3(st.w[i], sb, part, d);
        dst[part] = make_uint4(d[0], d[1], d[2], d[3]);
      } else if (part == 0) {
        uint32_t d[G / 2];
        dequant_group_bf16<BITS>(st.w[i], sb, d);
#pragma unroll
        for (int c = 0; c < G / 8; ++c) dst[c] = make_uint4(d[4 * c], d[4 * c + 1], d[4 * c + 2], d[4 * c + 3]);
      }
    }
  };
  auto store_tile = [&](int kt, const StageA& sa, const StageW& st, int s, const ScaleBlock& scb, int sc_c) {
#pragma unroll
    for (int part = 0; part < KSTEPS; ++part) store_part(kt, sa, st, s, part, scb, sc_c);
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int frag_row = lane & 31, frag_k = 8 * (lane >> 5);
  // MFMAs of the tile in stage s; slice ks of the next tile's store is issued after k-step ks
  // full: every 32-row block of the wave is live (the straight-line form); otherwise blocks >= live are skipped by
  // wave-uniform branches, fragments and all
  auto mfma_tile = [&](auto full, int s, int kt_store, const StageA& sa_store, const StageW& st_store,
                       const ScaleBlock& scb, int sc_c) {
    constexpr bool FULL = decltype(full)::value;
    const uint16_t* at = a_tile(s) + (wm0 + frag_row) * LDA + frag_k;
    const uint16_t* wt = w_tile(s) + (wn0 + frag_row) * LDA + frag_k;
    auto mma = [&](const half8_t& av, const half8_t& bv, float16_t& c) {
      if constexpr (BF)
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av), __builtin_bit_cast(bf16x8_t, bv), c,
                                                    0, 0, 0);
      else
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, c, 0, 0, 0);
    };
    if constexpr (TM == 4) {
      // Four row blocks per wave: the kernel runs close to the 256-register limit, and a spill reload inside this loop
      // would wait for every global load in flight.  The activation fragments therefore live in ONE set of registers:
      // block i of the next k-step is read right after the MFMAs that used block i of this one (six MFMAs ahead of its
      // own use); only the weight fragments are double-buffered (same speed as two sets, 16 registers fewer).
      half8_t af[TM], bf[2][TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        if (FULL || i < live) af[i] = *reinterpret_cast<const half8_t*>(at + i * 32 * LDA);
      if (FULL || live > 0) {
#pragma unroll
        for (int j = 0; j < TN; ++j) bf[0][j] = *reinterpret_cast<const half8_t*>(wt + j * 32 * LDA);
      }
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        const int cur = ks & 1, nxt = cur ^ 1;
        if (ks + 1 < KSTEPS && (FULL || live > 0)) {
#pragma unroll
          for (int j = 0; j < TN; ++j)
            bf[nxt][j] = *reinterpret_cast<const half8_t*>(wt + j * 32 * LDA + (ks + 1) * 16);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          if (FULL || i < live) {
#pragma unroll
            for (int j = 0; j < TN; ++j) mma(af[i], bf[cur][j], acc[i][j]);
            if (ks + 1 < KSTEPS) af[i] = *reinterpret_cast<const half8_t*>(at + i * 32 * LDA + (ks + 1) * 16);
          }
        }
        store_part(kt_store, sa_store, st_store, s ^ 1, ks, scb, sc_c);
        __builtin_amdgcn_sched_barrier(0);  // keep the slices where they were written
      }
    } else {  // fragments of k-step s+1 are read while the MFMAs of step s run
      half8_t af[2][TM], bf[2][TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        if (FULL || i < live) af[0][i] = *reinterpret_cast<const half8_t*>(at + i * 32 * LDA);
      if (FULL || live > 0) {
#pragma unroll
        for (int j = 0; j < TN; ++j) bf[0][j] = *reinterpret_cast<const half8_t*>(wt + j * 32 * LDA);
      }
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        const int cur = ks & 1, nxt = cur ^ 1;
        if (ks + 1 < KSTEPS) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
            if (FULL || i < live) af[nxt][i] = *reinterpret_cast<const half8_t*>(at + i * 32 * LDA + (ks + 1) * 16);
          if (FULL || live > 0) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
              bf[nxt][j] = *reinterpret_cast<const half8_t*>(wt + j * 32 * LDA + (ks + 1) * 16);
          }
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          if (FULL || i < live) {
#pragma unroll
            for (int j = 0; j < TN; ++j) mma(af[cur][i], bf[cur][j], acc[i][j]);
          }
        }
        store_part(kt_store, sa_store, st_store, s ^ 1, ks, scb, sc_c);
        __builtin_amdgcn_sched_barrier(0);  // keep the slices where they were written
      }
    }
  };

  // ---- pipeline: tile t in LDS stage t&1, tiles t+1 .. t+DEPTH-1 in registers, tile t+DEPTH in flight
  ScaleBlock sc_cur{}, sc_nxt{};  // (SCV) scales of the block of four K tiles being stored, and of the block after it
  if constexpr (SCV) {
    load_scales(0, sc_cur);
    load_scales(1, sc_nxt);
  }
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) load_a(kt0 + d, ra[d]);
#pragma unroll
  for (int d = 0; d < WD; ++d) load_w(kt0 + d, rw[d]);
  store_tile(kt0, ra[0], rw[0], 0, sc_cur, 0);
  load_a(kt0 + DEPTH, ra[0]);
  load_w(kt0 + WD, rw[0]);
  __syncthreads();
  // (a register stage is refilled right after the MFMA/store block that drains it; a tile past
  //  the end is stored as zeros and adds nothing)
  constexpr int TRIP = SCV ? 4 : WD;  // K tiles per trip: whole rounds of the register rings, and of a scale block
  static_assert(TRIP % WD == 0, "a trip walks whole rounds of the register rings");
  // one trip; SCV: the four tiles stored are 1..3 of block `cur` and the first of block `nxt`, after which `cur` is free
  // and takes the block after `nxt` (consumed four K tiles from there)
  auto trip = [&](auto full, int kt, ScaleBlock& cur, ScaleBlock& nxt) __attribute__((always_inline)) {
#pragma unroll
    for (int d = 0; d < TRIP; ++d) {
      // the tile stored during this step is kt + d + 1
      mfma_tile(full, d & 1, kt + d + 1, ra[(d + 1) % DEPTH], rw[(d + 1) % WD], (SCV && d == 3) ? nxt : cur, (d + 1) & 3);
      load_a(kt + d + 1 + DEPTH, ra[(d + 1) % DEPTH]);
      load_w(kt + d + 1 + WD, rw[(d + 1) % WD]);
      if constexpr (SCV) {
        if (d == 3) load_scales((kt - kt0) / 4 + 2, cur);
      }
      __syncthreads();
    }
  };
  auto k_loop = [&](auto full) {
    if constexpr (SCV) {
      // the two scale blocks swap roles from trip to trip: written out as two trips per round (no register copies, which
      // the compiler would place right behind the load they wait for); an odd last trip follows the loop (an exit in
      // the middle of the round would make the loop a join of two paths, where the wait-count insertion drains the queue)
      int kt = kt0;
      for (; kt + 2 * TRIP <= kt1; kt += 2 * TRIP) {
        trip(full, kt, sc_cur, sc_nxt);
        trip(full, kt + TRIP, sc_nxt, sc_cur);
      }
      if (kt < kt1) trip(full, kt, sc_cur, sc_nxt);
    } else {
      for (int kt = kt0; kt < kt1; kt += TRIP) trip(full, kt, sc_cur, sc_nxt);
    }
  };
  if (!SKIP || live == TM) k_loop(std::true_type{});
  else k_loop(std::false_type{});

  // ---- epilogue: D[i][j] of a 32x32 tile sits in lane (j + 32*((i/4)%2)), register 4*(i/8) + i%4
  if (p.paired && p.partial == nullptr) {
    const int half = p.N >> 1;
    if constexpr (TN % 2 == 0) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int jj = 0; jj < TN / 2; ++jj) {
          const int col = ((n0 + wn0) >> 1) + jj * 32 + (lane & 31);
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int row = m0 + wm0 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (row < seg_hi && col < half)
              static_cast<uint16_t*>(p.y)[static_cast<int64_t>(row) * half + col] =
                  silu_mul_t<BF>(acc[i][2 * jj][r], acc[i][2 * jj + 1][r]);
          }
        }
      }
    } else {
      static_assert(TN % 2 == 0 || TN == 1, "one accumulator per wave, or pairs of them");
      // columns 0..15 of the accumulator are gate rows, 16..31 the matching up rows
      const int col = ((n0 + wn0) >> 1) + (lane & 15);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float up = __shfl_xor(acc[i][0][r], 16, 64);  // every lane takes part
          const int row = m0 + wm0 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          if ((lane & 16) == 0 && row < seg_hi && col < half)
            static_cast<uint16_t*>(p.y)[static_cast<int64_t>(row) * half + col] = silu_mul_t<BF>(acc[i][0][r], up);
        }
      }
    }
    return;
  }
  // (one loop nest per output form keeps each fully unrolled nest small)
  auto for_each = [&](auto&& body) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = n0 + wn0 + j * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = m0 + wm0 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          if (row < seg_hi && col < p.N) body(row, col, acc[i][j][r]);
        }
      }
    }
  };
  if (p.partial != nullptr) {
    float* part = p.partial + static_cast<int64_t>(blockIdx.z) * p.rows * p.N;
    for_each([&](int row, int col, float v) { part[static_cast<int64_t>(row) * p.N + col] = v; });
  } else if (p.bias == nullptr && p.residual == nullptr) {
    if (p.out_f32)
      for_each([&](int row, int col, float v) { static_cast<float*>(p.y)[static_cast<int64_t>(row) * p.N + col] = v; });
    else
      for_each([&](int row, int col, float v) {
        static_cast<uint16_t*>(p.y)[static_cast<int64_t>(row) * p.N + col] = BF ? bf16_bits_of(v) : f2h(v);
      });
  } else {
    for_each([&](int row, int col, float v) {
      const int64_t o = static_cast<int64_t>(row) * p.N + col;
      const float t = v + (p.bias != nullptr ? (BF ? bf16_to_f32(p.bias[col]) : h2f(p.bias[col])) : 0.f) +
                      (p.residual != nullptr ? (BF ? bf16_to_f32(p.residual[o]) : h2f(p.residual[o])) : 0.f);
      if (p.out_f32) static_cast<float*>(p.y)[o] = t;
      else static_cast<uint16_t*>(p.y)[o] = BF ? bf16_bits_of(t) : f2h(t);
    });
  }
}

template <int BITS, int BM, int BN, int WM, int WN, int DEPTH, bool BF, bool SKIP, int WX, bool FAST>
static hipError_t launch_pipe_form(const GemmParams& p, hipStream_t s) {
  constexpr int BK = 2 * GemmTraits<BITS>::G;
  constexpr int LDA = BK + 8;
  constexpr size_t lds = size_t(2) * (BM + BN) * LDA * 2;
  auto kern = gemm_pipe_kernel<BITS, BM, BN, WM, WN, DEPTH, BF, SKIP, WX, FAST>;
  if (lds > 65536) {
    const hipError_t e = allow_large_lds(reinterpret_cast<const void*>(kern));
    if (e != hipSuccess) return e;
  }
  const int m_tiles = p.indptr ? (p.rows + BM - 1) / BM + p.num_experts : (p.rows + BM - 1) / BM;
  const int nk = (p.ng + 1) / 2;
  const int split = p.partial ? (nk + p.kt_per_split - 1) / p.kt_per_split : 1;
  // the fused gate/up form walks whole 64-column blocks (32 gate + 32 up rows)
  constexpr int PB = ((WN / 32) % 2 == 0) ? 32 : 16;
  const int n_cols = p.paired ? ((p.N / 2 + PB - 1) / PB) * 2 * PB : p.N;
  const int n_last = p.n_end > 0 ? p.n_end : n_cols;
  if (n_last <= p.n_begin) return hipSuccess;
  const dim3 grid((n_last - p.n_begin + BN - 1) / BN, m_tiles, split);
  note_kernel("gq::gemm_pipe_kernel<%d,%d,%d,%d,%d,%d,%s,%s,%d,%s>", BITS, BM, BN, WM, WN, DEPTH, BF ? "true" : "false",
              SKIP ? "true" : "false", WX, FAST ? "true" : "false");
  hipLaunchKernelGGL(kern, grid, dim3(64 * (BM / WM) * (BN / WN)), lds, s, p);
  return hipGetLastError();
}

template <int BITS, int BM, int BN, int WM, int WN, int DEPTH = 2, bool BF = false, bool SKIP = false, int WX = 0>
static hipError_t launch_pipe_cfg(const GemmParams& p, hipStream_t s) {
  // the form without zero-selects: K in whole K tiles (fast_ok), and every workgroup's share of them in whole rounds of
  // the register rings (all of K, or the split's share; the last split gets what is left)
  constexpr int WD = DEPTH + WX;
  const int nk = (p.ng + 1) / 2;
  const bool whole_rounds = nk % WD == 0 && (p.partial == nullptr || p.kt_per_split % WD == 0);
  // q4 reads its scales 16 bytes (four K tiles) at a time there: whole blocks of four K tiles, 16-byte aligned scale rows
  const bool scale_blocks = BITS != 4 || (nk % 4 == 0 && (p.partial == nullptr || p.kt_per_split % 4 == 0) &&
                                          (reinterpret_cast<uintptr_t>(p.qs) & 15) == 0 && p.ng % 8 == 0);
  if (p.fast_ok && whole_rounds && scale_blocks)
    return launch_pipe_form<BITS, BM, BN, WM, WN, DEPTH, BF, SKIP, WX, true>(p, s);
  return launch_pipe_form<BITS, BM, BN, WM, WN, DEPTH, BF, SKIP, WX, false>(p, s);
}

// y = sum over splits of partial[s] + bias + residual, in the output type (y may be the residual
// buffer itself: every element is read before the same thread writes it)
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, int split,
                                                            int64_t count /* rows * N */, int N,
                                                            const uint16_t* __restrict__ bias,
                                                            const uint16_t* residual, void* y, int out_f32, int bf16) {
  // bias, residual and a 16-bit y carry the model dtype: float16, or bfloat16 when bf16 is set
  auto in = [bf16](uint16_t bits) { return bf16 ? bf2f(bits) : h2f(bits); };
  auto out = [bf16](float v) { return bf16 ? f2bf(v) : f2h(v); };
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  if ((N & 3) == 0) {  // rows are 16-byte aligned: four columns per thread
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; 4 * i < count; i += stride) {
      float4 a = *reinterpret_cast<const float4*>(partial + 4 * i);
      for (int sidx = 1; sidx < split; ++sidx) {
        const float4 b = *reinterpret_cast<const float4*>(partial + sidx * count + 4 * i);
        a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
      }
      if (bias != nullptr) {
        const int col = static_cast<int>((4 * i) % N);
        const uint2 bb = *reinterpret_cast<const uint2*>(bias + col);
        a.x += in(static_cast<uint16_t>(bb.x & 0xffffu)); a.y += in(static_cast<uint16_t>(bb.x >> 16));
        a.z += in(static_cast<uint16_t>(bb.y & 0xffffu)); a.w += in(static_cast<uint16_t>(bb.y >> 16));
      }
      if (residual != nullptr) {
        const uint2 rr = *reinterpret_cast<const uint2*>(residual + 4 * i);
        a.x += in(static_cast<uint16_t>(rr.x & 0xffffu)); a.y += in(static_cast<uint16_t>(rr.x >> 16));
        a.z += in(static_cast<uint16_t>(rr.y & 0xffffu)); a.w += in(static_cast<uint16_t>(rr.y >> 16));
      }
      if (out_f32) {
        *reinterpret_cast<float4*>(static_cast<float*>(y) + 4 * i) = a;
      } else {
        uint2 o;
        o.x = static_cast<uint32_t>(out(a.x)) | (static_cast<uint32_t>(out(a.y)) << 16);
        o.y = static_cast<uint32_t>(out(a.z)) | (static_cast<uint32_t>(out(a.w)) << 16);
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(y) + 4 * i) = o;
      }
    }
  } else {
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < count; i += stride) {
      float a = partial[i];
      for (int sidx = 1; sidx < split; ++sidx) a += partial[sidx * count + i];
      if (bias != nullptr) a += in(bias[i % N]);
      if (residual != nullptr) a += in(residual[i]);
      if (out_f32) static_cast<float*>(y)[i] = a;
      else static_cast<uint16_t*>(y)[i] = out(a);
    }
  }
}

__global__ __launch_bounds__(256) void splitk_reduce_silu_kernel(const float* __restrict__ partial, int split,
                                                                 int64_t rows, int N, int pb,
                                                                 uint16_t* __restrict__ y, int bf16) {
  const int half = N >> 1;
  const int64_t count = rows * N, outs = rows * half;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < outs; i += stride) {
    const int64_t row = i / half;
    const int oc = static_cast<int>(i - row * half);
    const int64_t at = row * N + (oc / pb) * 2 * pb + oc % pb;  // pb gate columns, then their pb up columns
    float g = partial[at], u = partial[at + pb];
    for (int sidx = 1; sidx < split; ++sidx) {
      g += partial[sidx * count + at];
      u += partial[sidx * count + at + pb];
    }
    y[i] = bf16 ? silu_mul_bf(g, u) : silu_mul_h(g, u);
  }
}

SplitPlan plan_split_k(int64_t rows, int64_t N, int64_t K, int bits, int group_size, bool grouped) {
  SplitPlan plan{0, 1, 1 << 28};
  if (grouped || rows <= 0 || N <= 0 || K <= 0 || (K & 7) != 0) return plan;
  // few rows: the GEMM is bound by streaming the weights, and 128-wide column tiles alone leave
  // most CUs idle (o_proj / down have 32 of them).  Match the tile height to the rows and cut K
  // until about one workgroup per CU exists.
  // (up to 1024 rows: down_proj, 32 column tiles and a long K, ran 150 us flat from 257 to 512 rows unsplit)
  if (rows > 1024) return plan;
  const int bm = rows <= 32 ? 32 : (rows <= 64 ? 64 : 128);
  const int64_t tiles = ((rows + bm - 1) / bm) * ((N + 127) / 128);
  if (rows > 128 && tiles >= 200) return plan;  // the regular tiles already fill the chip
  plan.bm = bm;
  const int ng = static_cast<int>((K + group_size - 1) / group_size);
  const int nk = (ng + 1) / 2;
  // Splitting K pays with partial sums (split * rows * N * 8 bytes written and read back): only
  // when the tiles alone leave CUs idle, and never beyond about twice the weight bytes.
  int split = 1;
  if (tiles < 200 || options().gemm_split_k > 0) {
    // one workgroup per CU: measured 8-20 % faster than two (o_proj, qkv, down at 17..128 rows), whose
    // partial sums cost more than the second workgroup hides
    const int64_t want = options().gemm_split_k > 0 ? options().gemm_split_k : 256;  // (tuning override)
    split = static_cast<int>((want + tiles - 1) / tiles);
    const int64_t cap = K / (7 * rows);
    if (options().gemm_split_k <= 0 && split > cap) split = static_cast<int>(cap);
    if (split > nk / 4) split = nk / 4;  // at least four K tiles per workgroup
    if (split < 1) split = 1;
  }
  // the K loop advances four tiles at a time in the few-row kernels: whole rounds per workgroup
  plan.kt_per_split = ((nk + split - 1) / split + 3) / 4 * 4;
  plan.split = (nk + plan.kt_per_split - 1) / plan.kt_per_split;
  return plan;
}

int gemm_pipe_pair_block(const GemmParams& p, int bits) {
  return (p.bm_hint == 32 && options().gemm_variant < 0) ? 16 : 32;  // the 32 x 128 tile below
}

// Which of the three regular tiles a plain matmul of this shape should run: 2 = 256 x 256, 1 = 128 x 256,
// 0 = 128 x 128.  A launch costs rounds x (time of one tile), rounds = ceil(tiles / resident workgroups) (256 for
// the two large tiles, 512 for 128 x 128), tile times from the per-tile rates measured with balanced rounds (q4:
// 1035 / 870 / 806 TFLOP/s; q3, whose K tile does not fit the largest one: 739 / 566).  What the model is for is the
// last, partly filled round: 300 tiles of 256 x 256 take two rounds where 540 of 128 x 256 take three half-sized
// ones (13B qkv at 1025 rows: 584 -> 621 TFLOP/s; gate_up at 1025 rows: 699 -> 785; qkv 6144 x 4096 at 1536 rows, the
// other way round: 568 -> 706).
int pick_regular_tile(int64_t rows, int64_t N, int bits) {
  const int64_t ntw = (N + 255) / 256, ntn = (N + 127) / 128;
  const int64_t big = ((rows + 255) / 256) * ntw, mid = ((rows + 127) / 128) * ntw, small = ((rows + 127) / 128) * ntn;
  const double t_big = 65536.0 / (1035.0 / 256), t_mid = 32768.0 / ((bits == 4 ? 870.0 : 739.0) / 256),
               t_small = 16384.0 / ((bits == 4 ? 806.0 : 566.0) / 512);
  const double c_big = bits == 4 ? static_cast<double>((big + 255) / 256) * t_big : 1e30;
  const double c_mid = static_cast<double>((mid + 255) / 256) * t_mid;
  // 128 x 128: two workgroups share a CU; one on its own runs faster than its half of a pair (0.72 of the
  // pair's time fits 13B o_proj at 640 rows, 200 such tiles: 539 TFLOP/s against 420 on 100 tiles of 128 x 256)
  const int64_t per_cu = (small + 255) / 256;
  const double c_small = static_cast<double>(per_cu / 2) * t_small + static_cast<double>(per_cu % 2) * 0.72 * t_small;
  // a partly filled last round runs faster than a full one (the part is power-limited), which favours the larger
  // tile: a smaller tile has to win by 8 % on paper
  int pick = 2;
  double best = c_big;
  if (c_mid < 0.92 * best) { pick = 1; best = c_mid; }
  if (c_small < 0.92 * best) pick = 0;
  return pick;
}

hipError_t launch_gemm_pipe(const GemmParams& p, int bits, hipStream_t s) {
  if ((p.K & 7) != 0 || p.ng == 0) return hipErrorNotSupported;
  const int variant = options().gemm_variant;
  if (p.paired && (p.N & 1)) return hipErrorNotSupported;
  if (p.bf16) {
    // bfloat16 models: plain and grouped matmul (no folded activation)
    if (p.bm_hint > 0 && p.indptr == nullptr) {  // few rows, K possibly split (see plan_split_k)
      if (bits == 4 && p.bm_hint == 32) return launch_pipe_cfg<4, 32, 128, 32, 32, 4, true>(p, s);
      if (bits == 4 && p.bm_hint == 64) return launch_pipe_cfg<4, 64, 128, 32, 64, 4, true>(p, s);
      if (bits == 4) return launch_pipe_cfg<4, 128, 128, 64, 64, 2, true>(p, s);
      if (p.bm_hint == 32) return launch_pipe_cfg<3, 32, 128, 32, 32, 4, true>(p, s);
      if (p.bm_hint == 64) return launch_pipe_cfg<3, 64, 128, 32, 64, 4, true>(p, s);
      return launch_pipe_cfg<3, 128, 128, 64, 64, 2, true>(p, s);
    }
    if (p.partial != nullptr) return hipErrorNotSupported;
    if (p.indptr != nullptr) {
      const bool wide = p.rows >= 96 * p.num_experts &&
                        (static_cast<int64_t>(p.rows) / 128 + p.num_experts) * ((p.N + 255) / 256) >= 768;
      if (bits == 4) {
        // few rows per expert: the tile height follows them (there are no bf16 few-row kernels)
        if (p.rows <= 16 * p.num_experts) return launch_pipe_cfg<4, 32, 128, 32, 32, 4, true>(p, s);
        if (p.rows <= 48 * p.num_experts) return launch_pipe_cfg<4, 64, 128, 32, 64, 4, true>(p, s);
        return wide ? launch_pipe_cfg<4, 128, 256, 64, 64, 2, true>(p, s)
                    : launch_pipe_cfg<4, 128, 128, 64, 64, 2, true>(p, s);
      }
      return wide ? launch_pipe_cfg<3, 128, 256, 64, 64, 2, true>(p, s)
                  : launch_pipe_cfg<3, 128, 128, 64, 64, 2, true>(p, s);
    }
    if (bits == 4) {
      // few rows: tile height follows the rows (the float16 path's few-row tiles, unsplit)
      if (p.rows <= 32) return launch_pipe_cfg<4, 32, 128, 32, 32, 4, true>(p, s);
      if (p.rows <= 64) return launch_pipe_cfg<4, 64, 128, 32, 64, 4, true>(p, s);
      const int tile = pick_regular_tile(p.rows, p.N, 4);
      if (tile == 2) return launch_pipe_cfg<4, 256, 256, 128, 64, 2, true>(p, s);
      if (tile == 1) return launch_pipe_cfg<4, 128, 256, 64, 64, 2, true>(p, s);
      return launch_pipe_cfg<4, 128, 128, 64, 64, 2, true>(p, s);
    }
    if (pick_regular_tile(p.rows, p.N, 3) == 1) return launch_pipe_cfg<3, 128, 256, 64, 64, 2, true>(p, s);
    return launch_pipe_cfg<3, 128, 128, 64, 64, 2, true>(p, s);
  }
  if (p.bm_hint > 0 && variant < 0) {
    if (bits == 4 && p.bm_hint == 32) return launch_pipe_cfg<4, 32, 128, 32, 32, 4>(p, s);
    if (bits == 4 && p.bm_hint == 64) return launch_pipe_cfg<4, 64, 128, 32, 64, 4>(p, s);
    if (bits == 4) return launch_pipe_cfg<4, 128, 128, 64, 64>(p, s);
    if (p.bm_hint == 32) return launch_pipe_cfg<3, 32, 128, 32, 32, 4>(p, s);
    if (p.bm_hint == 64) return launch_pipe_cfg<3, 64, 128, 32, 64, 4>(p, s);
    return launch_pipe_cfg<3, 128, 128, 64, 64>(p, s);
  }
  // Grouped, from about 64 rows per expert on: 256-row tiles whose waves skip the 32-row blocks past the end of
  // the expert's segment.  A ragged segment then costs its rows rounded up to 32 in matrix work, and the expert's
  // weights are dequantised once per 256 rows instead of once per (often nearly empty) 128-row tile.  256 columns
  // per tile while that still makes two workgroups per CU, else 128 (e2 of a Mixtral layer: 32 column tiles).
  if (p.indptr != nullptr && ((variant < 0 && p.rows > 48 * p.num_experts) || variant == 10 || variant == 11)) {
    const int64_t mt = p.rows / 256 + p.num_experts;
    const bool wide = variant == 10 || (variant != 11 && bits == 4 && mt * ((p.N + 255) / 256) >= 512);
    if (bits == 4) {
      if (wide) {
        // A last round of workgroups that is at most about half full costs a whole round here (the kernel waits on
        // memory, not on the matrix pipe): its columns go to a second launch on the narrow tile, whose workgroups take
        // half as long.  (Mixtral's e1_e3, 112 column tiles x 8 experts = 3.5 rounds of 256.)
        const int64_t tiles_x = (p.N + 255) / 256;
        const int64_t live = p.num_experts > p.rows / 256 ? p.num_experts : p.rows / 256;  // row tiles that hold rows
        const int64_t rounds = tiles_x * live / 256, rest = tiles_x * live % 256;
        if (variant != 10 && rounds >= 1 && rest > 0 && rest <= 144 && p.n_end == 0 && p.n_begin == 0) {
          GemmParams a = p, b = p;
          a.n_end = static_cast<int>(rounds * 256 / live * 256);
          b.n_begin = a.n_end;
          if (a.n_end > 0 && a.n_end < p.N) {
            const hipError_t e = launch_pipe_cfg<4, 256, 256, 128, 64, 2, false, true, 2>(a, s);
            if (e != hipSuccess) return e;
            return launch_pipe_cfg<4, 256, 128, 64, 64, 2, false, true, 2>(b, s);
          }
        }
        return launch_pipe_cfg<4, 256, 256, 128, 64, 2, false, true, 2>(p, s);
      }
      // both tiles' weight loads run two more K tiles ahead than their activation loads (Mixtral's e2 on the narrow tile
      // at 64 / 128 / 256 rows per expert: 201 -> 177, 236 -> 213, 320 -> 305 us; e1_e3 on the wide one 1-2 %)
      return launch_pipe_cfg<4, 256, 128, 64, 64, 2, false, true, 2>(p, s);
    }
    return launch_pipe_cfg<3, 256, 128, 64, 64, 2, false, true>(p, s);
  }
  if (bits == 4) {
    // grouped, few rows per expert: the tile height follows them (Mixtral layer, 8 experts: 144-384 routed
    // rows 18-20 % faster than on 128-row tiles)
    if (p.indptr != nullptr && (variant < 0 || variant == 1)) {
      if (p.rows <= 16 * p.num_experts) return launch_pipe_cfg<4, 32, 128, 32, 32, 4>(p, s);
      if (p.rows <= 48 * p.num_experts) return launch_pipe_cfg<4, 64, 128, 32, 64, 4>(p, s);
    }
    // plain matmul: the tile whose rounds of workgroups cost least (variants 6 / 7 / 9 force one)
    const int tile = p.indptr != nullptr ? 0 : pick_regular_tile(p.rows, p.N, 4);
    const bool big = variant == 7 ? true : (variant == 6 ? false : tile == 2);
    if (variant == 9) return launch_pipe_cfg<4, 128, 256, 64, 64>(p, s);
    if (big) return launch_pipe_cfg<4, 256, 256, 128, 64>(p, s);
    if (variant != 6 && tile == 1) return launch_pipe_cfg<4, 128, 256, 64, 64>(p, s);
    // grouped: the wider tile once the experts' row tiles alone make several rounds of workgroups
    if (variant != 6 && p.indptr != nullptr && p.rows >= 96 * p.num_experts &&
        (static_cast<int64_t>(p.rows) / 128 + p.num_experts) * ((p.N + 255) / 256) >= 768)
      return launch_pipe_cfg<4, 128, 256, 64, 64>(p, s);
    return launch_pipe_cfg<4, 128, 128, 64, 64>(p, s);
  }
  if (p.indptr != nullptr && (variant < 0 || variant == 1)) {  // grouped, few rows per expert: as q4 above
    if (p.rows <= 16 * p.num_experts) return launch_pipe_cfg<3, 32, 128, 32, 32, 4>(p, s);
    if (p.rows <= 48 * p.num_experts) return launch_pipe_cfg<3, 64, 128, 32, 64, 4>(p, s);
  }
  // q3: a K tile is 80 wide, so the 256 x 256 tile does not fit LDS; 128 x 256 does
  const bool plain_wide = p.indptr == nullptr && pick_regular_tile(p.rows, p.N, 3) == 1;
  const bool grouped_wide = p.indptr != nullptr && p.rows >= 96 * p.num_experts &&
                            (static_cast<int64_t>(p.rows) / 128 + p.num_experts) * ((p.N + 255) / 256) >= 768;
  if (variant == 9 || (variant != 6 && (plain_wide || grouped_wide)))
    return launch_pipe_cfg<3, 128, 256, 64, 64>(p, s);
  return launch_pipe_cfg<3, 128, 128, 64, 64>(p, s);
}

}  // namespace gq
