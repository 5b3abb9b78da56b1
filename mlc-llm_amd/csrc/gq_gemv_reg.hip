// Decode GEMV, register-resident activations, persistent waves (the batch-1 workhorse).
//
// Same arithmetic as gq_gemv.hip (see there for the unpack trick); different data movement:
//  * a lane is pinned to the quantisation groups {lane + 64*i, i < ITERS} of every row it
//    visits, so its slice of x (ITERS * G halves, already in the pair order the masks produce)
//    and the matching correction terms stay in VGPRs for the whole kernel;
//  * x is read from global memory once per workgroup (staged through LDS with a single barrier
//    at kernel start) rather than once per wave: with thousands of waves the re-reads of x
//    through L2 would otherwise rival the weight stream itself;
//  * a wave walks the row sets {w, w + W, w + 2W, ...} (R rows per set, W waves in the grid) and
//    keeps the R * ITERS 128-bit loads of the next set in flight while it reduces the current
//    one, so each lane always has a full set of loads outstanding;
//  * the grid is sized to a few waves per SIMD (not one block per row block): fewer, longer
//    lived waves stream HBM better than thousands of short ones.
#include "gq_gemv_common.hpp"
#include "gq_topk.hpp"

namespace gq {

// MODE 1: a bias or residual operand exists (a template flag rather than a run-time test: their loads are
// two more memory instructions per set, measured at 4-6 % of the plain GEMV's time).
// MODE 2: fused gate/up form; a set holds R / 2 (gate, up) row pairs and stores R / 2 products.
// MODE 3: MODE 2 for one token that routes itself (the expert of a slot comes from the router logits, see below); its
// own instantiation so that no other form carries the selection code.
// MODE 4 (with KW = 2): one token's second expert matmul and the weighted sum over its two experts in one launch.  The
// four waves of a workgroup are (expert slot 0 | 1) x (half of K 0 | 1) and walk the same rows; each slot has its own row
// of x (both staged in LDS) and its own expert; after the walk the first wave forms
// out[n] = rnd(rnd(y0[n]) * w0) + rnd(rnd(y1[n]) * w1), rounded once more: what the matmul's store, the multiplication by the
// routing weights and the sum over the slots do in the model dtype.  `expert_ids` holds the two ids, `residual` points at
// the two routing weights.
// BF: bfloat16 model (x, scales, bias, residual and a 16-bit result are bfloat16); the same walk with
// group_dot_bf16.  Like the float16 form it multiplies x with the integer fields and applies the scale
// to the group sum in fp32, so the dequantised weight is never rounded to the model dtype on its own.
// The arguments behind the 56 bytes of leading ones, in the order of use: an expert form without sorted rows reads
// 48 bytes of them, the plain linear none.
struct GemvTail {
  const int32_t* expert_ids;
  int64_t expert_w_stride, expert_s_stride, x_slot_stride;
  const uint16_t* bias;
  const uint16_t* residual;
  int num_experts;
  int indptr_i64;
  const void* indptr;
  const int32_t* x_row_index;
  int x_src_rows;
};

// MOE: an expert form (expert ids, expert-sorted rows, one grid row per slot).  The plain linear's instantiation reads
// none of those fields.
// KW = 2 (long K, one row per set, plain epilogue): two neighbouring waves share every row, each with ITERS groups per
// lane of its half of K; the halves' sums wait in LDS and meet after the walk (one barrier in all).  A wave then holds
// half of x in registers, so two waves fit a SIMD where the whole-K form runs one.
template <int BITS, int NB, int R, int ITERS, int MODE, bool BF = false, bool MOE = true, int KW = 1>
__global__ __launch_bounds__(256) void gemv_reg_kernel(const uint16_t* x_, const uint32_t* qw_, const uint16_t* qs_,
                                                        void* y_, int N_, int K_, int ng_, int nsets, int nwaves_,
                                                        int out_f32_, const GemvTail t) {
  // The ten leading arguments (14 dwords) arrive in scalar registers with the wave (the library is compiled with
  // kernel argument preloading): the plain linear starts its x loads without a memory read for its own arguments.
  GemvParams p;
  p.x = x_; p.qw = qw_; p.qs = qs_; p.y = y_;
  p.N = N_; p.K = K_; p.ng = ng_; p.nw = 4 * ng_;
  p.nsets = nsets; p.nwaves = nwaves_; p.out_f32 = out_f32_;
  p.expert_ids = t.expert_ids; p.expert_w_stride = t.expert_w_stride; p.expert_s_stride = t.expert_s_stride;
  p.x_slot_stride = t.x_slot_stride; p.bias = t.bias; p.residual = t.residual; p.num_experts = t.num_experts;
  p.indptr_i64 = t.indptr_i64; p.indptr = t.indptr; p.x_row_index = t.x_row_index; p.x_src_rows = t.x_src_rows;
  using T = GemvTraits<BITS>;
  constexpr bool EXTRA = MODE == 1, PAIRED = MODE == 2 || MODE == 3, ROUTED = MODE == 3;
  auto to_f32 = [](uint16_t bits) { return BF ? bf2f(bits) : h2f(bits); };
  static_assert(!PAIRED || R % 2 == 0, "a set holds whole (gate, up) pairs");
  constexpr int G = T::G;
  constexpr int HP = G / 2;  // half pairs of x per group
  // 16-byte x chunks each of the 256 threads stages: NB * ITERS * 64 groups * G/8 chunks / 256
  constexpr int XS = ((MODE == 4 ? 2 : NB) * ITERS * KW * 64 * (G / 8) + 255) / 256;

  extern __shared__ uint4 smem[];  // x as [NB][ng * G] halves, zero beyond K
  const int kpad = p.ng * G;

  const int lane = threadIdx.x & 63;
  constexpr bool SUM2 = MODE == 4;
  static_assert(KW == 1 || (KW == 2 && R == 1 && NB == 1 && (MODE == 0 || SUM2)), "shared K: one row per set, plain epilogue");
  static_assert(!SUM2 || (KW == 2 && MOE), "the sum over two experts is a form of the shared-K expert GEMV");
  const int wave_all = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int ksub = KW == 2 ? (wave_all & 1) : 0;                                     // which half of K
  const int gw = SUM2 ? static_cast<int>(blockIdx.x) : (KW == 2 ? (wave_all >> 1) : wave_all);  // walker of row sets
  const int nwaves = SUM2 ? (p.nwaves >> 2) : (KW == 2 ? (p.nwaves >> 1) : p.nwaves);
  const int slot = SUM2 ? static_cast<int>((threadIdx.x >> 7) & 1) : (MOE ? static_cast<int>(blockIdx.y) : 0);
  constexpr int NBX = SUM2 ? 2 : NB;  // rows of x a workgroup stages

  const uint16_t* x = MOE ? p.x + slot * p.x_slot_stride : p.x;
  const uint32_t* qw = p.qw;
  const uint16_t* qs = p.qs;
  if constexpr (!MOE) {
    static_assert(MODE != 3, "a token that routes itself is an expert form");
  } else if (p.indptr != nullptr) {
    // expert-sorted rows: the segment ends at or before this row number its expert (each wave counts for itself)
    int e = 0;
    for (int e0 = 0; e0 < p.num_experts; e0 += 64) {
      const int i = e0 + lane;
      int64_t end = 0x7fffffffffffffffll;
      if (i < p.num_experts)
        end = p.indptr_i64 ? static_cast<const int64_t*>(p.indptr)[i + 1] : static_cast<const int32_t*>(p.indptr)[i + 1];
      e += __popcll(__ballot(end <= slot));
    }
    if (e >= p.num_experts) return;  // past the last segment (uniform over the workgroup)
    const int64_t begin = p.indptr_i64 ? static_cast<const int64_t*>(p.indptr)[e] : static_cast<const int32_t*>(p.indptr)[e];
    if (begin > slot) return;  // before the first segment
    qw += e * p.expert_w_stride;
    qs += e * p.expert_s_stride;
    int row = slot;
    if (p.x_row_index != nullptr) {
      row = p.x_row_index[slot];
      row = row < 0 ? 0 : (row >= p.x_src_rows ? p.x_src_rows - 1 : row);
    }
    x = p.x + static_cast<int64_t>(row) * p.K;
  } else if (ROUTED) {
    // every lane runs the same insertion over the token's logits (a few dozen instructions for 8 experts), so the expert
    // of this slot is known without a routing kernel in front; same arithmetic as topk_softmax_slots
    float val[2];
    int idx[2];
    // (in this form `bias` holds the logits, `residual` / `expert_ids` point at the weights and ids to write)
    const int top_k = static_cast<int>(gridDim.y);
    if (BF) topk_insert<2, MODEL_BF16>(p.bias, 0, p.num_experts, top_k, val, idx);
    else topk_insert<2, MODEL_F16>(p.bias, 0, p.num_experts, top_k, val, idx);
    const int e = __builtin_amdgcn_readfirstlane(slot == 0 ? idx[0] : idx[1]);
    qw += e * p.expert_w_stride;
    qs += e * p.expert_s_stride;
    if (blockIdx.x == 0 && threadIdx.x == 0 && slot == 0) {
      void* route_w = const_cast<uint16_t*>(p.residual);
      int32_t* route_ids = const_cast<int32_t*>(p.expert_ids);
      if (BF) softmax_store<2, MODEL_BF16>(val, idx, top_k, route_w, 0, route_ids);
      else softmax_store<2, MODEL_F16>(val, idx, top_k, route_w, 0, route_ids);
    }
  } else if (p.expert_ids != nullptr) {
    int e = p.expert_ids[slot];
    e = e < 0 ? 0 : (e >= p.num_experts ? p.num_experts - 1 : e);
    qw += e * p.expert_w_stride;
    qs += e * p.expert_s_stride;
  }

  // ---- x chunks go out first: waiting for them later must not wait for the weight loads,
  //      and the load counter retires in issue order
  const int chunks = NBX * (kpad / 8);
  // (the sum over two experts stages both slots' rows: row b of the staging is slot b's)
  const uint16_t* xs_base = SUM2 ? p.x : x;
  const int64_t xs_stride = SUM2 ? p.x_slot_stride : p.K;
  const bool vec = (p.K & 7) == 0;
  uint4 xv[XS];
  bool xok[XS];
#pragma unroll
  for (int i = 0; i < XS; ++i) {
    const int c = threadIdx.x + 256 * i;
    const int b = c / (kpad / 8);
    const int k = (c - b * (kpad / 8)) * 8;
    xok[i] = vec && c < chunks && k + 8 <= p.K;
    // always a valid, aligned 16-byte load (the base of x when the chunk is out of range or rows of x are not
    // 16-byte aligned, as an expert slot's row is when K is not a multiple of 8); zeroed at store time
    const uint16_t* src = xok[i] ? xs_base + static_cast<int64_t>(b) * xs_stride + k : p.x;
    xv[i] = *reinterpret_cast<const uint4*>(src);
  }

  // ---- this lane's groups (clamped so that every address is valid)
  int gidx[ITERS];
  bool gok[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int g = (ksub * ITERS + it) * 64 + lane;
    gok[it] = g < p.ng;
    gidx[it] = gok[it] ? g : p.ng - 1;
  }

  // ---- weight / scale / bias loads of one row set.  Branch-free on purpose: the wait-count
  //      insertion only keeps "the other buffer's loads may stay in flight" across the loop when
  //      every path issues the same loads.  A set past the end reads one cached line instead.
  uint4 wa[R][ITERS], wb[R][ITERS];
  uint32_t sa[R][ITERS], sb[R][ITERS];  // fp16 bits, kept 32 bits wide so that the in-flight values are never re-packed
  uint32_t ba = 0, bb = 0;  // low half: bias bits, high half: residual bits (lane r + R * b carries element (b, r))
  auto issue = [&](int set, uint4 (&wn)[R][ITERS], uint32_t (&sn)[R][ITERS], uint32_t& bn) {
    const bool live = set < nsets;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      int row = min(set * R + r, p.N - 1);  // rows past N are computed and dropped
      if (PAIRED) row = gate_up_row(row, p.N);
      const uint32_t* wr = qw + static_cast<int64_t>(row) * p.nw;
      const uint16_t* sr = qs + static_cast<int64_t>(row) * p.ng;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        wn[r][it] = *reinterpret_cast<const uint4*>(live ? wr + 4 * gidx[it] : qw);
        sn[r][it] = *(live ? sr + gidx[it] : qs);
      }
    }
    if constexpr (!EXTRA) return;
    // lane r carries the bias of row r of the set (read back with readlane at store time)
    const int brow = min(set * R + min(lane, R - 1), p.N - 1);
    bn = *((live && p.bias != nullptr) ? p.bias + brow : qs);
    // the residual rides with the set's loads too: fetched at store time it would sit behind the
    // next sets' weights in the in-order load queue and stall the wave until they all land
    const int e = min(lane, R * NB - 1);
    const int rrow = min(set * R + e % R, p.N - 1);
    const uint32_t rb = *((live && p.residual != nullptr)
                              ? p.residual + static_cast<int64_t>(slot + e / R) * p.N + rrow : qs);
    bn |= rb << 16;
  };
  int set_a = gw, set_b = gw + nwaves;
  issue(set_a, wa, sa, ba);
  issue(set_b, wb, sb, bb);

  // ---- stage x once per workgroup (zero beyond K), then one barrier
  if (vec) {
#pragma unroll
    for (int i = 0; i < XS; ++i) {
      const int c = threadIdx.x + 256 * i;
      if (c < chunks) smem[c] = xok[i] ? xv[i] : make_uint4(0, 0, 0, 0);
    }
  } else {  // K not a multiple of 8: rows of x are not 16-byte aligned, copy element-wise
    uint16_t* xs16 = reinterpret_cast<uint16_t*>(smem);
    for (int i = threadIdx.x; i < NBX * kpad; i += 256) {
      const int b = i / kpad, k = i - b * kpad;
      xs16[i] = k < p.K ? xs_base[static_cast<int64_t>(b) * xs_stride + k] : uint16_t(0);
    }
  }
  __syncthreads();

  // ---- this lane's x slice in pair order, and the correction terms
  uint32_t xr[NB][ITERS][HP];
  float corr[NB][ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      uint32_t nat[HP];
#pragma unroll
      for (int c = 0; c < G / 8; ++c) {
        uint4 raw = smem[((SUM2 ? slot : b) * kpad + gidx[it] * G) / 8 + c];
        if (!gok[it]) raw = make_uint4(0, 0, 0, 0);
        nat[4 * c + 0] = raw.x; nat[4 * c + 1] = raw.y; nat[4 * c + 2] = raw.z; nat[4 * c + 3] = raw.w;
      }
      corr[b][it] = permute_group<BITS, BF>(nat, xr[b][it]);
    }
  }

  // (shared K) the halves' row sums: [4 waves][kPartSlots] floats behind x
  constexpr int kPartSlots = 64;
  float* const part = reinterpret_cast<float*>(smem) + NBX * kpad / 2;
  int part_n = 0;
  // ---- persistent walk: reduce one set, then refill its registers with the set two strides on
  auto reduce = [&](int cur, const uint4 (&wc)[R][ITERS], const uint32_t (&sc)[R][ITERS],
                    uint32_t bias_bits) {
    float acc[R][NB];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        float a = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          const float sv = gok[it] ? to_f32(static_cast<uint16_t>(sc[r][it])) : 0.f;  // lanes past the last group add nothing
          const float gd = BF ? group_dot_bf16<BITS>(wc[r][it], xr[b][it], corr[b][it])
                              : group_dot<BITS>(wc[r][it], xr[b][it], corr[b][it]);
          a = fmaf(sv, gd, a);
        }
        acc[r][b] = wave_sum_last(a);
      }
    if constexpr (KW == 2) {
      // this half's sum of row `cur` waits in LDS: slot [wave of the workgroup][sets this wave has reduced so far]
      if (lane == 63 && cur < nsets) part[(threadIdx.x >> 6) * kPartSlots + part_n] = acc[0][0];
      ++part_n;
      return;
    }
    if constexpr (PAIRED) {
      if (lane == 63) {
#pragma unroll
        for (int r = 0; r < R; r += 2) {
          const int col = (cur * R + r) >> 1;
          if (col < (p.N >> 1)) {
#pragma unroll
            for (int b = 0; b < NB; ++b)
              static_cast<uint16_t*>(p.y)[static_cast<int64_t>(slot + b) * (p.N >> 1) + col] =
                  silu_mul_t<BF>(acc[r][b], acc[r + 1][b]);
          }
        }
      }
      return;
    }
    const float bias_lane = (EXTRA && p.bias != nullptr) ? to_f32(static_cast<uint16_t>(bias_bits & 0xffffu)) : 0.f;
    const float res_lane = (EXTRA && p.residual != nullptr) ? to_f32(static_cast<uint16_t>(bias_bits >> 16)) : 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float bias = __builtin_bit_cast(
          float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, bias_lane), r));
      const int row = cur * R + r;
      // read the other lanes' values here, with every lane active: inside the branch below only
      // lane 63 runs, and what a readlane sees of the inactive lanes is not defined
      float res[NB];
#pragma unroll
      for (int b = 0; b < NB; ++b)
        res[b] = EXTRA ? __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, res_lane), r + R * b))
                       : 0.f;
      if (lane == 63 && row < p.N) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          const float v = acc[r][b] + bias + res[b];
          const int64_t oi = static_cast<int64_t>(slot + b) * p.N + row;  // slot > 0 only if NB == 1
          if (p.out_f32) static_cast<float*>(p.y)[oi] = v;
          else static_cast<uint16_t*>(p.y)[oi] = BF ? f2bf(v) : f2h(v);
        }
      }
    }
  };
  // (the scheduling barriers keep each refill ahead of the next set's arithmetic: left alone, the scheduler starts that
  //  arithmetic first, and its wait for the set in flight then also holds back the refill: one set in flight, not two)
  while (set_a < nsets) {
    reduce(set_a, wa, sa, ba);
    set_a += 2 * nwaves;
    issue(set_a, wa, sa, ba);
    __builtin_amdgcn_sched_barrier(0);
    reduce(set_b, wb, sb, bb);  // past the end: rows >= N, nothing is stored
    set_b += 2 * nwaves;
    issue(set_b, wb, sb, bb);
    __builtin_amdgcn_sched_barrier(0);
  }
  if constexpr (KW == 2) {
    // the halves meet: lane i of the first wave of a pair owns the i-th set the pair walked (the launcher keeps that
    // count within kPartSlots)
    __syncthreads();
    const int set = gw + lane * nwaves;
    if constexpr (SUM2) {
      if (threadIdx.x < kPartSlots && set < nsets) {
        auto rnd = [](float v) { return BF ? bf2f(f2bf(v)) : h2f(f2h(v)); };
        const float y0 = rnd(part[lane] + part[kPartSlots + lane]);
        const float y1 = rnd(part[2 * kPartSlots + lane] + part[3 * kPartSlots + lane]);
        const float w0 = to_f32(p.residual[0]), w1 = to_f32(p.residual[1]);
        const float v = rnd(y0 * w0) + rnd(y1 * w1);
        static_cast<uint16_t*>(p.y)[set] = BF ? f2bf(v) : f2h(v);
      }
    } else if (ksub == 0 && lane < kPartSlots && set < nsets) {
      const int w = threadIdx.x >> 6;
      const float v = part[w * kPartSlots + lane] + part[(w + 1) * kPartSlots + lane];
      const int64_t oi = static_cast<int64_t>(slot) * p.N + set;
      if (p.out_f32) static_cast<float*>(p.y)[oi] = v;
      else static_cast<uint16_t*>(p.y)[oi] = BF ? f2bf(v) : f2h(v);
    }
  }
}

template <int BITS, int NB, int R, int ITERS, int MODE, bool MOE>
static hipError_t launch_mode(const GemvParams& p, dim3 grid, size_t lds, hipStream_t s) {
  const GemvTail t{p.expert_ids, p.expert_w_stride, p.expert_s_stride, p.x_slot_stride, p.bias, p.residual,
                   p.num_experts, p.indptr_i64, p.indptr, p.x_row_index, p.x_src_rows};
  if (p.bf16) hipLaunchKernelGGL((gemv_reg_kernel<BITS, NB, R, ITERS, MODE, true, MOE>), grid, dim3(256), lds, s,
                                    p.x, p.qw, p.qs, p.y, p.N, p.K, p.ng, p.nsets, p.nwaves, p.out_f32, t);
  else hipLaunchKernelGGL((gemv_reg_kernel<BITS, NB, R, ITERS, MODE, false, MOE>), grid, dim3(256), lds, s,
                          p.x, p.qw, p.qs, p.y, p.N, p.K, p.ng, p.nsets, p.nwaves, p.out_f32, t);
  return hipGetLastError();
}

template <int BITS, int NB, int R, int ITERS>
static hipError_t launch_k(const GemvParams& p0, int slots, int blocks, int nsets, hipStream_t s) {
  const size_t lds = static_cast<size_t>(NB) * p0.ng * GemvTraits<BITS>::G * 2;
  const dim3 grid(blocks, slots);
  GemvParams p = p0;
  p.nsets = nsets;
  p.nwaves = blocks * 4;
  const int mode = p.paired ? (p.routed ? 3 : 2) : ((p.bias != nullptr || p.residual != nullptr) ? 1 : 0);
  // the plain linear (one grid row, no expert ids, no expert-sorted rows) has an instantiation of its own
  const bool moe = slots != 1 || p.routed || p.indptr != nullptr || p.expert_ids != nullptr;
  note_kernel("gq::gemv_reg_kernel<%d,%d,%d,%d,%d,%s,%s,1>", BITS, NB, R, ITERS, mode, p.bf16 ? "true" : "false",
              moe ? "true" : "false");
  if (mode >= 2) {
    if constexpr (R % 2 == 0) {
      if (mode == 3) {  // (the launcher admits the routed form only as the fused gate/up form of one row)
        if constexpr (NB == 1) return launch_mode<BITS, NB, R, ITERS, 3, true>(p, grid, lds, s);
        else return hipErrorNotSupported;
      }
      return moe ? launch_mode<BITS, NB, R, ITERS, 2, true>(p, grid, lds, s)
                 : launch_mode<BITS, NB, R, ITERS, 2, false>(p, grid, lds, s);
    } else {
      return hipErrorNotSupported;
    }
  }
  if (mode == 1)
    return moe ? launch_mode<BITS, NB, R, ITERS, 1, true>(p, grid, lds, s)
               : launch_mode<BITS, NB, R, ITERS, 1, false>(p, grid, lds, s);
  return moe ? launch_mode<BITS, NB, R, ITERS, 0, true>(p, grid, lds, s)
             : launch_mode<BITS, NB, R, ITERS, 0, false>(p, grid, lds, s);
}

// Long K shared between two neighbouring waves (KW = 2): HALF groups per lane and wave.
template <int BITS, int HALF>
static hipError_t launch_shared_k(const GemvParams& p0, int slots, int blocks, int nsets, hipStream_t s) {
  const size_t lds = static_cast<size_t>(p0.sum2 ? 2 : 1) * p0.ng * GemvTraits<BITS>::G * 2 + 4 * 64 * sizeof(float);
  const dim3 grid(blocks, p0.sum2 ? 1 : slots);
  GemvParams p = p0;
  p.nsets = nsets;
  p.nwaves = blocks * 4;
  const bool moe = slots != 1 || p.indptr != nullptr || p.expert_ids != nullptr;
  note_kernel("gq::gemv_reg_kernel<%d,1,1,%d,0,%s,%s,2>", BITS, HALF, p.bf16 ? "true" : "false", moe ? "true" : "false");
  const GemvTail t{p.expert_ids, p.expert_w_stride, p.expert_s_stride, p.x_slot_stride, p.bias, p.residual,
                   p.num_experts, p.indptr_i64, p.indptr, p.x_row_index, p.x_src_rows};
#define GQ_SHARED_K(BF_, MOE_)                                                                                      \
  hipLaunchKernelGGL((gemv_reg_kernel<BITS, 1, 1, HALF, 0, BF_, MOE_, 2>), grid, dim3(256), lds, s, p.x, p.qw, p.qs, \
                     p.y, p.N, p.K, p.ng, p.nsets, p.nwaves, p.out_f32, t)
  if (p.sum2) {  // both expert slots in every workgroup, their results weighted and summed at the end
    note_kernel("gq::gemv_reg_kernel<%d,1,1,%d,4,%s,true,2>", BITS, HALF, p.bf16 ? "true" : "false");
    if (p.bf16)
      hipLaunchKernelGGL((gemv_reg_kernel<BITS, 1, 1, HALF, 4, true, true, 2>), grid, dim3(256), lds, s, p.x, p.qw, p.qs,
                         p.y, p.N, p.K, p.ng, p.nsets, p.nwaves, p.out_f32, t);
    else
      hipLaunchKernelGGL((gemv_reg_kernel<BITS, 1, 1, HALF, 4, false, true, 2>), grid, dim3(256), lds, s, p.x, p.qw, p.qs,
                         p.y, p.N, p.K, p.ng, p.nsets, p.nwaves, p.out_f32, t);
    return hipGetLastError();
  }
  if (p.bf16) {
    if (moe) GQ_SHARED_K(true, true);
    else GQ_SHARED_K(true, false);
  } else {
    if (moe) GQ_SHARED_K(false, true);
    else GQ_SHARED_K(false, false);
  }
#undef GQ_SHARED_K
  return hipGetLastError();
}

template <int BITS, int NB, int R>
static hipError_t launch_iters(const GemvParams& p, int slots, int iters, int blocks, int nsets,
                               hipStream_t s) {
  switch (iters) {
    case 1: return launch_k<BITS, NB, R, 1>(p, slots, blocks, nsets, s);
    case 2: return launch_k<BITS, NB, R, 2>(p, slots, blocks, nsets, s);
    case 3: if constexpr (R * NB <= 2) return launch_k<BITS, NB, R, 3>(p, slots, blocks, nsets, s); break;
    case 4: if constexpr (R * NB <= 2) return launch_k<BITS, NB, R, 4>(p, slots, blocks, nsets, s); break;
    case 5: if constexpr (R * NB == 1) return launch_k<BITS, NB, R, 5>(p, slots, blocks, nsets, s); break;
    case 6: if constexpr (R * NB == 1) return launch_k<BITS, NB, R, 6>(p, slots, blocks, nsets, s); break;
    case 7: if constexpr (R * NB == 1) return launch_k<BITS, NB, R, 7>(p, slots, blocks, nsets, s); break;
    case 8: if constexpr (R * NB == 1) return launch_k<BITS, NB, R, 8>(p, slots, blocks, nsets, s); break;
    // K up to 24 Ki (q3: 30 Ki): Qwen2-7B's down_proj, 3584 x 18944, runs 10 groups per lane
    case 9: case 10: if constexpr (R * NB == 1) return launch_k<BITS, NB, R, 10>(p, slots, blocks, nsets, s); break;
    case 11: case 12: if constexpr (R * NB == 1) return launch_k<BITS, NB, R, 12>(p, slots, blocks, nsets, s); break;
    default: break;
  }
  return hipErrorNotSupported;
}

template <int BITS>
static hipError_t launch_bits(const GemvParams& p, int nb, int slots, hipStream_t s) {
  const int iters = (p.ng + 63) / 64;
  if (iters < 1 || iters > 12) return hipErrorNotSupported;
  // register budget: R * ITERS loads in flight, NB * ITERS x slices resident
  int rmax = iters <= 2 ? 4 : (iters <= 4 ? 2 : 1);
  if (nb == 2) rmax = iters <= 2 ? 2 : (iters <= 4 ? 1 : 0);
  if (nb > 2 || rmax == 0) return hipErrorNotSupported;
  // Measured on MI355X (q4, batch 1): short K wants one row per set until the matrix is large
  // (fine-grained sets hide the pipeline fill of a 5 us kernel), large matrices want 2 rows per
  // set; long K is register-bound (one wave per SIMD, or two that share every row's K).
  const int64_t rows_total = static_cast<int64_t>(p.N) * slots;
  int R = options().gemv_rows_per_wave;
  if (R != 1 && R != 2 && R != 4) {
    // (four rows per set, once the choice for 65536 rows and more, measures 2 % behind two on 128256 x 4096 since the
    //  kernel's arguments arrive in registers: 47.1 -> 46.1 us)
    if (iters <= 2) R = rows_total >= 16384 ? 2 : 1;
    else R = 1;  // K of 5120 / 8192 (13B, 70B projections): 8-17 % faster than two rows per set
  }
  if (R > rmax) R = rmax;
  if (p.paired) {
    if (rmax < 2) return hipErrorNotSupported;
    if (R < 2) R = 2;
  }
  const int nsets = (p.N + R - 1) / R;
  int waves;
  if (options().gemv_waves > 0) {
    waves = options().gemv_waves;
  } else if (iters > 2) {
    // one wave per SIMD; two once the registers allow it (up to 4 groups per lane) and the rows keep them busy
    waves = (iters <= 4 && rows_total >= 12288) ? 2048 : 1024;
  } else {
    const int64_t half = static_cast<int64_t>(nsets) * slots / 2;  // about two sets per wave
    waves = half <= 3072 ? static_cast<int>(half) : 2048;
    if (waves < 1024) waves = 1024;
  }
  // grid.y = slots: whole workgroups per slot, rounded down, so that the grid stays within the one or two
  // workgroups per CU the totals above stand for (6 slots rounded up are 516 workgroups: four of them run alone
  // after the other 512, and 6 rows cost what 8 do)
  if (slots > 1) waves = waves / (4 * slots) * 4;
  if (waves < 4) waves = 4;
  const int rounds = (nsets + waves - 1) / waves;
  // Long K (5 to 12 groups per lane), one row, plain epilogue: two neighbouring waves share every row's K (3 to 6 groups
  // per lane each, so that two waves fit a SIMD where the whole-K form runs one), twice the waves.
  // Tuning override: gemv_ksplit 0 | 1.
  if (p.sum2) {
    // one token's e2 and the weighted sum over its two experts: four waves per row walker (2 slots x 2 halves of K),
    // 512 walkers; 2 to 6 groups per lane and wave, both rows of x in LDS
    const int half = (iters + 1) / 2;
    const int walkers = 512;
    const int rounds2 = (p.N + walkers - 1) / walkers;
    const int64_t lds2 = 2ll * p.ng * GemvTraits<BITS>::G * 2 + 1024;
    if (nb != 1 || slots != 2 || iters < 3 || rounds2 > 64 || lds2 > 65536) return hipErrorNotSupported;
    const int blocks2 = (p.N + rounds2 - 1) / rounds2;
    switch (half) {
      case 2: return launch_shared_k<BITS, 2>(p, slots, blocks2, p.N, s);
      case 3: return launch_shared_k<BITS, 3>(p, slots, blocks2, p.N, s);
      case 4: return launch_shared_k<BITS, 4>(p, slots, blocks2, p.N, s);
      case 5: return launch_shared_k<BITS, 5>(p, slots, blocks2, p.N, s);
      case 6: return launch_shared_k<BITS, 6>(p, slots, blocks2, p.N, s);
      default: return hipErrorNotSupported;
    }
  }
  const bool plain = !p.paired && !p.routed && p.bias == nullptr && p.residual == nullptr;
  // ... and on K = 4096 (two groups per lane: one per wave of a pair) for the mid-sized matrices, one row per set whatever
  // was chosen above: 28672 x 4096 14.8 -> 13.8 us on 4096 waves, 6144 x 4096 5.24 -> 5.03 on 6144; 4096 x 4096 and
  // 128256 x 4096 unchanged (same-process A/B, graph replay over rotating weights), so they keep the whole-K form.
  const bool short_pair = iters == 2 && slots == 1 && p.N >= 6144 && p.N < 65536 && options().gemv_waves <= 0 &&
                          options().gemv_rows_per_wave < 0;
  if ((iters >= 5 || short_pair || (options().gemv_ksplit == 1 && iters >= 2)) && nb == 1 && plain &&
      options().gemv_ksplit != 0) {
    const int nsets1 = p.N;
    int walkers = waves;  // (long K: twice the waves of the whole-K form)
    if (iters < 5) walkers = (options().gemv_waves > 0 ? options().gemv_waves : (p.N >= 16384 ? 4096 : 6144)) / 2;
    if (walkers < 1) walkers = 1;
    const int rounds1 = (nsets1 + walkers - 1) / walkers;
    if (rounds1 <= 64 && (iters < 5 || R == 1)) {
    const int half = (iters + 1) / 2;
    const int blocks2 = (2 * ((nsets1 + rounds1 - 1) / rounds1) + 3) / 4;
    switch (half) {
      case 1: return launch_shared_k<BITS, 1>(p, slots, blocks2, nsets1, s);
      case 2: return launch_shared_k<BITS, 2>(p, slots, blocks2, nsets1, s);
      case 3: return launch_shared_k<BITS, 3>(p, slots, blocks2, nsets1, s);
      case 4: return launch_shared_k<BITS, 4>(p, slots, blocks2, nsets1, s);
      case 5: return launch_shared_k<BITS, 5>(p, slots, blocks2, nsets1, s);
      case 6: return launch_shared_k<BITS, 6>(p, slots, blocks2, nsets1, s);
      default: break;
    }
    }
  }
  const int blocks = ((nsets + rounds - 1) / rounds + 3) / 4;  // even share of sets per wave
  if (nb == 1) {
    if (R == 4) return launch_iters<BITS, 1, 4>(p, slots, iters, blocks, nsets, s);
    if (R == 2) return launch_iters<BITS, 1, 2>(p, slots, iters, blocks, nsets, s);
    return launch_iters<BITS, 1, 1>(p, slots, iters, blocks, nsets, s);
  }
  if (R == 2) return launch_iters<BITS, 2, 2>(p, slots, iters, blocks, nsets, s);
  return launch_iters<BITS, 2, 1>(p, slots, iters, blocks, nsets, s);
}

hipError_t launch_gemv_reg(const GemvParams& p, int bits, int nb, int slots, hipStream_t s) {
  if (p.ng == 0) return hipErrorNotSupported;
  if (p.routed && (slots < 1 || slots > 2 || p.num_experts > 64 || nb != 1 || !p.paired)) return hipErrorNotSupported;
  // the x staging always issues whole 16-byte loads (from the base of x where a chunk is unusable): x must hold
  // at least 8 halves per row for that address to be readable
  if (p.K < 8) return hipErrorNotSupported;
  if (static_cast<int64_t>(nb) * p.ng * (bits == 4 ? 32 : 40) * 2 > 65536) return hipErrorNotSupported;
  return bits == 4 ? launch_bits<4>(p, nb, slots, s) : launch_bits<3>(p, nb, slots, s);
}

}  // namespace gq
