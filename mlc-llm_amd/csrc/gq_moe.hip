// Routing glue of the MoE layer: top-k + softmax, expert-major cumsum, gather/scatter plans,
// indptr, row gather/scatter, silu*mul and the weighted top-k combine.
//
// Replaces the TIR of python/mlc_llm/op/moe_misc.py in the reference: gating_softmax_topk
// (:135-235), moe_cumsum (:371-450), get_indices (:453-525), get_indptr (:528-605),
// scatter_output (:608-645), moe_sum (:14-32), and the elementwise glue of
// model/mixtral/mixtral_model.py:64-117.  All of it is integer / tiny fp16 work.
#include <type_traits>

#include "gq_common.hpp"
#include "gq_internal.hpp"
#include "gq_topk.hpp"

namespace gq {

constexpr int kMaxTopK = 8;

// One thread per token: insertion top-k with strict '>' (ties keep the lower expert index),
// then softmax over the k selected logits in fp32.
// KMAX: slots kept (k <= KMAX); the insertion is a chain of KMAX * KMAX predicated moves per expert,
// so the common k <= 2 gets its own, 16 times shorter, instance
template <int KMAX, int DT>
__device__ __forceinline__ void topk_softmax_slots(const void* __restrict__ logits, int64_t row0, int ne, int k,
                                                   void* __restrict__ w, int64_t w0, int32_t* __restrict__ ids) {
  float val[KMAX];
  int idx[KMAX];
  topk_insert<KMAX, DT>(logits, row0, ne, k, val, idx);
  softmax_store<KMAX, DT>(val, idx, k, w, w0, ids);
}

// token t: logits[t, :] -> w[t, :k], ids[t, :k]
template <int DT>
__device__ __forceinline__ void topk_softmax_token(const void* __restrict__ logits, int64_t t, int ne, int k,
                                                   void* __restrict__ w, int32_t* __restrict__ ids) {
  if (k <= 2) topk_softmax_slots<2, DT>(logits, t * ne, ne, k, w, t * k, ids + t * k);
  else if (k <= 4) topk_softmax_slots<4, DT>(logits, t * ne, ne, k, w, t * k, ids + t * k);
  else topk_softmax_slots<kMaxTopK, DT>(logits, t * ne, ne, k, w, t * k, ids + t * k);
}

template <int DT>
__global__ __launch_bounds__(256) void topk_softmax_kernel(const void* __restrict__ logits, int64_t T, int ne, int k,
                                                           void* __restrict__ w, int32_t* __restrict__ ids) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (t >= T) return;
  topk_softmax_token<DT>(logits, t, ne, k, w, ids);
}

// gating_topk (moe_misc.py:63-132) and the norm_topk_prob = False branch of gating_softmax_topk (:234-235), one
// thread per token: SOFTMAX computes softmax over ALL experts in fp32 (exp(x - max) / sum, summed left to right),
// rounds each score to the model dtype, and then, in both forms, the same insertion top-k runs on the scores and
// returns them as they are (no renormalisation).  Scores that round to the same value tie: lower index first.
template <int KMAX, int DT, bool SOFTMAX>
__device__ __forceinline__ void topk_scores_slots(const void* __restrict__ x, int64_t row0, int ne, int k,
                                                  void* __restrict__ w, int64_t w0, int32_t* __restrict__ ids) {
  float mx = 0.f, den = 0.f;
  if (SOFTMAX) {
    mx = Elem<DT>::load(x, row0);
    for (int e = 1; e < ne; ++e) mx = fmaxf(mx, Elem<DT>::load(x, row0 + e));
    for (int e = 0; e < ne; ++e) {
      const float ex = expf(Elem<DT>::load(x, row0 + e) - mx);
      den = e == 0 ? ex : den + ex;
    }
  }
  float val[KMAX];
  int idx[KMAX];
#pragma unroll
  for (int i = 0; i < KMAX; ++i) {
    val[i] = Elem<DT>::kLowest;
    idx[i] = 0;
  }
  for (int e = 0; e < ne; ++e) {
    float v = Elem<DT>::load(x, row0 + e);
    if (SOFTMAX) v = Elem<DT>::rnd(expf(v - mx) / den);
    bool placed = false;
#pragma unroll
    for (int i = 0; i < KMAX; ++i) {
      if (i < k && !placed && v > val[i]) {
#pragma unroll
        for (int j = KMAX - 1; j > 0; --j) {
          if (j > i && j < k) {
            val[j] = val[j - 1];
            idx[j] = idx[j - 1];
          }
        }
        val[i] = v;
        idx[i] = e;
        placed = true;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < KMAX; ++i) {
    if (i < k) {
      Elem<DT>::store(w, w0 + i, val[i]);
      ids[i] = idx[i];
    }
  }
}

template <int DT, bool SOFTMAX>
__global__ __launch_bounds__(256) void topk_scores_kernel(const void* __restrict__ x, int64_t T, int ne, int k,
                                                          void* __restrict__ w, int32_t* __restrict__ ids) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (t >= T) return;
  if (k <= 2) topk_scores_slots<2, DT, SOFTMAX>(x, t * ne, ne, k, w, t * k, ids + t * k);
  else topk_scores_slots<kMaxTopK, DT, SOFTMAX>(x, t * ne, ne, k, w, t * k, ids + t * k);
}

// One wave per token, for many experts or many slots (the thread-per-token insertion above costs
// ne * k * k predicated moves on one lane): lane l holds the logits of experts l, l + 64, ...; k rounds
// of a wave-wide arg-max (larger value first, equal values by lower expert index: the order the
// insertion produces) pick the slots (by rank counting up to 128 experts), and lane 0 finishes with the same softmax.  Logits that are not
// above min_value(dtype), NaN included, are never picked; slots left empty keep (min_value, expert 0).
constexpr int kWaveTopkChunks = 8;  // experts per lane: ne <= 512
template <int DT>
__device__ __forceinline__ void topk_softmax_wave(const void* __restrict__ logits, int64_t t, int ne, int k,
                                                  void* __restrict__ w, int32_t* __restrict__ ids) {
  const int lane = threadIdx.x & 63;
  const int nch = (ne + 63) >> 6;
  float v[kWaveTopkChunks];
  unsigned out_of_running = 0;  // bit c: expert lane + 64 * c is absent, not placeable or already picked
#pragma unroll
  for (int c = 0; c < kWaveTopkChunks; ++c) {
    const int e = lane + 64 * c;
    v[c] = Elem<DT>::kLowest;
    if (c < nch && e < ne) v[c] = Elem<DT>::load(logits, t * ne + e);
    if (!(v[c] > Elem<DT>::kLowest)) out_of_running |= 1u << c;
  }
  constexpr int kNone = 0x7fffffff;
  float val[kMaxTopK];
  int idx[kMaxTopK];
  if (nch <= 2) {
    // up to 128 experts: every lane counts the experts that come before its own in that order (their rank)
    // from lane broadcasts, with no trip through the LDS crossbar; slot i is the expert of rank i
    int rank[2] = {0, 0};
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2) {
      if (c2 < nch) {  // uniform
#pragma unroll
        for (int l = 0; l < 64; ++l) {
          const float ov = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v[c2]), l));
          const int oe = l + 64 * c2;  // (a logit that cannot be placed never wins the comparisons below)
          rank[0] += (ov > v[0] || (ov == v[0] && oe < lane)) ? 1 : 0;
          if (nch == 2) rank[1] += (ov > v[1] || (ov == v[1] && oe < lane + 64)) ? 1 : 0;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kMaxTopK; ++i) {
      val[i] = Elem<DT>::kLowest;
      idx[i] = 0;
      if (i < k) {
        const unsigned long long m0 = __ballot(!(out_of_running & 1u) && rank[0] == i);
        const unsigned long long m1 = __ballot(nch == 2 && !(out_of_running & 2u) && rank[1] == i);
        if (m0 != 0ull) {
          const int src = __builtin_ctzll(m0);
          val[i] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v[0]), src));
          idx[i] = src;
        } else if (m1 != 0ull) {
          const int src = __builtin_ctzll(m1);
          val[i] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v[1]), src));
          idx[i] = src + 64;
        }
      }
    }
    if (lane == 0) softmax_store<kMaxTopK, DT>(val, idx, k, w, t * k, ids + t * k);
    return;
  }
#pragma unroll
  for (int i = 0; i < kMaxTopK; ++i) {
    val[i] = Elem<DT>::kLowest;
    idx[i] = 0;
    if (i < k) {  // uniform
      float bv = Elem<DT>::kLowest;
      int be = kNone;
#pragma unroll
      for (int c = 0; c < kWaveTopkChunks; ++c)
        if (c < nch && !((out_of_running >> c) & 1u) && (be == kNone || v[c] > bv)) {
          bv = v[c];
          be = lane + 64 * c;
        }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off);
        const int oe = __shfl_xor(be, off);
        if (oe != kNone && (be == kNone || ov > bv || (ov == bv && oe < be))) {
          bv = ov;
          be = oe;
        }
      }
      if (be != kNone) {  // uniform: every lane ends with the same winner
        val[i] = bv;
        idx[i] = be;
        if ((be & 63) == lane) out_of_running |= 1u << (be >> 6);
      }
    }
  }
  if (lane == 0) softmax_store<kMaxTopK, DT>(val, idx, k, w, t * k, ids + t * k);
}

static inline bool use_wave_topk(int ne, int k) { return ne * k > 64 && ne <= 64 * kWaveTopkChunks; }

template <int DT>
__global__ __launch_bounds__(256) void topk_softmax_wave_kernel(const void* __restrict__ logits, int64_t T, int ne,
                                                                int k, void* __restrict__ w,
                                                                int32_t* __restrict__ ids) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (t >= T) return;  // whole waves
  topk_softmax_wave<DT>(logits, t, ne, k, w, ids);
}

// The whole routing step of a MoE layer in one workgroup, for batches a single workgroup can scan:
// top-k + softmax per token, then, expert by expert, the token-ordered positions of the (expert,
// token) pairs: the results of gating_softmax_topk, moe_cumsum, get_indices and get_indptr without
// the [experts, T] cumsum table in memory and without four launches.  pos_of_slot is the inverse of
// reverse_indices (where slot t * k + j sits in the expert-sorted order).
template <int DT>
__global__ __launch_bounds__(1024) void moe_route_kernel(const void* __restrict__ logits, int T, int ne,
                                                         int k, void* __restrict__ w,
                                                         int32_t* __restrict__ ids, int32_t* __restrict__ tok,
                                                         int32_t* __restrict__ rev,
                                                         int32_t* __restrict__ pos_of_slot, int out_i64,
                                                         void* indptr, int ids_in_lds) {
  __shared__ int wave_tot[2][16];
  extern __shared__ int32_t ids_lds[];  // [T * k] when the launch gave it room: the scans below read
                                        // every id once per expert, and a trip to L2 each time is what
                                        // the kernel would otherwise spend its time on
  const int tid = threadIdx.x, nthreads = blockDim.x;  // a multiple of 64, sized to the batch
  const int lane = tid & 63, wave = tid >> 6, nwaves = nthreads >> 6;
  for (int t = tid; t < T; t += nthreads) {
    topk_softmax_token<DT>(logits, t, ne, k, w, ids);
    if (ids_in_lds)
      for (int j = 0; j < k; ++j) ids_lds[t * k + j] = ids[static_cast<int64_t>(t) * k + j];  // own writes
  }
  __syncthreads();  // ids written above are read back by other threads below
  const int32_t* id_src = ids_in_lds ? ids_lds : ids;
  int base = 0, round = 0;
  if (tid == 0) {
    if (out_i64) static_cast<int64_t*>(indptr)[0] = 0;
    else static_cast<int32_t*>(indptr)[0] = 0;
  }
  for (int e = 0; e < ne; ++e) {
    for (int t0 = 0; t0 < T; t0 += nthreads, ++round) {
      const int t = t0 + tid;
      int slot = -1;  // the first j with ids[t, j] == e (the mask is boolean: a repeated id counts once)
      if (t < T)
        for (int j = k - 1; j >= 0; --j)
          if (id_src[static_cast<int64_t>(t) * k + j] == e) slot = t * k + j;
      // tokens of this expert among the wave's 64, and before this lane
      const unsigned long long m = __ballot(slot >= 0);
      const int before = __popcll(m & ((1ull << lane) - 1ull));
      int pre = 0, tot = __popcll(m);
      if (nwaves > 1) {  // uniform; the two LDS rows alternate so that one barrier per round is enough
        int* wt = wave_tot[round & 1];
        if (lane == 0) wt[wave] = tot;
        __syncthreads();
        tot = 0;
        for (int wv = 0; wv < nwaves; ++wv) {
          const int c = wt[wv];
          if (wv < wave) pre += c;
          tot += c;
        }
      }
      if (slot >= 0) {
        const int pos = base + pre + before;  // < T * k: every pair counted here is a distinct (t, j)
        tok[pos] = t;
        rev[pos] = slot;
        pos_of_slot[slot] = pos;
      }
      base += tot;
    }
    if (tid == 0) {
      if (out_i64) static_cast<int64_t*>(indptr)[e + 1] = base;
      else static_cast<int32_t*>(indptr)[e + 1] = base;
    }
  }
}

// The same routing step organised by slot, for up to 8 slots per thread and a count table that fits LDS: thread
// tid owns slots tid, tid + nthreads, ...; one pass of wave ballots per expert (or, past 16 experts, of
// pairwise id comparisons among the wave's lanes) gives every slot its rank among its wave's slots of the
// same expert and every (expert, 64-slot chunk) its count; a scan of that
// table in (expert, chunk) order turns the counts into offsets.  Three barriers in all, where the
// kernel above takes one per expert and round and re-reads k ids per token and expert.
// do_topk 0: ids (and w) were produced by an earlier launch.  wave_topk: one wave per token.
// flags = out_i64 | do_topk << 1 | wave_topk << 2 | waves of the workgroup << 8: with them in one word, everything the
// kernel needs before its first loads is among the arguments that arrive in scalar registers.
template <int DT>
__global__ __launch_bounds__(1024) void moe_route_slots_kernel(const void* __restrict__ logits, int T, int ne, int k,
                                                               int flags, void* __restrict__ w,
                                                               int32_t* __restrict__ ids, int32_t* __restrict__ tok,
                                                               int32_t* __restrict__ rev,
                                                               int32_t* __restrict__ pos_of_slot, void* indptr) {
  constexpr int kSlotsPerThread = 8;
  __shared__ int wave_tot[16];
  extern __shared__ int32_t cnt[];  // [ne, nchunks]: counts, then exclusive offsets
  const int out_i64 = flags & 1, do_topk = flags & 2, wave_topk = flags & 4;
  const int tid = threadIdx.x, nthreads = (flags >> 8) << 6;
  const int lane = tid & 63, wave = tid >> 6, nwaves = nthreads >> 6;
  const int S = T * k, nchunks = (S + 63) >> 6, N = ne * nchunks;
  if (do_topk) {
    if (wave_topk)
      for (int t = wave; t < T; t += nwaves) topk_softmax_wave<DT>(logits, t, ne, k, w, ids);
    else
      for (int t = tid; t < T; t += nthreads) topk_softmax_token<DT>(logits, t, ne, k, w, ids);
    __syncthreads();  // ids written above are read back by other threads below
  }
  if (ne > 16) {  // uniform
    for (int i = tid; i < N; i += nthreads) cnt[i] = 0;
    __syncthreads();
  }
  const unsigned long long lower = (1ull << lane) - 1ull;
  int myid[kSlotsPerThread], before[kSlotsPerThread];
#pragma unroll
  for (int r = 0; r < kSlotsPerThread; ++r) {
    const int s = r * nthreads + tid;
    myid[r] = -1;  // no slot, or a repeated id of its token (the mask is boolean: it counts once)
    before[r] = 0;
    if (r * nthreads + wave * 64 < S) {  // per wave: its 64-slot chunk exists
      if (s < S) {
        const int id = ids[s], j = s % k;
        bool repeated = false;
#pragma unroll
        for (int jj = 0; jj < kMaxTopK - 1; ++jj)  // unconditional loads (its own id past j), all in flight together
          repeated |= (ids[s - j + (jj < j ? jj : j)] == id) & (jj < j);
        if (!repeated) myid[r] = id;
      }
      if (ne > 16) {
        // many experts: the lanes compare ids pairwise instead (64 lane broadcasts whatever the expert count);
        // the last slot of an expert in the chunk records the expert's count in the zeroed table
        int after = 0;
#pragma unroll
        for (int l = 0; l < 64; ++l) {
          const int same = __builtin_amdgcn_readlane(myid[r], l) == myid[r] ? 1 : 0;
          before[r] += l < lane ? same : 0;
          after += l > lane ? same : 0;
        }
        if (myid[r] >= 0 && after == 0) cnt[myid[r] * nchunks + r * nwaves + wave] = before[r] + 1;
      } else
      for (int e0 = 0; e0 < ne; e0 += 64) {
        int mine = 0;  // lane l: slots of expert e0 + l in this wave's chunk
        const int e1 = e0 + 64 < ne ? e0 + 64 : ne;
        for (int e = e0; e < e1; ++e) {
          const unsigned long long m = __ballot(myid[r] == e);
          if (myid[r] == e) before[r] = __popcll(m & lower);
          if (lane == e - e0) mine = __popcll(m);
        }
        if (e0 + lane < ne) cnt[(e0 + lane) * nchunks + r * nwaves + wave] = mine;
      }
    }
  }
  __syncthreads();
  // exclusive scan of cnt[0, N): consecutive runs per thread, a wave scan of the run sums, wave totals
  const int per = (N + nthreads - 1) / nthreads;
  const int i0 = tid * per, i1 = (i0 + per < N) ? i0 + per : N;
  int sum = 0;
  for (int i = i0; i < i1; ++i) sum += cnt[i];
  int inc = sum;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int o = __shfl_up(inc, off);
    if (lane >= off) inc += o;
  }
  if (lane == 63) wave_tot[wave] = inc;
  __syncthreads();
  int pre = 0, total = 0;
  for (int wv = 0; wv < nwaves; ++wv) {
    const int c = wave_tot[wv];
    if (wv < wave) pre += c;
    total += c;
  }
  int run = pre + inc - sum;
  for (int i = i0; i < i1; ++i) {
    const int c = cnt[i];
    cnt[i] = run;
    run += c;
  }
  __syncthreads();
  for (int e = tid; e <= ne; e += nthreads) {
    const int v = e == 0 ? 0 : (e < ne ? cnt[e * nchunks] : total);
    if (out_i64) static_cast<int64_t*>(indptr)[e] = v;
    else static_cast<int32_t*>(indptr)[e] = v;
  }
#pragma unroll
  for (int r = 0; r < kSlotsPerThread; ++r) {
    if (myid[r] >= 0) {
      const int s = r * nthreads + tid;
      const int pos = cnt[myid[r] * nchunks + r * nwaves + wave] + before[r];  // < S: distinct (t, j) pairs
      tok[pos] = s / k;
      rev[pos] = s;
      pos_of_slot[s] = pos;
    }
  }
}

// Block e produces cumsum[e*T .. e*T+T): it first counts, on its own, how many (expert, token)
// mask bits precede expert e (LDS histogram over all ids), then scans expert e's token mask.
// No block depends on another, so the kernel needs no workspace and no grid sync.
__global__ __launch_bounds__(1024) void moe_cumsum_kernel(const int32_t* __restrict__ ids,
                                                          int64_t T, int k, int ne,
                                                          int32_t* __restrict__ cumsum) {
  __shared__ int hist[256];
  __shared__ int wave_tot[16];
  __shared__ int base_sh;
  const int e = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  if (tid < 256) hist[tid] = 0;
  __syncthreads();
  for (int64_t t = tid; t < T; t += 1024) {
    for (int j = 0; j < k; ++j) {
      const int id = ids[t * k + j];
      bool dup = false;  // the mask is boolean: a repeated id in one token counts once
      for (int j2 = 0; j2 < j; ++j2) dup |= (ids[t * k + j2] == id);
      if (!dup && id >= 0 && id < e) atomicAdd(&hist[id], 1);
    }
  }
  __syncthreads();
  if (tid == 0) {
    int s = 0;
    for (int i = 0; i < e; ++i) s += hist[i];
    base_sh = s;
  }
  __syncthreads();
  int base = base_sh;
  for (int64_t t0 = 0; t0 < T; t0 += 1024) {
    const int64_t t = t0 + tid;
    int bit = 0;
    if (t < T)
      for (int j = 0; j < k; ++j) bit |= (ids[t * k + j] == e);
    // inclusive scan inside the wave
    int v = bit;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int n = __shfl_up(v, off, 64);
      if (lane >= off) v += n;
    }
    if (lane == 63) wave_tot[wave] = v;
    __syncthreads();
    int pre = 0, tot = 0;
    for (int wv = 0; wv < 16; ++wv) {
      const int c = wave_tot[wv];
      if (wv < wave) pre += c;
      tot += c;
    }
    if (t < T) cumsum[static_cast<int64_t>(e) * T + t] = base + pre + v;
    base += tot;
    __syncthreads();
  }
}

__global__ __launch_bounds__(256) void get_indices_kernel(const int32_t* __restrict__ cumsum,
                                                          const int32_t* __restrict__ ids,
                                                          int64_t T, int k, int ne,
                                                          int32_t* __restrict__ rev,
                                                          int32_t* __restrict__ tok) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= T * k) return;
  const int64_t b = i / k;
  const int e = ids[i];
  if (e < 0 || e >= ne) return;  // an id outside the expert range owns no slot
  const int64_t pos = static_cast<int64_t>(cumsum[e * T + b]) - 1;
  if (pos >= 0 && pos < T * k) {
    rev[pos] = static_cast<int32_t>(i);
    tok[pos] = static_cast<int32_t>(b);
  }
}

__global__ void get_indptr_kernel(const int32_t* __restrict__ cumsum, int64_t ne, int64_t T,
                                  int inclusive, int out_i64, void* indptr) {
  const int64_t i = threadIdx.x + static_cast<int64_t>(blockIdx.x) * blockDim.x;
  const int64_t n = inclusive ? ne : ne + 1;
  if (i >= n) return;
  int32_t v;
  if (inclusive) v = cumsum[(i + 1) * T - 1];
  else v = i > 0 ? cumsum[i * T - 1] : 0;
  if (out_i64) static_cast<int64_t*>(indptr)[i] = v;
  else static_cast<int32_t*>(indptr)[i] = v;
}

// gather (out[r] = x[idx[r]]) or scatter (out[idx[r]] = x[r]) of fp16 rows; VEC halves per thread
template <int VEC>
__global__ __launch_bounds__(256) void move_rows_kernel(const uint16_t* __restrict__ x,
                                                        const int32_t* __restrict__ idx, int64_t R,
                                                        int64_t H, int64_t bound, int scatter,
                                                        uint16_t* __restrict__ out) {
  const int64_t per_row = H / VEC;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= R * per_row) return;
  const int64_t r = i / per_row;
  const int64_t c = (i - r * per_row) * VEC;
  int64_t j = idx[r];
  if (j < 0 || j >= bound) return;  // never touch memory outside the tensors
  const int64_t src = scatter ? r : j, dst = scatter ? j : r;
  if (VEC == 8) {
    *reinterpret_cast<uint4*>(out + dst * H + c) = *reinterpret_cast<const uint4*>(x + src * H + c);
  } else {
    out[dst * H + c] = x[src * H + c];
  }
}

// out[r, i] = fp16(silu(x[r, i])) * x[r, I + i]; silu in fp32, one rounding, then an fp16 product
// (other model dtypes: the same two roundings in that dtype; float32 evaluates silu with expf and a true divide)
template <int DT>
__global__ __launch_bounds__(256) void silu_mul_kernel(const void* __restrict__ x, int64_t R, int64_t I,
                                                       void* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= R * I) return;
  const int64_t r = i / I, c = i - r * I;
  const float x1 = Elem<DT>::load(x, r * 2 * I + c);
  const float x3 = Elem<DT>::load(x, r * 2 * I + I + c);
  if constexpr (DT == MODEL_F16) {
    static_cast<uint16_t*>(out)[i] = silu_mul_h(x1, x3);
  } else if constexpr (DT == MODEL_BF16) {
    static_cast<uint16_t*>(out)[i] = silu_mul_bf(x1, x3);  // (shared with the matmul kernels' folded form)
  } else {
    const float silu = Elem<DT>::rnd(x1 / (1.0f + expf(-x1)));
    Elem<DT>::store(out, i, silu * x3);
  }
}

// out[t, h] = sum_j fp16(y[t, j, h] * w[t, j]), fp16 adds left to right
// pos: where slot t * k + j sits among the rows of y (expert-sorted order), or null for y in slot order
template <int DT>
__global__ __launch_bounds__(256) void moe_combine_kernel(const void* __restrict__ y, const void* __restrict__ w,
                                                          const int32_t* __restrict__ pos, int64_t T, int k,
                                                          int64_t H, void* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= T * H) return;
  const int64_t t = i / H, h = i - t * H;
  float acc = 0.f;
  for (int j = 0; j < k; ++j) {
    int64_t row = t * k + j;
    if (pos != nullptr) {
      row = pos[row];
      row = row < 0 ? 0 : (row >= T * k ? T * k - 1 : row);
    }
    const float prod = Elem<DT>::rnd(Elem<DT>::load(y, row * H + h) * Elem<DT>::load(w, t * k + j));
    acc = (j == 0) ? prod : Elem<DT>::rnd(acc + prod);
  }
  Elem<DT>::store(out, i, acc);
}

// The same for 16-bit model dtypes with H a multiple of VEC (4 | 8) and 2 * VEC-byte aligned tensors: a thread owns VEC
// consecutive h of one token, so every access is 8 or 16 bytes (per element the arithmetic above, in the same order).
template <int DT, int VEC>
__global__ __launch_bounds__(256) void moe_combine_vec_kernel(const void* __restrict__ y, const void* __restrict__ w,
                                                              const int32_t* __restrict__ pos, int64_t T, int k,
                                                              int64_t H, void* __restrict__ out) {
  static_assert(DT != MODEL_F32, "16-bit elements");
  struct alignas(2 * VEC) Pack { uint16_t v[VEC]; };
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * VEC;
  if (i >= T * H) return;
  const int64_t t = i / H, h = i - t * H;
  float acc[VEC];
  for (int j = 0; j < k; ++j) {
    int64_t row = t * k + j;
    if (pos != nullptr) {
      row = pos[row];
      row = row < 0 ? 0 : (row >= T * k ? T * k - 1 : row);
    }
    const Pack yv = *reinterpret_cast<const Pack*>(static_cast<const uint16_t*>(y) + row * H + h);
    const float wj = Elem<DT>::load(w, t * k + j);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float ye = DT == MODEL_BF16 ? bf2f(yv.v[e]) : h2f(yv.v[e]);
      const float prod = Elem<DT>::rnd(ye * wj);
      acc[e] = (j == 0) ? prod : Elem<DT>::rnd(acc[e] + prod);
    }
  }
  Pack o;
#pragma unroll
  for (int e = 0; e < VEC; ++e) o.v[e] = k > 0 ? (DT == MODEL_BF16 ? f2bf(acc[e]) : f2h(acc[e])) : uint16_t(0);
  *reinterpret_cast<Pack*>(static_cast<uint16_t*>(out) + i) = o;
}

static inline unsigned blocks_for(int64_t n, int per) { return static_cast<unsigned>((n + per - 1) / per); }

// dispatch on the model dtype: fn(std::integral_constant<int, DT>)
template <typename Fn>
static hipError_t by_dtype(int model_dtype, Fn fn) {
  if (model_dtype == MODEL_F16) fn(std::integral_constant<int, MODEL_F16>{});
  else if (model_dtype == MODEL_F32) fn(std::integral_constant<int, MODEL_F32>{});
  else if (model_dtype == MODEL_BF16) fn(std::integral_constant<int, MODEL_BF16>{});
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launch_topk_softmax(const void* logits, int64_t T, int ne, int k, void* w, int32_t* ids, int model_dtype,
                               hipStream_t s) {
  if (T == 0) return hipSuccess;
  const bool by_wave = use_wave_topk(ne, k);
  return by_dtype(model_dtype, [&](auto dt) {
    if (by_wave)
      hipLaunchKernelGGL(topk_softmax_wave_kernel<decltype(dt)::value>, dim3(blocks_for(T, 4)), dim3(256), 0, s,
                         logits, T, ne, k, w, ids);
    else
      hipLaunchKernelGGL(topk_softmax_kernel<decltype(dt)::value>, dim3(blocks_for(T, 256)), dim3(256), 0, s, logits,
                         T, ne, k, w, ids);
  });
}

hipError_t launch_topk_scores(const void* x, int64_t T, int ne, int k, void* w, int32_t* ids, int model_dtype,
                              bool softmax_first, hipStream_t s) {
  if (T == 0) return hipSuccess;
  return by_dtype(model_dtype, [&](auto dt) {
    if (softmax_first)
      hipLaunchKernelGGL((topk_scores_kernel<decltype(dt)::value, true>), dim3(blocks_for(T, 256)), dim3(256), 0, s, x,
                         T, ne, k, w, ids);
    else
      hipLaunchKernelGGL((topk_scores_kernel<decltype(dt)::value, false>), dim3(blocks_for(T, 256)), dim3(256), 0, s,
                         x, T, ne, k, w, ids);
  });
}

hipError_t launch_moe_cumsum(const int32_t* ids, int64_t T, int k, int ne, int32_t* cumsum,
                             hipStream_t s) {
  if (T == 0 || ne == 0) return hipSuccess;
  hipLaunchKernelGGL(moe_cumsum_kernel, dim3(ne), dim3(1024), 0, s, ids, T, k, ne, cumsum);
  return hipGetLastError();
}

hipError_t launch_get_indices(const int32_t* cumsum, const int32_t* ids, int64_t T, int k, int ne,
                              int32_t* rev, int32_t* tok, hipStream_t s) {
  if (T * k == 0) return hipSuccess;
  hipLaunchKernelGGL(get_indices_kernel, dim3(blocks_for(T * k, 256)), dim3(256), 0, s, cumsum, ids,
                     T, k, ne, rev, tok);
  return hipGetLastError();
}

hipError_t launch_get_indptr(const int32_t* cumsum, int64_t ne, int64_t T, int inclusive,
                             int out_i64, void* indptr, hipStream_t s) {
  const int64_t n = inclusive ? ne : ne + 1;
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(get_indptr_kernel, dim3(blocks_for(n, 64)), dim3(64), 0, s, cumsum, ne, T,
                     inclusive, out_i64, indptr);
  return hipGetLastError();
}

hipError_t launch_take_rows(const uint16_t* x, const int32_t* idx, int64_t R, int64_t H,
                            int64_t x_rows, uint16_t* out, int scatter, hipStream_t s) {
  if (R * H == 0) return hipSuccess;
  const bool vec = (H % 8 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0) &&
                   ((reinterpret_cast<uintptr_t>(out) & 15) == 0);
  if (vec)
    hipLaunchKernelGGL(move_rows_kernel<8>, dim3(blocks_for(R * (H / 8), 256)), dim3(256), 0, s, x,
                       idx, R, H, x_rows, scatter, out);
  else
    hipLaunchKernelGGL(move_rows_kernel<1>, dim3(blocks_for(R * H, 256)), dim3(256), 0, s, x, idx,
                       R, H, x_rows, scatter, out);
  return hipGetLastError();
}

hipError_t launch_silu_mul(const void* x, int64_t R, int64_t I, void* out, int model_dtype, hipStream_t s) {
  if (R * I == 0) return hipSuccess;
  return by_dtype(model_dtype, [&](auto dt) {
    hipLaunchKernelGGL(silu_mul_kernel<decltype(dt)::value>, dim3(blocks_for(R * I, 256)), dim3(256), 0, s, x, R, I,
                       out);
  });
}

hipError_t launch_moe_combine(const void* y, const void* w, const int32_t* pos, int64_t T, int k, int64_t H,
                              void* out, int model_dtype, hipStream_t s) {
  if (T * H == 0) return hipSuccess;
  const uintptr_t addr = reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(out);
  if (model_dtype != MODEL_F32 && H % 4 == 0 && addr % 8 == 0) {
    // 16 bytes per access once that still leaves a workgroup per CU, 8 below
    const bool wide = H % 8 == 0 && addr % 16 == 0 && T * H >= 8 * 256 * 256;
    auto go = [&](auto dt, auto vec) {
      hipLaunchKernelGGL((moe_combine_vec_kernel<decltype(dt)::value, decltype(vec)::value>),
                         dim3(blocks_for(T * H, 256 * decltype(vec)::value)), dim3(256), 0, s, y, w, pos, T, k, H, out);
    };
    if (model_dtype == MODEL_F16) {
      if (wide) go(std::integral_constant<int, MODEL_F16>{}, std::integral_constant<int, 8>{});
      else go(std::integral_constant<int, MODEL_F16>{}, std::integral_constant<int, 4>{});
    } else if (model_dtype == MODEL_BF16) {
      if (wide) go(std::integral_constant<int, MODEL_BF16>{}, std::integral_constant<int, 8>{});
      else go(std::integral_constant<int, MODEL_BF16>{}, std::integral_constant<int, 4>{});
    } else {
      return hipErrorInvalidValue;
    }
    return hipGetLastError();
  }
  return by_dtype(model_dtype, [&](auto dt) {
    hipLaunchKernelGGL(moe_combine_kernel<decltype(dt)::value>, dim3(blocks_for(T * H, 256)), dim3(256), 0, s, y, w,
                       pos, T, k, H, out);
  });
}

// the slot-organised route kernel: 8 slots per thread, [experts, 64-slot chunks] counts in 32 KiB of LDS
bool moe_route_by_slot(int64_t T, int ne, int k) {
  const int64_t slots = T * k;
  return slots <= 8 * 1024 && ne <= 256 && static_cast<int64_t>(ne) * ((slots + 63) / 64) <= 8 * 1024;
}

hipError_t launch_moe_route(const void* logits, int64_t T, int ne, int k, void* w, int32_t* ids, int32_t* tok,
                            int32_t* rev, int32_t* pos_of_slot, int out_i64, void* indptr, int model_dtype,
                            hipStream_t s) {
  const int64_t slots = T * k;
  if (moe_route_by_slot(T, ne, k) && slots > 0) {
    // by slot; with many experts the top-k runs one wave per token, inside the kernel while one
    // workgroup is a single token's wave, as a launch of its own across the chip beyond that (never slower: T=16
    // 25.5 -> 18.0 us with 128 experts, and a route step of one or two waves instead of one per token)
    const bool by_wave = use_wave_topk(ne, k);
    const bool topk_first = by_wave && T > 1;
    if (topk_first) {
      const hipError_t err = launch_topk_softmax(logits, T, ne, k, w, ids, model_dtype, s);
      if (err != hipSuccess) return err;
    }
    int threads = static_cast<int>((slots + 63) / 64) * 64;
    if (by_wave && !topk_first && threads < 64 * T) threads = static_cast<int>(64 * T);
    threads = threads > 1024 ? 1024 : threads;
    const size_t lds = static_cast<size_t>(ne) * ((slots + 63) / 64) * sizeof(int32_t);
    return by_dtype(model_dtype, [&](auto dt) {
      hipLaunchKernelGGL(moe_route_slots_kernel<decltype(dt)::value>, dim3(1), dim3(threads), lds, s, logits,
                         static_cast<int>(T), ne, k,
                         (out_i64 ? 1 : 0) | (topk_first ? 0 : 2) | (by_wave ? 4 : 0) | (threads >> 6) << 8, w, ids, tok,
                         rev, pos_of_slot, indptr);
    });
  }
  int threads = static_cast<int>((T + 63) / 64) * 64;
  threads = threads < 64 ? 64 : (threads > 1024 ? 1024 : threads);
  const size_t lds = static_cast<size_t>(T) * k * sizeof(int32_t);
  const int ids_in_lds = lds <= 60 * 1024;
  return by_dtype(model_dtype, [&](auto dt) {
    hipLaunchKernelGGL(moe_route_kernel<decltype(dt)::value>, dim3(1), dim3(threads), ids_in_lds ? lds : 0, s, logits,
                       static_cast<int>(T), ne, k, w, ids, tok, rev, pos_of_slot, out_i64, indptr, ids_in_lds);
  });
}

}  // namespace gq
