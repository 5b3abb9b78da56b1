// Routing glue of the MoE layer: top-k + softmax, expert-major cumsum, gather/scatter plans,
// indptr, row gather/scatter, silu*mul and the weighted top-k combine.
//
// Replaces the TIR of python/mlc_llm/op/moe_misc.py in the reference: gating_softmax_topk
// (:135-235), moe_cumsum (:371-450), get_indices (:453-525), get_indptr (:528-605),
// scatter_output (:608-645), moe_sum (:14-32), and the elementwise glue of
// model/mixtral/mixtral_model.py:64-117.  All of it is integer / tiny fp16 work.
#include "gq_common.hpp"
#include "gq_internal.hpp"

namespace gq {

constexpr int kMaxTopK = 8;

// One thread per token: insertion top-k with strict '>' (ties keep the lower expert index),
// then softmax over the k selected logits in fp32.
__global__ __launch_bounds__(256) void topk_softmax_kernel(const uint16_t* __restrict__ logits,
                                                           int64_t T, int ne, int k,
                                                           uint16_t* __restrict__ w,
                                                           int32_t* __restrict__ ids) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (t >= T) return;
  float val[kMaxTopK];
  int idx[kMaxTopK];
#pragma unroll
  for (int i = 0; i < kMaxTopK; ++i) {
    val[i] = -65504.0f;  // min_value(fp16)
    idx[i] = 0;
  }
  const uint16_t* row = logits + t * ne;
  for (int e = 0; e < ne; ++e) {
    const float v = h2f(row[e]);
    bool placed = false;
#pragma unroll
    for (int i = 0; i < kMaxTopK; ++i) {
      if (i < k && !placed && v > val[i]) {
#pragma unroll
        for (int j = kMaxTopK - 1; j > 0; --j) {
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
  float mx = val[0];
#pragma unroll
  for (int i = 1; i < kMaxTopK; ++i)
    if (i < k) mx = fmaxf(mx, val[i]);
  float ex[kMaxTopK];
  float den = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxTopK; ++i) {
    if (i < k) {
      ex[i] = expf(val[i] - mx);
      den = (i == 0) ? ex[0] : den + ex[i];
    }
  }
#pragma unroll
  for (int i = 0; i < kMaxTopK; ++i) {
    if (i < k) {
      w[t * k + i] = f2h(ex[i] / den);
      ids[t * k + i] = idx[i];
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
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t* __restrict__ x, int64_t R,
                                                       int64_t I, uint16_t* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= R * I) return;
  const int64_t r = i / I, c = i - r * I;
  const float x1 = h2f(x[r * 2 * I + c]);
  const float x3 = h2f(x[r * 2 * I + I + c]);
  out[i] = silu_mul_h(x1, x3);
}

// out[t, h] = sum_j fp16(y[t, j, h] * w[t, j]), fp16 adds left to right
__global__ __launch_bounds__(256) void moe_combine_kernel(const uint16_t* __restrict__ y,
                                                          const uint16_t* __restrict__ w,
                                                          int64_t T, int k, int64_t H,
                                                          uint16_t* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= T * H) return;
  const int64_t t = i / H, h = i - t * H;
  float acc = 0.f;
  for (int j = 0; j < k; ++j) {
    const float prod = h2f(f2h(h2f(y[(t * k + j) * H + h]) * h2f(w[t * k + j])));
    acc = (j == 0) ? prod : h2f(f2h(acc + prod));
  }
  out[i] = f2h(acc);
}

static inline unsigned blocks_for(int64_t n, int per) { return static_cast<unsigned>((n + per - 1) / per); }

hipError_t launch_topk_softmax(const uint16_t* logits, int64_t T, int ne, int k, uint16_t* w,
                               int32_t* ids, hipStream_t s) {
  if (T == 0) return hipSuccess;
  hipLaunchKernelGGL(topk_softmax_kernel, dim3(blocks_for(T, 256)), dim3(256), 0, s, logits, T, ne,
                     k, w, ids);
  return hipGetLastError();
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

hipError_t launch_silu_mul(const uint16_t* x, int64_t R, int64_t I, uint16_t* out, hipStream_t s) {
  if (R * I == 0) return hipSuccess;
  hipLaunchKernelGGL(silu_mul_kernel, dim3(blocks_for(R * I, 256)), dim3(256), 0, s, x, R, I, out);
  return hipGetLastError();
}

hipError_t launch_moe_combine(const uint16_t* y, const uint16_t* w, int64_t T, int k, int64_t H,
                              uint16_t* out, hipStream_t s) {
  if (T * H == 0) return hipSuccess;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(blocks_for(T * H, 256)), dim3(256), 0, s, y, w, T, k,
                     H, out);
  return hipGetLastError();
}

}  // namespace gq
