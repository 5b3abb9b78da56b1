// Decode GEMV: y[b, n] = sum_k x[b, k] * dequant(W)[n, k], batch 1..8, q4f16_1 and q3f16_1.
//
// Replaces the TVM-generated fused_dequantize*_NT_matmul kernels that GroupQuantizeLinear.forward
// lowers to for M <= 8 (python/mlc_llm/quantization/group_quantization.py:390-437,
// compiler_pass/low_batch_specialization.py:22-57) and moe_matmul.dequantize_gemv
// (python/mlc_llm/op/moe_matmul.py:147-176) through the expert_ids indirection.
//
// HBM-bound: the only large stream is q_weight (K/2 bytes per row for 4 bit).  Mapping:
//  * one 128-bit load per lane = 4 storage words = exactly one quantisation group (both schemes),
//    so one fp16 scale belongs to each load; a wave covers 64 consecutive groups of a row (1 KiB,
//    fully coalesced) and R rows at a time to keep R loads per lane in flight;
//  * fields are turned into halves without shifts or converts by OR-ing them into the mantissa
//    of 1024.0 (0x6400): (w & 0x000f000f) | 0x64006400 is the half pair (1024+q0, 1024+q4).
//    Fields that sit higher in the mantissa come out multiplied by 16 (q4) or 8/64 (q3); they
//    accumulate in their own v_dot2_f32_f16 chain and are rescaled once per group in fp32;
//  * the "1024 + offset" terms are removed with one fp32 subtraction per group:
//    sum_k x_k (1024 + q_k) - corr, corr precomputed per (batch row, group) while x is staged;
//  * x is staged once per block in LDS, already permuted into the pair order the masks produce
//    and laid out [chunk][group] so that consecutive lanes read consecutive 16-byte chunks
//    (conflict-free ds_read_b128); values beyond K are staged as 0, which also neutralises the
//    zero padding fields of the last q3 group;
//  * the per-row sum over lanes is a DPP/bpermute wave reduction.
#include "gq_gemv_common.hpp"

namespace gq {

// Stage groups [gbase, gbase + gcount) of NB activation rows into LDS (permuted) + corr terms.
template <int BITS, int NB>
__device__ __forceinline__ void stage_x(const uint16_t* __restrict__ x, int K, int gbase,
                                        int gcount, int gc, uint4* xs, float* corr) {
  using T = GemvTraits<BITS>;
  constexpr int E = Scheme<BITS>::kElem;
  const int items = NB * gcount * 4;
  for (int it = threadIdx.x; it < ((items + 3) & ~3); it += 256) {
    const bool live = it < items;
    const int itc = live ? it : items - 1;
    const int word = itc & 3;
    const int gl = (itc >> 2) % gcount;
    const int b = (itc >> 2) / gcount;
    const int k0 = (gbase + gl) * T::G + word * E;
    const uint16_t* xr = x + static_cast<int64_t>(b) * K;
    uint16_t v[E];
    if (BITS == 4 && k0 + E <= K && (K & 7) == 0) {
      const uint4 raw = *reinterpret_cast<const uint4*>(xr + k0);
      v[0] = raw.x & 0xffffu; v[1] = raw.x >> 16; v[2] = raw.y & 0xffffu; v[3] = raw.y >> 16;
      v[4] = raw.z & 0xffffu; v[5] = raw.z >> 16; v[6] = raw.w & 0xffffu; v[7] = raw.w >> 16;
    } else if (BITS == 3 && k0 + E <= K && (K & 1) == 0) {
      const uint32_t* p = reinterpret_cast<const uint32_t*>(xr + k0);
#pragma unroll
      for (int i = 0; i < E / 2; ++i) {
        const uint32_t r = p[i];
        v[2 * i] = r & 0xffffu;
        v[2 * i + 1] = r >> 16;
      }
    } else {
#pragma unroll
      for (int i = 0; i < E; ++i) v[i] = (k0 + i < K) ? xr[k0 + i] : uint16_t(0);
    }
    float c;
    if (BITS == 4) {
      // pairs (0,4) (1,5) (2,6) (3,7); odd fields come out of the mask multiplied by 16
      uint4 pk;
      pk.x = v[0] | (static_cast<uint32_t>(v[4]) << 16);
      pk.y = v[1] | (static_cast<uint32_t>(v[5]) << 16);
      pk.z = v[2] | (static_cast<uint32_t>(v[6]) << 16);
      pk.w = v[3] | (static_cast<uint32_t>(v[7]) << 16);
      if (live) xs[(b * T::CH + word) * gc + gl] = pk;
      const float lo = h2f(v[0]) + h2f(v[4]) + h2f(v[2]) + h2f(v[6]);
      const float hi = h2f(v[1]) + h2f(v[5]) + h2f(v[3]) + h2f(v[7]);
      c = 1031.0f * lo + 71.0f * hi;  // (1024 + 7) and (1024/16 + 7)
    } else {
      // pairs (j, j+5); pair j sits at mantissa bit 3*(j mod 3): scale 1, 8, 64, 1, 8
      uint32_t* xw = reinterpret_cast<uint32_t*>(xs);
      float s1 = 0.f, s8 = 0.f, s64 = 0.f;
#pragma unroll
      for (int j = 0; j < 5; ++j) {
        const int h = word * 5 + j;
        const uint32_t pk = v[j] | (static_cast<uint32_t>(v[j + 5]) << 16);
        if (live) xw[((b * T::CH + (h >> 2)) * gc + gl) * 4 + (h & 3)] = pk;
        const float sum = h2f(v[j]) + h2f(v[j + 5]);
        if (j == 0 || j == 3) s1 += sum;
        else if (j == 1 || j == 4) s8 += sum;
        else s64 += sum;
      }
      c = 1027.0f * s1 + 131.0f * s8 + 19.0f * s64;  // 1024/c + 3
    }
    c += dpp_f<0xB1>(c);
    c += dpp_f<0x4E>(c);
    if (live && word == 0) corr[b * gc + gl] = c;
  }
}

template <int BITS, int NB, int R>
__global__ __launch_bounds__(256) void gemv_dot2_kernel(const GemvParams p) {
  using T = GemvTraits<BITS>;
  extern __shared__ uint4 smem[];
  uint4* xs = smem;
  float* corr = reinterpret_cast<float*>(smem + NB * T::CH * p.gc);

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int slot = blockIdx.y;
  const int row0 = (blockIdx.x * 4 + wave) * R;

  const uint16_t* x = p.x + slot * p.x_slot_stride;
  const uint32_t* qw = p.qw;
  const uint16_t* qs = p.qs;
  if (p.expert_ids != nullptr) {
    int e = p.expert_ids[slot];
    e = e < 0 ? 0 : (e >= p.num_experts ? p.num_experts - 1 : e);
    qw += e * p.expert_w_stride;
    qs += e * p.expert_s_stride;
  }
  const uint32_t* wrow[R];
  const uint16_t* srow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int row = min(row0 + r, p.N - 1);  // clamped rows are computed and dropped
    wrow[r] = qw + static_cast<int64_t>(row) * p.nw;
    srow[r] = qs + static_cast<int64_t>(row) * p.ng;
  }

  float acc[R][NB];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[r][b] = 0.f;

  // depth-1 software pipeline over (chunk, group): the weights of the next group are in flight
  // while x is staged / the current group is computed
  uint4 wn[R];
  uint16_t sn[R];
  bool have_next = lane < p.ng;
  if (have_next) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      wn[r] = *reinterpret_cast<const uint4*>(wrow[r] + 4 * lane);
      sn[r] = srow[r][lane];
    }
  }

  for (int gbase = 0; gbase < p.ng; gbase += p.gc) {
    const int gcount = min(p.gc, p.ng - gbase);
    if (gbase > 0) __syncthreads();
    stage_x<BITS, NB>(x, p.K, gbase, gcount, p.gc, xs, corr);
    __syncthreads();
    for (int gl = lane; gl < gcount; gl += 64) {
      uint4 wc[R];
      float sc[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        wc[r] = wn[r];
        sc[r] = h2f(sn[r]);
      }
      // next group of this lane: same chunk, or the first one of the next chunk
      int gnext = gbase + gl + 64;
      if (gl + 64 >= gcount) gnext = gbase + p.gc + lane;
      if (gnext < p.ng) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          wn[r] = *reinterpret_cast<const uint4*>(wrow[r] + 4 * static_cast<int64_t>(gnext));
          sn[r] = srow[r][gnext];
        }
      }
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        uint32_t xr[T::CH * 4];
#pragma unroll
        for (int c = 0; c < T::CH; ++c) {
          const uint4 v = xs[(b * T::CH + c) * p.gc + gl];
          xr[4 * c + 0] = v.x; xr[4 * c + 1] = v.y; xr[4 * c + 2] = v.z; xr[4 * c + 3] = v.w;
        }
        const float cr = corr[b * p.gc + gl];
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r][b] = fmaf(sc[r], group_dot<BITS>(wc[r], xr, cr), acc[r][b]);
      }
    }
  }

#pragma unroll
  for (int r = 0; r < R; ++r) {
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const float v = wave_sum(acc[r][b]);
      const int row = row0 + r;
      if (lane == 0 && row < p.N) {
        const int64_t oi = static_cast<int64_t>(slot + b) * p.N + row;  // slot > 0 only when NB == 1
        const float o = v + (p.bias ? h2f(p.bias[row]) : 0.f) + (p.residual ? h2f(p.residual[oi]) : 0.f);
        if (p.out_f32) static_cast<float*>(p.y)[oi] = o;
        else static_cast<uint16_t*>(p.y)[oi] = f2h(o);
      }
    }
  }
}

template <int BITS, int NB, int R>
static hipError_t launch_one(const GemvParams& p, int slots, hipStream_t s) {
  using T = GemvTraits<BITS>;
  const size_t lds = static_cast<size_t>(NB) * p.gc * (T::CH * 16 + 4);
  const dim3 grid((p.N + 4 * R - 1) / (4 * R), slots);
  note_kernel("gq::gemv_dot2_kernel<%d,%d,%d>", BITS, NB, R);
  hipLaunchKernelGGL((gemv_dot2_kernel<BITS, NB, R>), grid, dim3(256), lds, s, p);
  return hipGetLastError();
}

template <int BITS, int NB>
static hipError_t launch_r(const GemvParams& p, int slots, int R, hipStream_t s) {
  switch (R) {
    case 1: return launch_one<BITS, NB, 1>(p, slots, s);
    case 2: return launch_one<BITS, NB, 2>(p, slots, s);
    default: return launch_one<BITS, NB, 4>(p, slots, s);
  }
}

template <int BITS>
static hipError_t launch_nb(const GemvParams& p, int slots, int nb, int R, hipStream_t s) {
  switch (nb) {
    case 1: return launch_r<BITS, 1>(p, slots, R, s);
    case 2: return launch_r<BITS, 2>(p, slots, R, s);
    case 3: return launch_r<BITS, 3>(p, slots, R, s);
    case 4: return launch_r<BITS, 4>(p, slots, R, s);
    case 5: return launch_r<BITS, 5>(p, slots, R, s);
    case 6: return launch_r<BITS, 6>(p, slots, R, s);
    case 7: return launch_r<BITS, 7>(p, slots, R, s);
    default: return launch_r<BITS, 8>(p, slots, R, s);
  }
}

hipError_t launch_gemv_lds(const GemvParams& p_in, int bits, int nb, int slots, hipStream_t s) {
  GemvParams p = p_in;
  const int ch = bits == 4 ? 4 : 5;
  // LDS chunk: whole K if it fits 64 KiB, else the largest multiple of 64 groups that does
  int gc = (p.ng + 63) & ~63;
  const int cap = (65536 / (nb * (ch * 16 + 4))) & ~63;
  if (gc > cap) gc = cap < 64 ? 64 : cap;
  p.gc = gc;
  int R = options().gemv_rows_per_wave;
  if (R != 1 && R != 2 && R != 4) {
    // enough waves to cover the 256 CUs a few times over, else fewer rows per wave
    const int64_t waves4 = (static_cast<int64_t>(p.N) + 3) / 4 * slots;
    R = waves4 >= 4096 ? 4 : (waves4 >= 1024 ? 2 : 1);
    if (nb > 4 && R > 2) R = 2;  // register budget
  }
  if (bits == 4) return launch_nb<4>(p, slots, nb, R, s);
  return launch_nb<3>(p, slots, nb, R, s);
}

hipError_t launch_gemv(const GemvArgs& a, hipStream_t s) {
  GemvParams p;
  p.x = a.x; p.qw = a.q_weight; p.qs = a.q_scale; p.bias = a.bias; p.residual = a.residual; p.y = a.y;
  p.expert_ids = a.expert_ids;
  p.x_slot_stride = a.x_slot_stride;
  p.N = static_cast<int>(a.N); p.K = static_cast<int>(a.K);
  p.ng = static_cast<int>((a.K + a.group_size - 1) / a.group_size);
  p.nw = 4 * p.ng;
  p.expert_w_stride = a.N * p.nw;
  p.expert_s_stride = a.N * p.ng;
  p.num_experts = static_cast<int>(a.num_experts);
  p.out_f32 = a.out_f32;
  p.gc = 0;
  p.paired = a.paired;
  p.bf16 = a.bf16;
  p.indptr = a.indptr; p.indptr_i64 = a.indptr_i64; p.x_row_index = a.x_row_index;
  p.x_src_rows = static_cast<int>(a.x_src_rows);
  p.routed = a.gate != nullptr;
  if (p.routed) {  // (see GemvParams: three fields carry the router's tensors in this form)
    if (a.bias != nullptr || a.residual != nullptr || a.expert_ids != nullptr) return hipErrorNotSupported;
    p.bias = static_cast<const uint16_t*>(a.gate);
    p.residual = static_cast<const uint16_t*>(a.route_w);
    p.expert_ids = a.route_ids;
  }
  if (a.sum_weights != nullptr) {
    if (p.routed || a.bias != nullptr || a.residual != nullptr || a.expert_ids == nullptr || a.slots != 2 || a.M != 1 ||
        a.paired || a.out_f32 || a.indptr != nullptr)
      return hipErrorNotSupported;
    p.sum2 = 1;
    p.residual = static_cast<const uint16_t*>(a.sum_weights);
  }
  if (a.N == 0 || a.slots == 0) return hipSuccess;
  const int nb = static_cast<int>(a.M);
  const int slots = static_cast<int>(a.slots);
  const int variant = options().gemv_variant;  // -1 auto, 0 LDS-staged kernel, 1 register kernel
  if (variant != 0) {
    const hipError_t e = launch_gemv_reg(p, a.bits, nb, slots, s);
    if (e != hipErrorNotSupported) return e;
  }
  if (p.paired || p.bf16 || p.indptr != nullptr || p.routed || p.sum2) return hipErrorNotSupported;  // only the register kernel has these forms
  return launch_gemv_lds(p, a.bits, nb, slots, s);
}

}  // namespace gq
