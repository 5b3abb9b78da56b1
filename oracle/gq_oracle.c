/*
 * CPU oracle (plain C) for MLC-LLM's group-quantized linear path.
 *
 * TEST INFRASTRUCTURE ONLY: linked by nothing that ships.  tests/, the smoke
 * check and the benchmark's cpu_baseline leg load it through ctypes to check
 * (and to time, as a CPU baseline) the same arithmetic the HIP kernels do.
 *
 * Restates, from the reference checkout:
 *   python/mlc_llm/quantization/group_quantization.py:235-306  _quantize
 *   python/mlc_llm/quantization/group_quantization.py:155-186  _dequantize
 *   python/mlc_llm/quantization/utils.py:15-48                 convert_uint_to_float
 *   python/mlc_llm/quantization/utils.py:136-188               pack_weight
 *   python/mlc_llm/compiler_pass/fuse_transpose_matmul.py:64-129 NT_matmul (loop nest of
 *       fused_dequantize_NT_matmul: parallel over N, inner K, inline dequantize)
 *   python/mlc_llm/op/moe_matmul.py:632-722                    dequantize_group_gemm
 *
 * PARITY UNPINNED (depends on TVM's lowering, which the checkout does not hold):
 * the tie rule of round() in _quantize (round_mode 0 = half away from zero, the
 * llvm/rocm lowering; 1 = half to even) and the code emitted for an all-zero
 * group (0/0 -> NaN -> compare+select max -> 0).  The rounding points themselves
 * (fp16 divide, fp16 add, then round) are pinned: tests/ compares the codes with
 * exact integer arithmetic on a million values.
 *
 * fp16 values travel as uint16_t bit patterns.  Each fp16 operation is done in
 * float and rounded to nearest-even half straight away; for + - * / that equals
 * the correctly rounded fp16 result (24 >= 2*11+2 significand bits).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#if defined(__AVX2__) && defined(__F16C__) && defined(__FMA__)
#include <immintrin.h>
#define GQO_AVX2 1
#endif

static inline float h2f(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        e++;
      } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* float -> half, round to nearest even, IEEE overflow to inf, subnormals kept */
static inline uint16_t f2h(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) return (uint16_t)(sign | (ax > 0x7f800000u ? 0x7e00u : 0x7c00u));
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
  if (ax < 0x33000001u) return sign;                          /* <= 2^-25 rounds to 0  */
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t man = (ax & 0x7fffffu) | 0x800000u;
  int shift = (e < -14) ? (13 + (-14 - e)) : 13;
  uint32_t half_man = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
  uint32_t out;
  if (e < -14) {
    out = half_man; /* subnormal; a carry into bit 10 lands on the smallest normal */
  } else {
    out = ((uint32_t)(e + 15) << 10) + (half_man - 0x400u); /* mantissa carry bumps exponent */
  }
  return (uint16_t)(sign | out);
}

int gqo_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

uint16_t gqo_f2h(float f) { return f2h(f); }
float gqo_h2f(uint16_t h) { return h2f(h); }

/* group_quantization.py:235-306, NK layout, axis = last.
 * w [rows, K] fp16; q_weight [rows, nw] uint32; q_scale [rows, ng] fp16. */
int gqo_quantize(const uint16_t* w, int64_t rows, int64_t K, int bits, int group_size,
                 int round_mode, uint32_t* q_weight, uint16_t* q_scale) {
  if (bits != 3 && bits != 4) return -1;
  const int E = 32 / bits;
  if (group_size % E) return -1;
  const int S = group_size / E;
  const int m = (1 << (bits - 1)) - 1;
  const int64_t ng = (K + group_size - 1) / group_size;
  const int64_t nw = S * ng;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < rows; ++n) {
    const uint16_t* wr = w + n * K;
    uint32_t* qr = q_weight + n * nw;
    memset(qr, 0, (size_t)nw * 4);
    for (int64_t g = 0; g < ng; ++g) {
      int64_t k0 = g * group_size;
      int64_t k1 = k0 + group_size < K ? k0 + group_size : K;
      /* :250-267 max of |w|; |x| on the bit pattern orders like the value for non-NaN */
      float mx = -65504.0f;
      for (int64_t k = k0; k < k1; ++k) {
        float a = fabsf(h2f(wr[k]));
        if (a > mx) mx = a;
      }
      uint16_t sh = f2h(mx / (float)m); /* :268-272 */
      q_scale[n * ng + g] = sh;
      float s = h2f(sh);
      for (int64_t k = k0; k < k1; ++k) {
        float t = h2f(f2h(h2f(wr[k]) / s));      /* :279-280 fp16 divide */
        t = h2f(f2h(t + (float)m));               /* :281 fp16 add       */
        float r = round_mode == 0 ? roundf(t) : nearbyintf(t); /* :278 */
        r = (r > 0.0f) ? r : 0.0f;                /* select(a > b, a, b): NaN -> 0 */
        r = (r < (float)(2 * m)) ? r : (float)(2 * m);
        uint32_t q = (uint32_t)r;
        qr[k / E] += q << ((k % E) * bits);       /* utils.py:174-187 */
      }
    }
  }
  return 0;
}

/* group_quantization.py:176-185 with utils.py:31-47; out [rows, K] fp16 */
int gqo_dequantize(const uint32_t* q_weight, const uint16_t* q_scale, int64_t rows, int64_t K,
                   int bits, int group_size, uint16_t* out) {
  if (bits != 3 && bits != 4) return -1;
  const int E = 32 / bits;
  const int S = group_size / E;
  const int m = (1 << (bits - 1)) - 1;
  const uint32_t mask = (1u << bits) - 1u;
  const int64_t ng = (K + group_size - 1) / group_size;
  const int64_t nw = S * ng;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < rows; ++n) {
    for (int64_t k = 0; k < K; ++k) {
      uint32_t u = (q_weight[n * nw + k / E] >> ((k % E) * bits)) & mask;
      float d = (float)u - (float)m; /* exact in fp16 */
      out[n * K + k] = f2h(d * h2f(q_scale[n * ng + k / group_size]));
    }
  }
  return 0;
}

/* One output row of fused_dequantize_NT_matmul for M activation rows (xf = x as float).
 * fp16 dequantised weight (rounded as the reference rounds it), fp32 accumulation. */
static void row_dot(const uint32_t* qr, const uint16_t* sr, const float* xf, int64_t M, int64_t K,
                    int bits, int group_size, float* acc /* [M] */) {
  const int E = 32 / bits;
  const int m = (1 << (bits - 1)) - 1;
  const uint32_t mask = (1u << bits) - 1u;
  for (int64_t i = 0; i < M; ++i) acc[i] = 0.0f;
#ifdef GQO_AVX2
  if (bits == 4 && group_size % 8 == 0 && K % 8 == 0) {
    const __m256i shifts = _mm256_setr_epi32(0, 4, 8, 12, 16, 20, 24, 28);
    const __m256i vmask = _mm256_set1_epi32(15);
    const __m256 vm = _mm256_set1_ps(7.0f);
    for (int64_t i = 0; i < M; ++i) {
      __m256 a = _mm256_setzero_ps();
      const float* xr = xf + i * K;
      for (int64_t wd = 0; wd < K / 8; ++wd) {
        __m256 s = _mm256_set1_ps(h2f(sr[(wd * 8) / group_size]));
        __m256i u = _mm256_and_si256(_mm256_srlv_epi32(_mm256_set1_epi32((int)qr[wd]), shifts), vmask);
        __m256 d = _mm256_mul_ps(_mm256_sub_ps(_mm256_cvtepi32_ps(u), vm), s);
        d = _mm256_cvtph_ps(_mm256_cvtps_ph(d, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
        a = _mm256_fmadd_ps(d, _mm256_loadu_ps(xr + wd * 8), a);
      }
      __m128 lo = _mm_add_ps(_mm256_castps256_ps128(a), _mm256_extractf128_ps(a, 1));
      lo = _mm_add_ps(lo, _mm_movehl_ps(lo, lo));
      lo = _mm_add_ss(lo, _mm_shuffle_ps(lo, lo, 1));
      acc[i] = _mm_cvtss_f32(lo);
    }
    return;
  }
#endif
  for (int64_t k = 0; k < K; ++k) {
    uint32_t u = (qr[k / E] >> ((k % E) * bits)) & mask;
    float wv = h2f(f2h(((float)u - (float)m) * h2f(sr[k / group_size])));
    for (int64_t i = 0; i < M; ++i) acc[i] += xf[i * K + k] * wv;
  }
}

/* y[M, N] (float) = x[M, K] (fp16) . dequant(W)[N, K]^T (+ bias fp16 [N] if non-null).
 * Parallel over N like the reference's CPU GEMV schedule. scratch_xf: caller-owned [M*K] floats. */
int gqo_linear(const uint16_t* x, const uint32_t* q_weight, const uint16_t* q_scale,
               const uint16_t* bias, int64_t M, int64_t N, int64_t K, int bits, int group_size,
               float* scratch_xf, float* y) {
  if (bits != 3 && bits != 4) return -1;
  if (M > 64) return -2;
  const int E = 32 / bits;
  const int64_t ng = (K + group_size - 1) / group_size;
  const int64_t nw = (group_size / E) * ng;
  for (int64_t i = 0; i < M * K; ++i) scratch_xf[i] = h2f(x[i]);
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    float acc[64];
    row_dot(q_weight + n * nw, q_scale + n * ng, scratch_xf, M, K, bits, group_size, acc);
    float b = bias ? h2f(bias[n]) : 0.0f;
    for (int64_t i = 0; i < M; ++i) y[i * N + n] = acc[i] + b;
  }
  return 0;
}

/* moe_matmul.py:632-722: rows indptr[e]..indptr[e+1] of x meet expert e.  y float [rows, N]. */
int gqo_group_gemm(const uint16_t* x, const uint32_t* q_weight, const uint16_t* q_scale,
                   const int32_t* indptr, int64_t num_experts, int64_t N, int64_t K, int bits,
                   int group_size, float* scratch_xf, float* y) {
  if (bits != 3 && bits != 4) return -1;
  const int E = 32 / bits;
  const int64_t ng = (K + group_size - 1) / group_size;
  const int64_t nw = (group_size / E) * ng;
  const int64_t rows = indptr[num_experts];
  for (int64_t i = 0; i < rows * K; ++i) scratch_xf[i] = h2f(x[i]);
  for (int64_t e = 0; e < num_experts; ++e) {
    int64_t lo = indptr[e], hi = indptr[e + 1];
    if (hi <= lo) continue;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
      for (int64_t r0 = lo; r0 < hi; r0 += 64) {
        int64_t mm = hi - r0 < 64 ? hi - r0 : 64;
        float acc[64];
        row_dot(q_weight + (e * N + n) * nw, q_scale + (e * N + n) * ng, scratch_xf + r0 * K, mm,
                K, bits, group_size, acc);
        for (int64_t i = 0; i < mm; ++i) y[(r0 + i) * N + n] = acc[i];
      }
    }
  }
  return 0;
}
