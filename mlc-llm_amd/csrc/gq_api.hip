// C ABI of libmi355gq.so: argument validation, error reporting, dispatch to the launchers.
// Declarations (with the reference interface each entry replaces) live in include/mi355gq.h.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <atomic>
#include <cstring>

#include "../../include/mi355gq.h"
#include "gq_internal.hpp"
#include "gq_testing.h"

namespace gq {
Options& options() {
  thread_local Options o;
  return o;
}

static thread_local char g_last_kernel[160] = "";

void note_kernel(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_kernel, sizeof(g_last_kernel), fmt, ap);
  va_end(ap);
}

// Raises a kernel's dynamic-LDS limit to the CU's 160 KiB, once per (kernel, device).  Called on every launch that
// wants more than 64 KiB, from any thread: a lock-free table (open addressing on the kernel's address, a device bit mask
// per entry) answers the repeat calls with two atomic loads.  A race on a new entry at worst sets the attribute twice.
hipError_t allow_large_lds(const void* kernel) {
  constexpr int kSlots = 1024;  // a few dozen instantiations exist
  static std::atomic<const void*> keys[kSlots];
  static std::atomic<uint64_t> masks[kSlots];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  int slot = -1;
  if (dev >= 0 && dev < 64) {
    unsigned h = static_cast<unsigned>((reinterpret_cast<uintptr_t>(kernel) >> 4) * 2654435761u) % kSlots;
    for (int probe = 0; probe < kSlots; ++probe, h = (h + 1) % kSlots) {
      const void* k = keys[h].load(std::memory_order_acquire);
      if (k == nullptr) {
        const void* expected = nullptr;
        if (keys[h].compare_exchange_strong(expected, kernel, std::memory_order_acq_rel)) k = kernel;
        else k = expected;
      }
      if (k == kernel) {
        slot = static_cast<int>(h);
        break;
      }
    }
    if (slot >= 0 && (masks[slot].load(std::memory_order_acquire) >> dev) & 1u) return hipSuccess;
  }
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  if (e == hipSuccess && slot >= 0) masks[slot].fetch_or(uint64_t(1) << dev, std::memory_order_release);
  return e;
}
}  // namespace gq

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int hip_result(hipError_t e, const char* what) {
  if (e == hipSuccess) return MI355GQ_OK;
  return fail(MI355GQ_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }
bool aligned2(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 1u) == 0; }

// q4f16_1-like (bits 4, G = 32) and q3f16_1-like (bits 3, G = 40): a group is 4 storage words
int check_scheme(int bits, int group_size) {
  if (bits != 4 && bits != 3)
    return fail(MI355GQ_ERR_UNSUPPORTED, "bits=%d: only int4 and int3 group quantization is built", bits);
  const int e = 32 / bits;
  if (group_size <= 0 || group_size % e != 0)
    return fail(MI355GQ_ERR_ARG, "group_size=%d is not a multiple of %d elements per storage word",
                group_size, e);
  if (group_size != 4 * e)
    return fail(MI355GQ_ERR_UNSUPPORTED,
                "group_size=%d with bits=%d: kernels are built for 4 storage words per group "
                "(q4f16_1: 32, q3f16_1: 40)", group_size, bits);
  return MI355GQ_OK;
}

#define GQ_REQUIRE(cond, ...) \
  do {                        \
    if (!(cond)) return fail(MI355GQ_ERR_ARG, __VA_ARGS__); \
  } while (0)

#define GQ_CHECK(expr)        \
  do {                        \
    const int rc_ = (expr);   \
    if (rc_ != MI355GQ_OK) return rc_; \
  } while (0)

hipStream_t as_stream(mi355gq_stream_t s) { return static_cast<hipStream_t>(s); }

constexpr int64_t kMaxDim = int64_t(1) << 31;

// K = 0: the product is empty, the output is bias + residual (zeros without them).  The matmul
// kernels all assume at least one group, so this case never reaches them.
__global__ void empty_k_kernel(const __half* bias, const __half* residual, void* y, int64_t count,
                               int64_t N, int out_f32) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float v = bias ? __half2float(bias[i % N]) : 0.f;  // one rounding at the end, as in the matmul epilogues
  if (residual) v += __half2float(residual[i]);
  if (out_f32) static_cast<float*>(y)[i] = v;
  else static_cast<__half*>(y)[i] = __float2half(v);
}

int launch_empty_k(const void* bias, const void* residual, void* y, int64_t rows, int64_t N, int out_f32,
                   hipStream_t s) {
  const int64_t count = rows * N;
  if (count >= (int64_t(1) << 39)) return fail(MI355GQ_ERR_ARG, "K=0 output of %lld elements", (long long)count);
  hipLaunchKernelGGL(empty_k_kernel, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, s,
                     static_cast<const __half*>(bias), static_cast<const __half*>(residual), y, count, N,
                     out_f32);
  return hip_result(hipGetLastError(), "K=0 fill launch");
}

}  // namespace

extern "C" {

int mi355gq_version(void) { return MI355GQ_VERSION; }

const char* mi355gq_last_error(void) { return g_err; }

int mi355gq_check_device(void) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_result(e, "hipGetDevice");
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return hip_result(e, "hipGetDeviceProperties");
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(MI355GQ_ERR_UNSUPPORTED, "device %d is %s; this library holds gfx950 code only", dev,
                prop.gcnArchName);
  return MI355GQ_OK;
}

const char* mi355gq_testing_last_kernel(void) { return gq::g_last_kernel; }

int mi355gq_testing_set_option(const char* name, int value) {
  GQ_REQUIRE(name != nullptr, "option name is null");
  gq::Options& o = gq::options();
  if (value < 0) value = -1;  // any negative value restores the heuristic
  if (!strcmp(name, "gemv_rows_per_wave")) {
    GQ_REQUIRE(value == -1 || value == 1 || value == 2 || value == 4 || value == 8, "gemv_rows_per_wave=%d (1, 2, 4, 8)", value);
    o.gemv_rows_per_wave = value;
  } else if (!strcmp(name, "gemm_fast_loop")) {
    GQ_REQUIRE(value == -1 || value == 0, "gemm_fast_loop=%d (0)", value);
    o.gemm_fast_loop = value;
  } else if (!strcmp(name, "gemv_ksplit")) {
    GQ_REQUIRE(value >= -1 && value <= 1, "gemv_ksplit=%d (-1, 0, 1)", value);
    o.gemv_ksplit = value;
  } else if (!strcmp(name, "quad_ksplit")) {
    GQ_REQUIRE(value >= -1 && value <= 3, "quad_ksplit=%d (-1, 0, 1, 2, 3)", value);
    o.quad_ksplit = value;
  } else if (!strcmp(name, "quad_pairs")) {
    GQ_REQUIRE(value == -1 || value == 1 || value == 2, "quad_pairs=%d (1, 2)", value);
    o.quad_pairs = value;
  } else if (!strcmp(name, "gemv_variant")) {
    GQ_REQUIRE(value <= 15, "gemv_variant=%d (-1..15)", value);
    o.gemv_variant = value;
  } else if (!strcmp(name, "gemm_variant")) {
    GQ_REQUIRE(value <= 15, "gemm_variant=%d (-1..15)", value);
    o.gemm_variant = value;
  } else if (!strcmp(name, "gemv_waves")) {
    GQ_REQUIRE(value == -1 || (value >= 4 && value <= 16384), "gemv_waves=%d (4..16384)", value);
    o.gemv_waves = value;
  } else if (!strcmp(name, "gemm_split_k")) {
    GQ_REQUIRE(value == -1 || (value >= 1 && value <= 4096), "gemm_split_k=%d (1..4096)", value);
    o.gemm_split_k = value;
  } else {
    return fail(MI355GQ_ERR_ARG, "unknown option '%s'", name);
  }
  return MI355GQ_OK;
}

int mi355gq_testing_stream_read(const void* a, int64_t a_bytes, const void* b, int64_t b_bytes, void* sink,
                                void* stream) {
  GQ_REQUIRE(a_bytes >= 0 && b_bytes >= 0 && (a_bytes % 16) == 0 && (b_bytes % 16) == 0,
             "testing_stream_read: sizes must be non-negative multiples of 16");
  GQ_REQUIRE((a_bytes == 0 || a) && (b_bytes == 0 || b), "testing_stream_read: null pointer");
  GQ_REQUIRE(aligned16(a) && aligned16(b) && aligned4(sink), "testing_stream_read: 16-byte alignment");
  return hip_result(gq::launch_stream_read(a, a_bytes, b, b_bytes, sink, as_stream(stream)),
                    "stream read launch");
}

int mi355gq_quantize(const void* w, int64_t rows, int64_t K, int bits, int group_size,
                     int round_mode, void* q_weight, void* q_scale, mi355gq_stream_t stream) {
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(rows >= 0 && K >= 0 && rows < kMaxDim && K < kMaxDim, "quantize: bad shape [%lld, %lld]",
             (long long)rows, (long long)K);
  GQ_REQUIRE(round_mode == MI355GQ_ROUND_HALF_AWAY || round_mode == MI355GQ_ROUND_HALF_EVEN,
             "quantize: round_mode=%d", round_mode);
  if (rows == 0 || K == 0) return MI355GQ_OK;
  GQ_REQUIRE(w && q_weight && q_scale, "quantize: null pointer");
  GQ_REQUIRE(aligned16(w) && aligned16(q_weight) && aligned2(q_scale),
             "quantize: w and q_weight must be 16-byte aligned");
  return hip_result(gq::launch_quantize(static_cast<const uint16_t*>(w), rows, K, bits, group_size,
                                        round_mode, static_cast<uint32_t*>(q_weight),
                                        static_cast<uint16_t*>(q_scale), as_stream(stream)),
                    "quantize launch");
}

int mi355gq_dequantize(const void* q_weight, const void* q_scale, int64_t rows, int64_t K,
                       int bits, int group_size, void* out, mi355gq_stream_t stream) {
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(rows >= 0 && K >= 0 && rows < kMaxDim && K < kMaxDim, "dequantize: bad shape");
  if (rows == 0 || K == 0) return MI355GQ_OK;
  GQ_REQUIRE(q_weight && q_scale && out, "dequantize: null pointer");
  GQ_REQUIRE(aligned16(q_weight) && aligned16(out) && aligned2(q_scale),
             "dequantize: q_weight and out must be 16-byte aligned");
  return hip_result(gq::launch_dequantize(nullptr, rows, static_cast<const uint32_t*>(q_weight),
                                          static_cast<const uint16_t*>(q_scale), rows, K, bits,
                                          group_size, static_cast<uint16_t*>(out), as_stream(stream)),
                    "dequantize launch");
}

int mi355gq_embedding_take(const void* ids, int64_t T, const void* q_weight, const void* q_scale,
                           int64_t num_rows, int64_t K, int bits, int group_size, void* out,
                           mi355gq_stream_t stream) {
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(T >= 0 && K >= 0 && num_rows >= 0 && T < kMaxDim && K < kMaxDim,
             "embedding_take: bad shape");
  if (T == 0 || K == 0) return MI355GQ_OK;
  GQ_REQUIRE(num_rows > 0, "embedding_take: empty table");
  GQ_REQUIRE(ids && q_weight && q_scale && out, "embedding_take: null pointer");
  GQ_REQUIRE(aligned4(ids) && aligned16(q_weight) && aligned16(out),
             "embedding_take: q_weight and out must be 16-byte aligned");
  return hip_result(
      gq::launch_dequantize(static_cast<const int32_t*>(ids), T,
                            static_cast<const uint32_t*>(q_weight),
                            static_cast<const uint16_t*>(q_scale), num_rows, K, bits, group_size,
                            static_cast<uint16_t*>(out), as_stream(stream)),
      "embedding_take launch");
}

static int check_model_dtype(int model_dtype, const char* what) {
  if (model_dtype != MI355GQ_F16 && model_dtype != MI355GQ_F32 && model_dtype != MI355GQ_BF16)
    return fail(MI355GQ_ERR_ARG, "%s: model_dtype=%d (MI355GQ_F16, MI355GQ_F32 or MI355GQ_BF16)", what, model_dtype);
  return MI355GQ_OK;
}

int mi355gq_quantize_dt(const void* w, int64_t rows, int64_t K, int bits, int group_size, int round_mode,
                        int model_dtype, void* q_weight, void* q_scale, mi355gq_stream_t stream) {
  GQ_CHECK(check_model_dtype(model_dtype, "quantize_dt"));
  if (model_dtype == MI355GQ_F16)
    return mi355gq_quantize(w, rows, K, bits, group_size, round_mode, q_weight, q_scale, stream);
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(rows >= 0 && K >= 0 && rows < kMaxDim && K < kMaxDim, "quantize_dt: bad shape [%lld, %lld]",
             (long long)rows, (long long)K);
  GQ_REQUIRE(round_mode == MI355GQ_ROUND_HALF_AWAY || round_mode == MI355GQ_ROUND_HALF_EVEN,
             "quantize_dt: round_mode=%d", round_mode);
  if (rows == 0 || K == 0) return MI355GQ_OK;
  GQ_REQUIRE(w && q_weight && q_scale, "quantize_dt: null pointer");
  GQ_REQUIRE(aligned4(w) && aligned4(q_weight) && aligned2(q_scale) &&
                 (model_dtype != MI355GQ_F32 || aligned4(q_scale)),
             "quantize_dt: misaligned tensor");
  return hip_result(gq::launch_quantize_dt(w, rows, K, bits, group_size, round_mode, model_dtype,
                                           static_cast<uint32_t*>(q_weight), q_scale, as_stream(stream)),
                    "quantize_dt launch");
}

int mi355gq_dequantize_dt(const void* q_weight, const void* q_scale, int64_t rows, int64_t K, int bits,
                          int group_size, int model_dtype, void* out, mi355gq_stream_t stream) {
  GQ_CHECK(check_model_dtype(model_dtype, "dequantize_dt"));
  if (model_dtype == MI355GQ_F16)
    return mi355gq_dequantize(q_weight, q_scale, rows, K, bits, group_size, out, stream);
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(rows >= 0 && K >= 0 && rows < kMaxDim && K < kMaxDim, "dequantize_dt: bad shape");
  if (rows == 0 || K == 0) return MI355GQ_OK;
  GQ_REQUIRE(q_weight && q_scale && out, "dequantize_dt: null pointer");
  GQ_REQUIRE(aligned4(q_weight) && aligned2(out) && aligned2(q_scale) &&
                 (model_dtype != MI355GQ_F32 || (aligned4(q_scale) && aligned4(out))),
             "dequantize_dt: misaligned tensor");
  return hip_result(gq::launch_dequantize_dt(nullptr, rows, static_cast<const uint32_t*>(q_weight), q_scale, rows,
                                             K, bits, group_size, model_dtype, out, as_stream(stream)),
                    "dequantize_dt launch");
}

int mi355gq_embedding_take_dt(const void* ids, int64_t T, const void* q_weight, const void* q_scale,
                              int64_t num_rows, int64_t K, int bits, int group_size, int model_dtype,
                              void* out, mi355gq_stream_t stream) {
  GQ_CHECK(check_model_dtype(model_dtype, "embedding_take_dt"));
  if (model_dtype == MI355GQ_F16)
    return mi355gq_embedding_take(ids, T, q_weight, q_scale, num_rows, K, bits, group_size, out, stream);
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(T >= 0 && K >= 0 && num_rows >= 0 && T < kMaxDim && K < kMaxDim, "embedding_take_dt: bad shape");
  if (T == 0 || K == 0) return MI355GQ_OK;
  GQ_REQUIRE(num_rows > 0, "embedding_take_dt: empty table");
  GQ_REQUIRE(ids && q_weight && q_scale && out, "embedding_take_dt: null pointer");
  GQ_REQUIRE(aligned4(ids) && aligned4(q_weight) && aligned2(out) && aligned2(q_scale) &&
                 (model_dtype != MI355GQ_F32 || (aligned4(q_scale) && aligned4(out))),
             "embedding_take_dt: misaligned tensor");
  return hip_result(gq::launch_dequantize_dt(static_cast<const int32_t*>(ids), T,
                                             static_cast<const uint32_t*>(q_weight), q_scale, num_rows, K, bits,
                                             group_size, model_dtype, out, as_stream(stream)),
                    "embedding_take_dt launch");
}

// with_slices false: what the shape needs when the K slices of the kernel on unscaled weight operands go without
static int64_t linear_workspace_need(int64_t M, int64_t N, int64_t K, int bits, int group_size, bool with_slices) {
  if (check_scheme(bits, group_size) != MI355GQ_OK || M < 0 || N < 0 || K < 0 || M >= kMaxDim ||
      N >= kMaxDim || K >= kMaxDim)
    return 0;
  // q4 at 9..32 rows of a K beyond 4096, at 5..8 rows of a K beyond 8192: the K slices of the kernel on unscaled weight
  // operands (see linear_impl)
  const int64_t mid = (with_slices && bits == 4 && M <= 32 && (M > 8 || (M > 4 && K > 8192)))
                          ? gq::midrow_workspace_bytes(M, N, K)
                          : 0;
  // only the few-row GEMM (more rows than the GEMV / skinny kernels take, at most 256) splits K
  // (q4 at 9..16 rows: the skinny kernel, except on matrices of 40 M to 256 M weights, see linear_impl)
  if (M <= 16 && bits == 4 && !(M > 8 && N * K >= (40ll << 20) && N * K < (256ll << 20))) return mid;
  if (M <= 8) return mid;
  const int64_t gemm = gq::gemm_workspace_bytes(M, N, K, bits, group_size);
  return gemm > mid ? gemm : mid;
}

int64_t mi355gq_linear_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits, int group_size) {
  return linear_workspace_need(M, N, K, bits, group_size, true);
}

int64_t mi355gq_linear_dt_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits, int group_size,
                                          int model_dtype) {
  if (model_dtype == MI355GQ_F16) return mi355gq_linear_workspace_bytes(M, N, K, bits, group_size);
  if (model_dtype != MI355GQ_BF16 || check_scheme(bits, group_size) != MI355GQ_OK || M < 2 || N < 0 || K < 0 ||
      M >= kMaxDim || N >= kMaxDim || K >= kMaxDim)
    return 0;
  // bfloat16: every batch from two rows on may run the few-row GEMM (there are no bf16 skinny kernels); 9..16 rows of a
  // long K: the K slices of the kernel on unscaled weight operands
  const int64_t mid = (bits == 4 && M <= 16 && (M > 8 || (M > 4 && K > 8192))) ? gq::midrow_workspace_bytes(M, N, K) : 0;
  const int64_t gemm = gq::gemm_workspace_bytes(M, N, K, bits, group_size);
  return gemm > mid ? gemm : mid;
}

int64_t mi355gq_linear_silu_mul_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits, int group_size) {
  if (check_scheme(bits, group_size) != MI355GQ_OK || M < 0 || N < 0 || K < 0 || M >= kMaxDim ||
      N >= kMaxDim || K >= kMaxDim)
    return 0;
  // q4 at 9..32 rows of a K beyond 4096, at 5..8 rows of a K beyond 8192: the K slices of the kernel on unscaled weight
  // operands (as the plain linear)
  const int64_t mid = (bits == 4 && M <= 32 && (M > 8 || (M > 4 && K > 8192)) && (N % 32) == 0)
                          ? gq::midrow_workspace_bytes(M, N, K)
                          : 0;
  // GEMV / few-row kernels, or a shape that never splits
  if (M <= 8 || (N % 64) != 0) return mid;
  if (M <= 16 && !(bits == 4 && N * K >= (40ll << 20) && N * K < (256ll << 20))) return mid;
  const int64_t gemm = gq::gemm_workspace_bytes(M, N, K, bits, group_size);
  return gemm > mid ? gemm : mid;
}

// paired: the fused gate/up form (y fp16 [M, N / 2]); a shape no fused kernel takes is an
// MI355GQ_ERR_UNSUPPORTED, for which the caller runs linear and silu_mul
static int linear_impl(const void* x, const void* q_weight, const void* q_scale, const void* bias,
                       const void* residual, int64_t M, int64_t N, int64_t K, int bits, int group_size,
                       int out_dtype, void* y, void* workspace, int64_t workspace_bytes,
                       mi355gq_stream_t stream, bool paired = false) {
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(M >= 0 && N >= 0 && K >= 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim,
             "linear: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  GQ_REQUIRE(out_dtype == MI355GQ_F16 || out_dtype == MI355GQ_F32, "linear: out_dtype=%d", out_dtype);
  GQ_REQUIRE(workspace_bytes >= 0, "linear: negative workspace size");
  if (M == 0 || N == 0) return MI355GQ_OK;
  GQ_REQUIRE(y != nullptr, "linear: y is null");
  GQ_REQUIRE(K == 0 || (x && q_weight && q_scale), "linear: null pointer");
  GQ_REQUIRE(aligned16(x) && aligned16(q_weight) && aligned2(q_scale) && aligned4(y) &&
                 aligned2(bias) && aligned2(residual),
             "linear: x and q_weight must be 16-byte aligned");
  // y may be the residual buffer itself (same element type), nothing else may overlap it
  GQ_REQUIRE(residual == nullptr || residual != y || out_dtype == MI355GQ_F16,
             "linear: in-place residual needs a float16 output");
  if (paired) {
    GQ_REQUIRE((N & 1) == 0, "linear_silu_mul: N=%lld must be even (gate rows, then up rows)", (long long)N);
    if (K == 0) return launch_empty_k(nullptr, nullptr, y, M, N / 2, 0, as_stream(stream));  // silu(0) * 0
  }
  if (K == 0) return launch_empty_k(bias, residual, y, M, N, out_dtype == MI355GQ_F32, as_stream(stream));
  // regimes: M <= 2 register GEMV; 3..8 quad-row kernel (LDS GEMV when it declines a q3 shape);
  // 9..16 MFMA skinny kernel (q4); else GEMM
  gq::GemmArgs g{};
  g.x = static_cast<const uint16_t*>(x);
  g.q_weight = static_cast<const uint32_t*>(q_weight);
  g.q_scale = static_cast<const uint16_t*>(q_scale);
  g.bias = static_cast<const uint16_t*>(bias);
  g.residual = static_cast<const uint16_t*>(residual);
  g.y = y;
  g.indptr = nullptr; g.indptr_i64 = 0;
  g.rows = M; g.N = N; g.K = K; g.num_experts = 1;
  g.bits = bits; g.group_size = group_size; g.out_f32 = out_dtype == MI355GQ_F32;
  g.workspace = workspace; g.workspace_bytes = workspace ? workspace_bytes : 0;
  g.paired = paired;
  // q3, 9..16 rows as passes of the quad-row kernel: only on the smaller matrices (see below)
  const bool q3_passes_lose = bits == 3 && M > 8 && gq::options().gemv_variant < 0 && N * K >= (40ll << 20) &&
                              (K & 7) == 0;
  // q4, 9..16 rows: the skinny kernel on the small projections and on the largest one; in between (40 M to 256 M weights) the
  // GEMM's 32-row tile is ahead of it since it reads its scales in bulk, provided its split of K has its scratch
  // (28672 x 4096 at 9 / 12 / 16 rows 30.3 / 32.5 / 33.4 us against 27.5-28.3, 4096 x 14336 21.9-22.0 against 19.5-20.4; while
  //  4096 x 4096 stays at 9.3 against 11.5, 6144 x 4096 at 12.4-13.2 against 13.1 and 128256 x 4096 at 85-92 against 99)
  bool q4_skinny_loses = false;
  if (bits == 4 && M > 8 && M <= 16 && gq::options().gemv_variant < 0 && (K & 7) == 0 && N * K >= (40ll << 20) &&
      N * K < (256ll << 20)) {
    const int64_t need = gq::gemm_workspace_bytes(M, N, K, bits, group_size);
    q4_skinny_loses = need == 0 || (workspace != nullptr && workspace_bytes >= need);
  }
  // q4, 9..16 rows of a K that one phase covers (up to 4096; two phases: below), from about 24 M weights on: the kernel that multiplies
  // unscaled weight operands and scales the matrix instruction's result (28672 x 4096 at 9 / 16 rows 20.0 / 20.3 us
  // against 27.8-28.1 for the GEMM's 32-row tile, 6144 x 4096 10.4 / 10.9 against 12.2 / 13.1 for the skinny kernel;
  // 4096 x 4096 stays with the skinny kernel, 9.0-9.4 either way, and a longer K with the GEMM's tiles, 4096 x 14336
  // 26-27 against 20).  The same test for the plain and the fused gate/up form: both must add in the same order.
  // (K of two phases, up to 8192, from 48 M weights on: 10240 x 8192 28 -> 21-22 us, 8192 x 8192 21 -> 17-18.5, 57344 x 8192
  //  100-106 -> 74-78, 15360 x 5120 24.5 -> 21-22, 27648 x 5120 33.4-34.4 -> 32.4-33.8)
  // 17..32 rows (two batch tiles per pass, the offsets subtracted from the weight operand): one phase and 48 M weights or more
  // (14336 x 4096 at 17 / 24 / 32 rows 19.4 / 19.9 / 20.4 -> 16.9 / 17.9 / 19.0 us, 28672 x 4096 28.3 / 28.0 / 27.9 -> 26.0 / 26.1 / 27.5, 128256 x
  //  4096 99-101 -> 84-87; 6144 x 4096 13.4-14.4 against 12.3-14.1 and 4096 x 4096 stay with the GEMM's tile).
  // A longer K runs as K slices over workgroups where the caller brings the scratch for their partial sums
  // (mi355gq_linear_workspace_bytes), ahead of the phases everywhere and of the GEMM's tiles at 9..16 rows from 24 M weights
  // on (4096 x 14336 20.1 / 19.5 -> 16.5 / 17.2 us at 9 / 16 rows, 5120 x 13824 24.2 / 24.7 -> 18.7 / 19.4, 8192 x 28672 49.7 / 51.9 -> 38.7 / 39.8,
  //  57344 x 8192 72.9 / 77.4 in phases -> 64.5 / 68.1) and at 17..32 rows from 256 M weights on (57344 x 8192 97 -> 85; 4096 x 14336
  //  20.0 against 22.1 and 8192 x 28672 52 against 52 stay with the tiles).
  const bool slices_ok = K > 4096 && workspace != nullptr && aligned16(workspace) &&
                         workspace_bytes >= gq::midrow_workspace_bytes(M, N, K) && gq::options().gemv_ksplit != 0;
  // 5..8 rows of a K beyond 8192 from 64 M weights on, as K slices: the quad-row kernels read x once per four rows and K
  // share there (8192 x 28672 at 5 / 8 rows 46.1 / 47.3 -> 37.0 us, 5120 x 13824 22.3 / 23.2 -> 18.2 / 18.6; 4096 x 14336 15.3-16.1 against
  // 15.9-16.2 and up to four rows, 36.6 against 36.5 and 17.2 against 18.4, stay with them)
  const bool mid_size =
      (M > 4 && M <= 8 && slices_ok && K > 8192 && N * K >= (64ll << 20)) ||
      (M > 8 && M <= 16 && N * K >= (24ll << 20) && (K <= 4096 || slices_ok || (K <= 8192 && N * K >= (48ll << 20)))) ||
      (M > 16 && M <= 32 && ((K <= 4096 && N * K >= (48ll << 20)) || (slices_ok && N * K >= (256ll << 20))));
  const bool mid_rows = bits == 4 && mid_size && gq::options().gemm_variant < 0 &&
                        (gq::options().gemv_variant < 0 || gq::options().gemv_variant == 10) && (K & 255) == 0 &&
                        (N & 31) == 0;
  if (mid_rows || gq::options().gemv_variant == 10) {  // (10: forced, whatever the shape)
    const hipError_t e = gq::launch_midrow(g, static_cast<int>(M), as_stream(stream));
    if (e != hipErrorNotSupported) return hip_result(e, "mid-row launch");
  }
  if (paired) {
    // the regimes of the plain linear: register GEMV up to 2 rows, quad-row kernel up to 8 (q3: 16),
    // skinny kernel up to 16 (q4), else the pipelined GEMM
    hipError_t e = hipErrorNotSupported;
    const int gvp2 = gq::options().gemv_variant;
    if (M == 2 && bits == 4 && gq::options().gemm_variant < 0 && (gvp2 < 0 || gvp2 == 9))  // as the plain linear
      e = gq::launch_quadreg(g, static_cast<int>(M), as_stream(stream));
    if (e == hipErrorNotSupported &&
        ((M == 2 && (K > 8192 || N * K >= (bits == 3 ? (80ll << 20) : (1ll << 28)))) || (M <= 2 && K > 24576)))
      e = gq::launch_quadrow(g, static_cast<int>(M), as_stream(stream));
    if (e != hipErrorNotSupported) {
      // served above
    } else if (M <= 2) {
      gq::GemvArgs a{};
      a.x = g.x; a.q_weight = g.q_weight; a.q_scale = g.q_scale; a.bias = nullptr; a.y = y;
      a.expert_ids = nullptr;
      a.M = M; a.N = N; a.K = K; a.slots = 1; a.x_slot_stride = 0; a.num_experts = 1;
      a.bits = bits; a.group_size = group_size; a.out_f32 = 0; a.paired = 1;
      e = gq::launch_gemv(a, as_stream(stream));
    } else if (M <= (bits == 3 ? 16 : 8) && !q3_passes_lose) {
      const int gvp = gq::options().gemv_variant;
      if (M <= 8 && (gvp < 0 || gvp == 9)) e = gq::launch_quadreg(g, static_cast<int>(M), as_stream(stream));
      if (e == hipErrorNotSupported) e = gq::launch_quadrow(g, static_cast<int>(M), as_stream(stream));
    }
    // (one or two rows never reach the matrix-core kernels in the plain linear either: without a fused form
    //  the caller runs the two steps, and the result stays the same bit for bit)
    if (e == hipErrorNotSupported && M > 2 && M <= 16 && bits == 4 && !q4_skinny_loses)
      e = gq::launch_skinny(g, static_cast<int>(M), as_stream(stream));
    if (e == hipErrorNotSupported && M > 2) e = gq::launch_gemm(g, as_stream(stream));
    if (e == hipErrorNotSupported)
      return fail(MI355GQ_ERR_UNSUPPORTED, "linear_silu_mul: no fused kernel for M=%lld N=%lld K=%lld (K %% 8 != 0?)",
                  (long long)M, (long long)N, (long long)K);
    return hip_result(e, "linear_silu_mul launch");
  }
  const int gv = gq::options().gemv_variant;  // 2..5 force a gq_skinny.hip form, 6..8 the quad-row kernel
  const int gm = gq::options().gemm_variant;  // 1: GEMM only, 2: GEMV up to 8 rows
  // (q3 has no 16x16x32 skinny kernel: 9..16 rows run as two concurrent 8-row passes of the quad-row kernel)
  // (... on the smaller matrices: from about 40 M weights on, the GEMM's 32-row tile is ahead of them: gate_up 38
  //  against 42-46 us, down 25.6 against 27-29.5, while qkv stays at 14.7 against 17.1 and o_proj at 10.3 against 15.2)
  // 3..8 rows: the 4x4x4 kernel with x resident in registers, where it applies
  // (q4 also at 2 rows: 28672 x 4096 13.9 us against 17.1 for the two-row GEMV, 6144 x 4096 5.8 / 6.2, 4096 x 4096 4.9 / 5.2,
  //  128256 x 4096 52 against 56 for the kernel with x in LDS)
  if (M >= (bits == 4 ? 2 : 3) && M <= 8 && gm < 0 && (gv < 0 || gv == 9)) {
    const hipError_t q = gq::launch_quadreg(g, static_cast<int>(M), as_stream(stream));
    if (q != hipErrorNotSupported) return hip_result(q, "quad-row (registers) launch");
  }
  if (bits == 3 && M >= 3 && M <= 16 && gm != 1 && (M > 8 || gm != 2) && (gv < 0 || (gv >= 6 && gv <= 8)) &&
      !q3_passes_lose) {
    const hipError_t q = gq::launch_quadrow(g, static_cast<int>(M), as_stream(stream));
    if (q != hipErrorNotSupported) return hip_result(q, "quad-row launch");
  }
  // two rows of a long K (down_proj): the register GEMV holds 6-7 groups per lane there and measured 19.0 us (q4)
  // / 17.9 us (q3) on 4096 x 14336 against 14.3-16.4 us for the quad-row kernel at 3-4 rows
  // (beyond K = 24 Ki the register GEMV does not apply at all and the quad-row kernel also takes single rows)
  const bool long_k = (M == 2 && K > 8192) || K > 24576;
  // ... and two rows of a very large matrix (lm_head 128256 x 4096: 56 us against 70; 70B gate_up 58 against 66)
  // (q3f16_1 from about 80 M weights: 22016 x 4096 13.4 us against 14.9, while 12288 x 4096 stays at 9.8 against 10.2)
  const bool huge2 = M == 2 && N * K >= (bits == 3 ? (80ll << 20) : (1ll << 28));
  if (M <= 2 && gm < 0 && ((gv < 0 && (long_k || huge2)) || (gv >= 6 && gv <= 8))) {
    const hipError_t q = gq::launch_quadrow(g, static_cast<int>(M), as_stream(stream));
    if (q != hipErrorNotSupported) return hip_result(q, "quad-row launch");
  }
  const bool use_gemv = M <= 2 || (M <= 8 && (bits != 4 || gm == 2));
  if (use_gemv) {
    gq::GemvArgs a{};
    a.x = static_cast<const uint16_t*>(x);
    a.q_weight = static_cast<const uint32_t*>(q_weight);
    a.q_scale = static_cast<const uint16_t*>(q_scale);
    a.bias = static_cast<const uint16_t*>(bias);
    a.residual = static_cast<const uint16_t*>(residual);
    a.y = y;
    a.expert_ids = nullptr;
    a.M = M; a.N = N; a.K = K; a.slots = 1; a.x_slot_stride = 0; a.num_experts = 1;
    a.bits = bits; a.group_size = group_size; a.out_f32 = out_dtype == MI355GQ_F32;
    return hip_result(gq::launch_gemv(a, as_stream(stream)), "gemv launch");
  }
  if (M <= 16 && bits == 4 && gm != 1 && !q4_skinny_loses) {
    if ((gv < 0 && M <= 8) || (gv >= 6 && gv <= 8)) {
      const hipError_t q = gq::launch_quadrow(g, static_cast<int>(M), as_stream(stream));
      if (q != hipErrorNotSupported) return hip_result(q, "quad-row launch");
    }
    const hipError_t e = gq::launch_skinny(g, static_cast<int>(M), as_stream(stream));
    if (e != hipErrorNotSupported) return hip_result(e, "skinny launch");
  }
  return hip_result(gq::launch_gemm(g, as_stream(stream)), "gemm launch");
}

int mi355gq_linear(const void* x, const void* q_weight, const void* q_scale, const void* bias,
                   int64_t M, int64_t N, int64_t K, int bits, int group_size, int out_dtype,
                   void* y, void* workspace, int64_t workspace_bytes, mi355gq_stream_t stream) {
  return linear_impl(x, q_weight, q_scale, bias, nullptr, M, N, K, bits, group_size, out_dtype, y,
                     workspace, workspace_bytes, stream);
}

// ---- the linear for callers that cannot allocate: split-K partial sums in a device array of the library's own
constexpr int64_t kStaticScratchBytes = int64_t(32) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// The array's device address on the current device (each GPU holds its own copy at its own address), looked up
// once per device.  In host code `scratch` is only a handle for this lookup, never an address.
static int static_scratch_ptr(void** out) {
  constexpr int kMaxDevices = 64;
  static std::atomic<void*> ptrs[kMaxDevices];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_result(e, "hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices) return fail(MI355GQ_ERR_UNSUPPORTED, "linear_static_scratch: device %d", dev);
  void* p = ptrs[dev].load(std::memory_order_acquire);
  if (p == nullptr) {  // (two threads that race here look the same address up twice)
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hip_result(e, "hipGetSymbolAddress(scratch)");
    if (p == nullptr) return fail(MI355GQ_ERR_HIP, "hipGetSymbolAddress(scratch) returned a null address");
    ptrs[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return MI355GQ_OK;
}

int64_t mi355gq_linear_static_scratch_max_bytes(void) { return kStaticScratchBytes; }

int mi355gq_linear_static_scratch_init(void) {
  void* p = nullptr;
  return static_scratch_ptr(&p);
}

int mi355gq_linear_static_scratch(const void* x, const void* q_weight, const void* q_scale, const void* bias,
                                  int64_t M, int64_t N, int64_t K, int bits, int group_size, int out_dtype,
                                  void* y, mi355gq_stream_t stream) {
  // (the K slices of 5..32 rows are an option of the dispatch: where their sums do not fit, the shape runs without them)
  int64_t need = linear_workspace_need(M, N, K, bits, group_size, true);
  if (need > kStaticScratchBytes) need = linear_workspace_need(M, N, K, bits, group_size, false);
  if (need > kStaticScratchBytes)
    return fail(MI355GQ_ERR_WORKSPACE,
                "linear_static_scratch: M=%lld N=%lld K=%lld wants %lld bytes of split-K partial sums, the library's "
                "array holds %lld; call mi355gq_linear with a workspace of the caller's",
                (long long)M, (long long)N, (long long)K, (long long)need, (long long)kStaticScratchBytes);
  void* ws = nullptr;
  if (need > 0) GQ_CHECK(static_scratch_ptr(&ws));
  return linear_impl(x, q_weight, q_scale, bias, nullptr, M, N, K, bits, group_size, out_dtype, y, ws,
                     ws ? kStaticScratchBytes : 0, stream);
}

// ---- KN layout (q4f16_0 / q3f16_0): tensors as convert_weight stores them
static int64_t align256(int64_t v) { return (v + 255) & ~int64_t(255); }

int mi355gq_kn_to_nk(const void* q_weight_kn, const void* q_scale_kn, int64_t N, int64_t K, int bits, int group_size,
                     void* q_weight_nk, void* q_scale_nk, mi355gq_stream_t stream) {
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(N >= 0 && K >= 0 && N < kMaxDim && K < kMaxDim, "kn_to_nk: bad shape N=%lld K=%lld", (long long)N, (long long)K);
  if (N == 0 || K == 0) return MI355GQ_OK;
  GQ_REQUIRE(q_weight_kn && q_scale_kn && q_weight_nk && q_scale_nk, "kn_to_nk: null pointer");
  GQ_REQUIRE(aligned4(q_weight_kn) && aligned4(q_weight_nk) && aligned2(q_scale_kn) && aligned2(q_scale_nk),
             "kn_to_nk: misaligned tensor");
  const int64_t ng = (K + group_size - 1) / group_size, nw = 4 * ng;
  return hip_result(gq::launch_kn_transpose(static_cast<const uint32_t*>(q_weight_kn), static_cast<const uint16_t*>(q_scale_kn),
                                            nw, ng, N, static_cast<uint32_t*>(q_weight_nk),
                                            static_cast<uint16_t*>(q_scale_nk), as_stream(stream)),
                    "kn_to_nk launch");
}

int mi355gq_nk_to_kn(const void* q_weight_nk, const void* q_scale_nk, int64_t N, int64_t K, int bits, int group_size,
                     void* q_weight_kn, void* q_scale_kn, mi355gq_stream_t stream) {
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(N >= 0 && K >= 0 && N < kMaxDim && K < kMaxDim, "nk_to_kn: bad shape N=%lld K=%lld", (long long)N, (long long)K);
  if (N == 0 || K == 0) return MI355GQ_OK;
  GQ_REQUIRE(q_weight_kn && q_scale_kn && q_weight_nk && q_scale_nk, "nk_to_kn: null pointer");
  GQ_REQUIRE(aligned4(q_weight_kn) && aligned4(q_weight_nk) && aligned2(q_scale_kn) && aligned2(q_scale_nk),
             "nk_to_kn: misaligned tensor");
  const int64_t ng = (K + group_size - 1) / group_size, nw = 4 * ng;
  // both source tensors have N rows; their widths differ, so they go as two transposes
  hipError_t e = gq::launch_kn_transpose(static_cast<const uint32_t*>(q_weight_nk), nullptr, N, 0, nw,
                                         static_cast<uint32_t*>(q_weight_kn), nullptr, as_stream(stream));
  if (e == hipSuccess)
    e = gq::launch_kn_transpose(nullptr, static_cast<const uint16_t*>(q_scale_nk), 0, N, ng, nullptr,
                                static_cast<uint16_t*>(q_scale_kn), as_stream(stream));
  return hip_result(e, "nk_to_kn launch");
}

int mi355gq_dequantize_kn(const void* q_weight, const void* q_scale, int64_t N, int64_t K, int bits, int group_size,
                          void* out, mi355gq_stream_t stream) {
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(N >= 0 && K >= 0 && N < kMaxDim && K < kMaxDim, "dequantize_kn: bad shape");
  if (N == 0 || K == 0) return MI355GQ_OK;
  GQ_REQUIRE(q_weight && q_scale && out, "dequantize_kn: null pointer");
  GQ_REQUIRE(aligned4(q_weight) && aligned2(q_scale) && aligned2(out), "dequantize_kn: misaligned tensor");
  return hip_result(gq::launch_dequantize_kn(static_cast<const uint32_t*>(q_weight), static_cast<const uint16_t*>(q_scale), N,
                                             K, bits, static_cast<uint16_t*>(out), as_stream(stream)),
                    "dequantize_kn launch");
}

// workspace of mi355gq_linear_kn: the GEMV's partial sums (M <= 8), or an NK copy of both tensors plus what mi355gq_linear
// wants for the shape
int64_t mi355gq_linear_kn_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits, int group_size) {
  if (check_scheme(bits, group_size) != MI355GQ_OK || M < 0 || N < 0 || K < 0 || M >= kMaxDim || N >= kMaxDim || K >= kMaxDim)
    return 0;
  const int64_t ng = (K + group_size - 1) / group_size, nw = 4 * ng;
  if (M >= 1 && M <= 8 && (N & 3) == 0) return gq::gemv_kn_workspace_bytes(M, N, K, bits);
  return align256(N * nw * 4) + align256(N * ng * 2) + mi355gq_linear_workspace_bytes(M, N, K, bits, group_size);
}

int mi355gq_linear_kn(const void* x, const void* q_weight, const void* q_scale, const void* bias, int64_t M, int64_t N,
                      int64_t K, int bits, int group_size, int out_dtype, void* y, void* workspace,
                      int64_t workspace_bytes, mi355gq_stream_t stream) {
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(M >= 0 && N >= 0 && K >= 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim,
             "linear_kn: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  GQ_REQUIRE(out_dtype == MI355GQ_F16 || out_dtype == MI355GQ_F32, "linear_kn: out_dtype=%d", out_dtype);
  GQ_REQUIRE(workspace_bytes >= 0, "linear_kn: negative workspace size");
  if (M == 0 || N == 0) return MI355GQ_OK;
  GQ_REQUIRE(y != nullptr, "linear_kn: y is null");
  if (K == 0) return launch_empty_k(bias, nullptr, y, M, N, out_dtype == MI355GQ_F32, as_stream(stream));
  GQ_REQUIRE(x && q_weight && q_scale, "linear_kn: null pointer");
  GQ_REQUIRE(aligned2(x) && aligned4(q_weight) && aligned2(q_scale) && aligned4(y) && aligned2(bias),
             "linear_kn: misaligned tensor");
  if (workspace == nullptr) workspace_bytes = 0;
  if (M <= 8) {
    const hipError_t e = gq::launch_gemv_kn(static_cast<const uint16_t*>(x), static_cast<const uint32_t*>(q_weight),
                                            static_cast<const uint16_t*>(q_scale), static_cast<const uint16_t*>(bias), M, N,
                                            K, bits, out_dtype == MI355GQ_F32, y, workspace, workspace_bytes,
                                            as_stream(stream));
    if (e != hipErrorNotSupported) return hip_result(e, "linear_kn launch");
  }
  // every other shape: an NK copy in the workspace, then the NK kernels
  const int64_t ng = (K + group_size - 1) / group_size, nw = 4 * ng;
  const int64_t w_bytes = align256(N * nw * 4), s_bytes = align256(N * ng * 2);
  if (workspace_bytes < w_bytes + s_bytes || !aligned16(workspace))
    return fail(MI355GQ_ERR_WORKSPACE,
                "linear_kn: M=%lld N=%lld K=%lld runs on an NK copy of the weights and needs a 16-byte aligned workspace of "
                "%lld bytes (mi355gq_linear_kn_workspace_bytes); got %lld",
                (long long)M, (long long)N, (long long)K,
                (long long)mi355gq_linear_kn_workspace_bytes(M, N, K, bits, group_size), (long long)workspace_bytes);
  char* const ws = static_cast<char*>(workspace);
  GQ_CHECK(mi355gq_kn_to_nk(q_weight, q_scale, N, K, bits, group_size, ws, ws + w_bytes, stream));
  return linear_impl(x, ws, ws + w_bytes, bias, nullptr, M, N, K, bits, group_size, out_dtype, y, ws + w_bytes + s_bytes,
                     workspace_bytes - w_bytes - s_bytes, stream);
}

int mi355gq_linear_residual(const void* x, const void* q_weight, const void* q_scale,
                            const void* bias, const void* residual, int64_t M, int64_t N, int64_t K,
                            int bits, int group_size, int out_dtype, void* y, void* workspace,
                            int64_t workspace_bytes, mi355gq_stream_t stream) {
  GQ_REQUIRE(residual != nullptr || M == 0 || N == 0, "linear_residual: residual is null");
  return linear_impl(x, q_weight, q_scale, bias, residual, M, N, K, bits, group_size, out_dtype, y,
                     workspace, workspace_bytes, stream);
}

int mi355gq_linear_silu_mul(const void* x, const void* q_weight, const void* q_scale, int64_t M, int64_t N,
                            int64_t K, int bits, int group_size, void* y, void* workspace,
                            int64_t workspace_bytes, mi355gq_stream_t stream) {
  return linear_impl(x, q_weight, q_scale, nullptr, nullptr, M, N, K, bits, group_size, MI355GQ_F16, y,
                     workspace, workspace_bytes, stream, true);
}

static int moe_gemv_impl(const void* x, int64_t x_rows, const void* q_weight, const void* q_scale,
                         const void* expert_ids, int64_t top_k, int64_t num_experts, int64_t N,
                         int64_t K, int bits, int group_size, void* out, mi355gq_stream_t stream,
                         bool paired) {
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(top_k >= 0 && top_k <= 65535 && N >= 0 && K >= 0 && N < kMaxDim && K < kMaxDim &&
                 num_experts > 0 && num_experts < kMaxDim,
             "moe_gemv: bad shape");
  GQ_REQUIRE(x_rows == 1 || x_rows == top_k, "moe_gemv: x has %lld rows, expected 1 or top_k=%lld",
             (long long)x_rows, (long long)top_k);
  if (top_k == 0 || N == 0) return MI355GQ_OK;
  GQ_REQUIRE(out && (K == 0 || (x && q_weight && q_scale && expert_ids)), "moe_gemv: null pointer");
  GQ_REQUIRE(aligned16(x) && aligned16(q_weight) && aligned4(expert_ids) && aligned2(out),
             "moe_gemv: x and q_weight must be 16-byte aligned");
  GQ_REQUIRE(!paired || (N & 1) == 0, "moe_gemv_silu_mul: N=%lld must be even", (long long)N);
  if (K == 0) return launch_empty_k(nullptr, nullptr, out, top_k, paired ? N / 2 : N, 0, as_stream(stream));
  gq::GemvArgs a{};
  a.x = static_cast<const uint16_t*>(x);
  a.q_weight = static_cast<const uint32_t*>(q_weight);
  a.q_scale = static_cast<const uint16_t*>(q_scale);
  a.bias = nullptr;
  a.y = out;
  a.expert_ids = static_cast<const int32_t*>(expert_ids);
  a.M = 1; a.N = N; a.K = K; a.slots = top_k; a.x_slot_stride = x_rows == 1 ? 0 : K;
  a.num_experts = num_experts;
  a.bits = bits; a.group_size = group_size; a.out_f32 = 0; a.paired = paired;
  const hipError_t e = gq::launch_gemv(a, as_stream(stream));
  if (paired && e == hipErrorNotSupported)
    return fail(MI355GQ_ERR_UNSUPPORTED, "moe_gemv_silu_mul: no fused kernel for N=%lld K=%lld", (long long)N,
                (long long)K);
  return hip_result(e, "moe_gemv launch");
}

// paired: the fused gate/up form (y in the model dtype, [M, N / 2]); float16 and bfloat16 models
static int linear_dt_impl(const void* x, const void* q_weight, const void* q_scale, const void* bias,
                          const void* residual, int64_t M, int64_t N, int64_t K, int bits, int group_size,
                          int model_dtype, int out_dtype, void* y, void* workspace, int64_t workspace_bytes,
                          mi355gq_stream_t stream, bool paired = false) {
  GQ_CHECK(check_model_dtype(model_dtype, "linear_dt"));
  if (model_dtype == MI355GQ_F16)
    return linear_impl(x, q_weight, q_scale, bias, residual, M, N, K, bits, group_size, out_dtype, y, workspace,
                       workspace_bytes, stream, paired);
  if (paired) {
    GQ_REQUIRE((N & 1) == 0, "linear_silu_mul_dt: N=%lld must be even", (long long)N);
    if (model_dtype != MI355GQ_BF16)
      return fail(MI355GQ_ERR_UNSUPPORTED, "linear_silu_mul_dt: no fused kernel for float32 models");
  }
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(M >= 0 && N >= 0 && K >= 1 && M < kMaxDim && N < kMaxDim && K < kMaxDim,
             "linear_dt: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  GQ_REQUIRE(out_dtype == MI355GQ_F32 || out_dtype == model_dtype,
             "linear_dt: out_dtype=%d (the model dtype or MI355GQ_F32)", out_dtype);
  if (M == 0 || N == 0) return MI355GQ_OK;
  GQ_REQUIRE(y && x && q_weight && q_scale, "linear_dt: null pointer");
  const bool f32 = model_dtype == MI355GQ_F32;
  GQ_REQUIRE(aligned16(q_weight) && (f32 ? aligned4(x) && aligned4(q_scale) && aligned4(bias) && aligned4(residual)
                                         : aligned2(x) && aligned2(q_scale) && aligned2(bias) && aligned2(residual)) &&
                 (out_dtype == MI355GQ_F32 ? aligned4(y) : aligned2(y)),
             "linear_dt: q_weight must be 16-byte aligned, the other tensors naturally aligned");
  if (model_dtype == MI355GQ_BF16 && M == 2 && bits == 4 && (K & 7) == 0 && aligned16(x) && gq::options().gemm_variant < 0 &&
      (gq::options().gemv_variant < 0 || gq::options().gemv_variant == 9)) {
    // two rows of q4: the few-row kernel with x in registers, as in the float16 linear (28672 x 4096 14.6 us against 17.4
    // for the two-row GEMV, 6144 x 4096 6.1 / 6.4, 4096 x 4096 4.9 / 5.2, 128256 x 4096 51 / 62)
    gq::GemmArgs g2{};
    g2.x = static_cast<const uint16_t*>(x);
    g2.q_weight = static_cast<const uint32_t*>(q_weight);
    g2.q_scale = static_cast<const uint16_t*>(q_scale);
    g2.bias = static_cast<const uint16_t*>(bias);
    g2.residual = static_cast<const uint16_t*>(residual);
    g2.y = y;
    g2.indptr = nullptr; g2.indptr_i64 = 0;
    g2.rows = M; g2.N = N; g2.K = K; g2.num_experts = 1;
    g2.bits = bits; g2.group_size = group_size; g2.out_f32 = out_dtype == MI355GQ_F32;
    g2.bf16 = 1;
    g2.paired = paired;
    const hipError_t qr = gq::launch_quadreg(g2, static_cast<int>(M), as_stream(stream));
    if (qr != hipErrorNotSupported) return hip_result(qr, "linear_dt quad-row (registers) launch");
  }
  if (model_dtype == MI355GQ_BF16 && M <= 2 && aligned16(x)) {
    // one or two rows: the float16 path's register-resident GEMV on v_dot2_f32_bf16
    gq::GemvArgs a{};
    a.x = static_cast<const uint16_t*>(x);
    a.q_weight = static_cast<const uint32_t*>(q_weight);
    a.q_scale = static_cast<const uint16_t*>(q_scale);
    a.bias = static_cast<const uint16_t*>(bias);
    a.residual = static_cast<const uint16_t*>(residual);
    a.y = y;
    a.expert_ids = nullptr;
    a.M = M; a.N = N; a.K = K; a.slots = 1; a.x_slot_stride = 0; a.num_experts = 1;
    a.bits = bits; a.group_size = group_size; a.out_f32 = out_dtype == MI355GQ_F32;
    a.bf16 = 1;
    a.paired = paired;
    const hipError_t e = gq::launch_gemv(a, as_stream(stream));
    if (e != hipErrorNotSupported) return hip_result(e, "linear_dt gemv launch");
    // (one or two rows: the plain linear may still take the GEMV where its fused form does not exist, so the
    //  caller runs the two steps and the result stays the same bit for bit)
    if (paired) return fail(MI355GQ_ERR_UNSUPPORTED, "linear_silu_mul_dt: no fused GEMV for M=%lld K=%lld",
                            (long long)M, (long long)K);
  }
  if (paired && M <= 2)
    return fail(MI355GQ_ERR_UNSUPPORTED, "linear_silu_mul_dt: x must be 16-byte aligned");
  if (model_dtype == MI355GQ_BF16 && M > 1 && (K & 7) == 0 && aligned16(x)) {
    gq::GemmArgs g{};
    g.x = static_cast<const uint16_t*>(x);
    g.q_weight = static_cast<const uint32_t*>(q_weight);
    g.q_scale = static_cast<const uint16_t*>(q_scale);
    g.bias = static_cast<const uint16_t*>(bias);
    g.residual = static_cast<const uint16_t*>(residual);
    g.y = y;
    g.indptr = nullptr; g.indptr_i64 = 0;
    g.rows = M; g.N = N; g.K = K; g.num_experts = 1;
    g.bits = bits; g.group_size = group_size; g.out_f32 = out_dtype == MI355GQ_F32;
    g.workspace = workspace; g.workspace_bytes = workspace ? workspace_bytes : 0;
    g.bf16 = 1;
    g.paired = paired;
    // 9..16 rows of q4: the bfloat16 instance of the float16 linear's kernel for this range (ahead of the few-row kernels
    // below because a long K takes it from five rows on); K of one phase from 4 M
    // weights on (there is no bfloat16 skinny kernel: 6144 x 4096 at 16 rows 30.4 -> 10.8 us, 28672 x 4096 31.5 -> 20.3,
    // 128256 x 4096 105 -> 71, 4096 x 4096 12.2 -> 9.4, 2048 x 2048 9.4 -> 8.8)
    {
      const int gvm = gq::options().gemv_variant;
      const bool slices_ok = K > 4096 && workspace != nullptr && aligned16(workspace) &&
                             workspace_bytes >= gq::midrow_workspace_bytes(M, N, K) && gq::options().gemv_ksplit != 0;
      // (5..8 rows of a K beyond 8192 from 64 M weights on, as K slices, like the float16 linear: 8192 x 28672 at 5 / 8 rows
      //  49.1 / 50.6 -> 38.0 / 37.5 us, 5120 x 13824 23.1 / 23.7 -> 18.6 / 18.2; 4096 x 14336 15.5-16.3 against 15.7-16.1 stays)
      const bool mid_size =
          (M > 4 && M <= 8 && slices_ok && K > 8192 && N * K >= (64ll << 20)) ||
          (M > 8 && M <= 16 &&
           ((K <= 4096 && N * K >= (4ll << 20)) || (slices_ok && N * K >= (24ll << 20)) || (K <= 8192 && N * K >= (48ll << 20))));
      const bool mid_rows = bits == 4 && mid_size && gq::options().gemm_variant < 0 && gvm < 0 && (K & 255) == 0 && (N & 31) == 0;
      if (mid_rows || gvm == 10) {
        const hipError_t e = gq::launch_midrow(g, static_cast<int>(M), as_stream(stream));
        if (e != hipErrorNotSupported) return hip_result(e, "linear_dt mid-row launch");
      }
    }
    // up to 8 rows: the float16 path's quad-row kernels on the bf16 4x4x4 matrix instruction (x in registers where that
    // form applies, as in the float16 linear)
    if (M <= 8) {
      const int gvq = gq::options().gemv_variant;
      if (gq::options().gemm_variant < 0 && (gvq < 0 || gvq == 9)) {
        const hipError_t qr = gq::launch_quadreg(g, static_cast<int>(M), as_stream(stream));
        if (qr != hipErrorNotSupported) return hip_result(qr, "linear_dt quad-row (registers) launch");
      }
      const hipError_t q = gq::launch_quadrow(g, static_cast<int>(M), as_stream(stream));
      if (q != hipErrorNotSupported) return hip_result(q, "linear_dt quad-row launch");
    }
    // the float16 GEMM's tiles on the bf16 matrix instruction
    const hipError_t e = gq::launch_gemm(g, as_stream(stream));
    if (e != hipErrorNotSupported) return hip_result(e, "linear_dt gemm launch");
  }
  if (paired)
    return fail(MI355GQ_ERR_UNSUPPORTED, "linear_silu_mul_dt: no fused kernel for M=%lld N=%lld K=%lld (K %% 8 != 0?)",
                (long long)M, (long long)N, (long long)K);
  return hip_result(gq::launch_linear_dt(x, static_cast<const uint32_t*>(q_weight), q_scale, bias, residual, M, N, K,
                                         bits, group_size, model_dtype, out_dtype, y, as_stream(stream)),
                    "linear_dt launch");
}

int mi355gq_linear_dt(const void* x, const void* q_weight, const void* q_scale, const void* bias, int64_t M,
                      int64_t N, int64_t K, int bits, int group_size, int model_dtype, int out_dtype, void* y,
                      void* workspace, int64_t workspace_bytes, mi355gq_stream_t stream) {
  return linear_dt_impl(x, q_weight, q_scale, bias, nullptr, M, N, K, bits, group_size, model_dtype, out_dtype, y,
                        workspace, workspace_bytes, stream);
}

int64_t mi355gq_linear_silu_mul_dt_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits, int group_size,
                                                   int model_dtype) {
  if (model_dtype == MI355GQ_F16) return mi355gq_linear_silu_mul_workspace_bytes(M, N, K, bits, group_size);
  // (the GEMM's partial sums of the fused form need whole 32 + 32 column blocks; the K slices of the kernel on unscaled
  //  weight operands, 9..16 rows, do not)
  if ((N % 64) != 0)
    return (model_dtype == MI355GQ_BF16 && check_scheme(bits, group_size) == MI355GQ_OK && bits == 4 && M <= 16 &&
            (M > 8 || (M > 4 && K > 8192)) &&
            N > 0 && K > 0 && N < kMaxDim && K < kMaxDim && (N % 32) == 0)
               ? gq::midrow_workspace_bytes(M, N, K)
               : 0;
  return mi355gq_linear_dt_workspace_bytes(M, N, K, bits, group_size, model_dtype);
}

int mi355gq_linear_silu_mul_dt(const void* x, const void* q_weight, const void* q_scale, int64_t M, int64_t N,
                               int64_t K, int bits, int group_size, int model_dtype, void* y, void* workspace,
                               int64_t workspace_bytes, mi355gq_stream_t stream) {
  return linear_dt_impl(x, q_weight, q_scale, nullptr, nullptr, M, N, K, bits, group_size, model_dtype, model_dtype, y,
                        workspace, workspace_bytes, stream, true);
}

int mi355gq_linear_residual_dt(const void* x, const void* q_weight, const void* q_scale, const void* bias,
                               const void* residual, int64_t M, int64_t N, int64_t K, int bits, int group_size,
                               int model_dtype, int out_dtype, void* y, void* workspace, int64_t workspace_bytes,
                               mi355gq_stream_t stream) {
  GQ_REQUIRE(residual != nullptr || M == 0 || N == 0, "linear_residual_dt: residual is null");
  return linear_dt_impl(x, q_weight, q_scale, bias, residual, M, N, K, bits, group_size, model_dtype, out_dtype, y,
                        workspace, workspace_bytes, stream);
}

int mi355gq_moe_gemv(const void* x, int64_t x_rows, const void* q_weight, const void* q_scale,
                     const void* expert_ids, int64_t top_k, int64_t num_experts, int64_t N,
                     int64_t K, int bits, int group_size, void* out, mi355gq_stream_t stream) {
  return moe_gemv_impl(x, x_rows, q_weight, q_scale, expert_ids, top_k, num_experts, N, K, bits, group_size,
                       out, stream, false);
}

int mi355gq_moe_gemv_silu_mul(const void* x, int64_t x_rows, const void* q_weight, const void* q_scale,
                              const void* expert_ids, int64_t top_k, int64_t num_experts, int64_t N,
                              int64_t K, int bits, int group_size, void* out, mi355gq_stream_t stream) {
  return moe_gemv_impl(x, x_rows, q_weight, q_scale, expert_ids, top_k, num_experts, N, K, bits, group_size,
                       out, stream, true);
}

int mi355gq_moe_gemv_routed_silu_mul(const void* x, const void* gate_logits, int64_t num_experts, int64_t top_k,
                                     const void* q_weight, const void* q_scale, int64_t N, int64_t K, int bits,
                                     int group_size, int model_dtype, void* expert_weights, void* expert_ids, void* out,
                                     mi355gq_stream_t stream) {
  GQ_CHECK(check_model_dtype(model_dtype, "moe_gemv_routed_silu_mul"));
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(top_k >= 1 && N >= 0 && K >= 1 && N < kMaxDim && K < kMaxDim && num_experts >= top_k &&
                 num_experts < kMaxDim && (N & 1) == 0,
             "moe_gemv_routed_silu_mul: bad shape (N=%lld even, K=%lld, %lld experts, top_k=%lld)", (long long)N,
             (long long)K, (long long)num_experts, (long long)top_k);
  GQ_REQUIRE(x && gate_logits && q_weight && q_scale && expert_weights && expert_ids && (out || N == 0),
             "moe_gemv_routed_silu_mul: null pointer");
  if (model_dtype == MI355GQ_F32 || top_k > 2 || num_experts > 64 || !aligned16(x) || !aligned16(q_weight) ||
      !aligned2(gate_logits) || !aligned2(expert_weights) || !aligned4(expert_ids) || !aligned2(out))
    return fail(MI355GQ_ERR_UNSUPPORTED, "moe_gemv_routed_silu_mul: float16 / bfloat16 models, top_k <= 2, at most 64 "
                                         "experts, 16-byte aligned x and q_weight");
  if (N == 0) {  // nothing to multiply: the routing alone
    return hip_result(gq::launch_topk_softmax(gate_logits, 1, static_cast<int>(num_experts), static_cast<int>(top_k),
                                              expert_weights, static_cast<int32_t*>(expert_ids), model_dtype,
                                              as_stream(stream)),
                      "moe_gemv_routed_silu_mul routing launch");
  }
  gq::GemvArgs a{};
  a.x = static_cast<const uint16_t*>(x);
  a.q_weight = static_cast<const uint32_t*>(q_weight);
  a.q_scale = static_cast<const uint16_t*>(q_scale);
  a.bias = nullptr;
  a.y = out;
  a.expert_ids = nullptr;
  a.M = 1; a.N = N; a.K = K; a.slots = top_k; a.x_slot_stride = 0;
  a.num_experts = num_experts;
  a.bits = bits; a.group_size = group_size; a.out_f32 = 0; a.paired = 1;
  a.bf16 = model_dtype == MI355GQ_BF16;
  a.gate = gate_logits;
  a.route_w = expert_weights;
  a.route_ids = static_cast<int32_t*>(expert_ids);
  const hipError_t e = gq::launch_gemv(a, as_stream(stream));
  if (e == hipErrorNotSupported)
    return fail(MI355GQ_ERR_UNSUPPORTED, "moe_gemv_routed_silu_mul: no fused kernel for N=%lld K=%lld", (long long)N,
                (long long)K);
  return hip_result(e, "moe_gemv_routed_silu_mul launch");
}

int mi355gq_moe_gemv_combine(const void* x, const void* q_weight, const void* q_scale, int64_t N, int64_t K, int bits,
                             int group_size, int model_dtype, int64_t num_experts, const void* expert_ids,
                             const void* expert_weights, int64_t top_k, void* out, mi355gq_stream_t stream) {
  GQ_CHECK(check_model_dtype(model_dtype, "moe_gemv_combine"));
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(top_k >= 1 && N >= 0 && K >= 1 && N < kMaxDim && K < kMaxDim && num_experts >= 1 && num_experts < kMaxDim,
             "moe_gemv_combine: bad shape (N=%lld, K=%lld, %lld experts, top_k=%lld)", (long long)N, (long long)K,
             (long long)num_experts, (long long)top_k);
  GQ_REQUIRE(x && q_weight && q_scale && expert_ids && expert_weights && (out || N == 0), "moe_gemv_combine: null pointer");
  if (model_dtype == MI355GQ_F32 || top_k != 2 || (K & 7) != 0 || !aligned16(x) || !aligned16(q_weight) ||
      !aligned2(q_scale) || !aligned4(expert_ids) || !aligned2(expert_weights) || !aligned2(out))
    return fail(MI355GQ_ERR_UNSUPPORTED, "moe_gemv_combine: float16 / bfloat16 models, top_k = 2, K a multiple of 8, "
                                         "16-byte aligned x and q_weight");
  if (N == 0) return MI355GQ_OK;
  gq::GemvArgs a{};
  a.x = static_cast<const uint16_t*>(x);
  a.q_weight = static_cast<const uint32_t*>(q_weight);
  a.q_scale = static_cast<const uint16_t*>(q_scale);
  a.bias = nullptr;
  a.y = out;
  a.expert_ids = static_cast<const int32_t*>(expert_ids);
  a.M = 1; a.N = N; a.K = K; a.slots = top_k; a.x_slot_stride = K;
  a.num_experts = num_experts;
  a.bits = bits; a.group_size = group_size; a.out_f32 = 0; a.paired = 0;
  a.bf16 = model_dtype == MI355GQ_BF16;
  a.sum_weights = expert_weights;
  const hipError_t e = gq::launch_gemv(a, as_stream(stream));
  if (e == hipErrorNotSupported)
    return fail(MI355GQ_ERR_UNSUPPORTED, "moe_gemv_combine: no fused kernel for N=%lld K=%lld", (long long)N, (long long)K);
  return hip_result(e, "moe_gemv_combine launch");
}

// Expert-sorted rows, about one per expert: the register GEMV with one grid row per activation row streams an
// expert's weights once per row, the quad-row kernel once per expert but at well under half the GEMV's rate, so up
// to num_experts rows (about 1.5 rows per distinct expert under uniform routing) the GEMV is ahead or level.
// Measured on expert matmuls, quad-row -> GEMV: Mixtral-8x7B e1_e3 T=2 62 -> 38 us, T=4 116 -> 80, e2 35 -> 24 and
// 72 -> 40; Qwen2-MoE-57B shapes (64 experts, top-8) T=2 58 -> 33, T=4 83 -> 51; past num_experts rows the order flips
// (Mixtral T=6 132 -> 152).
static bool moe_rows_by_gemv(const gq::GemmArgs& g) {
  return g.rows <= (g.num_experts > 4 ? g.num_experts : 4) && g.rows <= 256 && g.num_experts <= 256 && (g.K & 7) == 0;
}

static hipError_t moe_row_gemv(const gq::GemmArgs& g, hipStream_t s) {
  gq::GemvArgs a{};
  a.x = g.x; a.q_weight = g.q_weight; a.q_scale = g.q_scale; a.bias = nullptr; a.y = g.y;
  a.expert_ids = nullptr;
  a.M = 1; a.N = g.N; a.K = g.K; a.slots = g.rows; a.x_slot_stride = 0; a.num_experts = g.num_experts;
  a.bits = g.bits; a.group_size = g.group_size; a.out_f32 = 0; a.paired = g.paired; a.bf16 = g.bf16;
  a.indptr = g.indptr; a.indptr_i64 = g.indptr_i64;
  a.x_row_index = g.x_rows; a.x_src_rows = g.x_rows ? g.x_src_rows : g.rows;
  return gq::launch_gemv(a, s);
}

// Expert segments on the kernel that scales the matrix instruction's result (gq_midrow.hip): rows per pass (16 or 32), or
// 0 where the quad-row kernel (fewer rows) or the GEMM's tiles (more) stay ahead.  A segment longer than a pass takes
// another pass over its expert's weights while the other experts' workgroups are done, so the bounds keep the longest
// segment inside one pass: with 8 experts 4 to 8 rows per expert on average for 16-row passes, with 64 experts (whose
// longest segment is further above the average: 12 at an average of 6, 17 at 9) 2 to 6; beyond that, up to 24 resp. 16 on
// average, the two-tile instance where K is one phase.  Measured, 8 experts x top-2 (Mixtral, e1_e3 / e2 in us): 24 tokens
// 156 / 102 -> 115 / 76, 32 tokens 170 / 106 -> 117 / 78, 16 tokens 118 / 75 against the quad-row kernel's 122 / 74, 40 tokens
// with 16-row passes 203 / 131 against the GEMM's 166 / 104; two tiles at 40 / 64 / 96 tokens 166 / 167 / 195 -> 140 / 143 / 153
// for e1_e3 (e2, K = 14336 in phases, 113-131 against 96-112: stays with the GEMM).  64 experts x top-6, 2816 x 2048 / 2048 x
// 1536 / 5120 x 3584 at 144..384 rows: 55-64 / 46-49 / 142-197 -> 51-53 / 34-35 / 142-145; at 576 rows (two tiles) 83 / 49 / 211
// -> 69 / 48 / 191.
static int midrow_rows_per_pass(int64_t rows, int64_t num_experts, int64_t K, int bits) {
  const int gv = gq::options().gemv_variant;
  if (gv == 10) return 16;  // (forced)
  if (gv == 11) return 32;
  if (gv >= 0 || bits != 4 || gq::options().gemm_variant >= 0) return 0;
  const bool many = num_experts > 16;
  const int64_t lo = (many ? 2 : 4) * num_experts, mid = (many ? 6 : 8) * num_experts,
                hi = (many ? 16 : 24) * num_experts;
  if (rows > lo && rows <= mid) return 16;
  if (rows > mid && rows <= hi && K <= 4096) return 32;
  return 0;
}

static int moe_group_gemm_impl(const void* x, int64_t rows, const void* q_weight, const void* q_scale,
                               const void* indptr, int indptr_dtype, int64_t num_experts, int64_t N,
                               int64_t K, int bits, int group_size, void* out, mi355gq_stream_t stream,
                               bool paired, const void* x_row_index = nullptr, int64_t x_rows = 0) {
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(rows >= 0 && N >= 0 && K >= 0 && rows < kMaxDim && N < kMaxDim && K < kMaxDim &&
                 num_experts > 0 && num_experts <= 65536,
             "moe_group_gemm: bad shape");
  GQ_REQUIRE(indptr_dtype == MI355GQ_I32 || indptr_dtype == MI355GQ_I64,
             "moe_group_gemm: indptr_dtype=%d", indptr_dtype);
  if (rows == 0 || N == 0) return MI355GQ_OK;
  GQ_REQUIRE(out && (K == 0 || (x && q_weight && q_scale && indptr)), "moe_group_gemm: null pointer");
  GQ_REQUIRE(aligned16(x) && aligned16(q_weight) && aligned16(out) &&
                 (indptr_dtype == MI355GQ_I32 ? aligned4(indptr)
                                              : (reinterpret_cast<uintptr_t>(indptr) & 7u) == 0),
             "moe_group_gemm: x, q_weight and out must be 16-byte aligned");
  GQ_REQUIRE(!paired || (N & 1) == 0, "moe_group_gemm_silu_mul: N=%lld must be even", (long long)N);
  if (K == 0) return launch_empty_k(nullptr, nullptr, out, rows, paired ? N / 2 : N, 0, as_stream(stream));
  gq::GemmArgs g{};
  g.x = static_cast<const uint16_t*>(x);
  g.q_weight = static_cast<const uint32_t*>(q_weight);
  g.q_scale = static_cast<const uint16_t*>(q_scale);
  g.bias = nullptr;
  g.y = out;
  g.indptr = indptr; g.indptr_i64 = indptr_dtype == MI355GQ_I64;
  g.rows = rows; g.N = N; g.K = K; g.num_experts = num_experts;
  g.bits = bits; g.group_size = group_size; g.out_f32 = 0; g.paired = paired;
  if (x_row_index != nullptr) {
    GQ_REQUIRE(x_rows >= 1 && x_rows < kMaxDim && aligned4(x_row_index), "moe_experts: x has %lld rows",
               (long long)x_rows);
    g.x_rows = static_cast<const int32_t*>(x_row_index);
    g.x_src_rows = x_rows;
  }
  // few rows in total: every expert is a skinny problem bound by streaming its weights
  const int gv = gq::options().gemv_variant;
  if (gv < 0 && moe_rows_by_gemv(g)) {
    const hipError_t e = moe_row_gemv(g, as_stream(stream));
    if (e != hipErrorNotSupported) return hip_result(e, "moe row GEMV launch");
    // (the unfused form may still take that kernel: the caller runs the two steps and the bits stay the same)
    if (paired) return fail(MI355GQ_ERR_UNSUPPORTED, "moe_group_gemm_silu_mul: no fused GEMV for N=%lld K=%lld",
                            (long long)N, (long long)K);
  }
  // (up to about seven rows per expert.  Mixtral layer, 8 experts, whole layer in us at 40 / 48 / 56 / 64 / 80 routed rows:
  //  this kernel 249 / 258 / 262 / 300 / 319, the GEMM's 32-row tiles 270 / 266 / 276 / 272 / 272, the skinny kernel
  //  282 / 292 / 301 / 307 / 343: the skinny kernel, once the step between the two, is behind both since the GEMM reads
  //  its scales in bulk, and only a forced variant runs it on expert segments.  The same rows per expert hold for many
  //  experts: 64 experts x top-6 (2048 x 1408 projections), whole layer at 144 / 192 / 288 / 384 / 432 routed rows
  //  112 / 115 / 117 / 127 / 142 us against 137 / 141 / 146 / 143 / 144 on the GEMM's tiles)
  if (const int per_pass = midrow_rows_per_pass(rows, num_experts, K, bits)) {
    const hipError_t q = gq::launch_midrow(g, per_pass, as_stream(stream));
    if (q != hipErrorNotSupported) return hip_result(q, "moe mid-row launch");
  }
  const int64_t quad_rows = 7 * num_experts > 32 ? 7 * num_experts : 32;
  if ((rows <= 128 || rows <= 8 * num_experts) && gq::options().gemm_variant != 1 &&
      ((gv < 0 && rows <= quad_rows) || (gv >= 6 && gv <= 8))) {
    const hipError_t q = gq::launch_quadrow(g, static_cast<int>(rows), as_stream(stream));
    if (q != hipErrorNotSupported) return hip_result(q, "moe quad-row launch");
  }
  if (rows <= 128 && rows <= 10 * num_experts && bits == 4 && gq::options().gemm_variant != 1 && gv >= 2 && gv <= 5) {
    const hipError_t e = gq::launch_skinny(g, static_cast<int>(rows), as_stream(stream));
    if (e != hipErrorNotSupported) return hip_result(e, "moe skinny launch");
  }
  const hipError_t e = gq::launch_gemm(g, as_stream(stream));
  if (paired && e == hipErrorNotSupported)
    return fail(MI355GQ_ERR_UNSUPPORTED, "moe_group_gemm_silu_mul: no fused kernel for N=%lld K=%lld",
                (long long)N, (long long)K);
  return hip_result(e, "moe_group_gemm launch");
}

int mi355gq_moe_group_gemm(const void* x, int64_t rows, const void* q_weight, const void* q_scale,
                           const void* indptr, int indptr_dtype, int64_t num_experts, int64_t N,
                           int64_t K, int bits, int group_size, void* out,
                           mi355gq_stream_t stream) {
  return moe_group_gemm_impl(x, rows, q_weight, q_scale, indptr, indptr_dtype, num_experts, N, K, bits,
                             group_size, out, stream, false);
}

int mi355gq_moe_group_gemm_silu_mul(const void* x, int64_t rows, const void* q_weight, const void* q_scale,
                                    const void* indptr, int indptr_dtype, int64_t num_experts, int64_t N,
                                    int64_t K, int bits, int group_size, void* out,
                                    mi355gq_stream_t stream) {
  return moe_group_gemm_impl(x, rows, q_weight, q_scale, indptr, indptr_dtype, num_experts, N, K, bits,
                             group_size, out, stream, true);
}

int mi355gq_moe_experts(const void* x, int64_t x_rows, const void* x_row_index, int64_t rows,
                        const void* q_weight, const void* q_scale, const void* indptr, int indptr_dtype,
                        int64_t num_experts, int64_t N, int64_t K, int bits, int group_size, int epilogue,
                        void* out, mi355gq_stream_t stream) {
  GQ_REQUIRE(epilogue == MI355GQ_EPILOGUE_NONE || epilogue == MI355GQ_EPILOGUE_SILU_MUL,
             "moe_experts: epilogue=%d", epilogue);
  GQ_REQUIRE(x_row_index != nullptr || x_rows == rows, "moe_experts: x has %lld rows, expected %lld",
             (long long)x_rows, (long long)rows);
  return moe_group_gemm_impl(x, rows, q_weight, q_scale, indptr, indptr_dtype, num_experts, N, K, bits,
                             group_size, out, stream, epilogue == MI355GQ_EPILOGUE_SILU_MUL, x_row_index,
                             x_rows);
}

static int moe_gemv_dt_impl(const void* x, int64_t x_rows, const void* q_weight, const void* q_scale,
                            const void* expert_ids, int64_t top_k, int64_t num_experts, int64_t N, int64_t K,
                            int bits, int group_size, int model_dtype, void* out, mi355gq_stream_t stream,
                            bool paired) {
  GQ_CHECK(check_model_dtype(model_dtype, "moe_gemv_dt"));
  if (model_dtype == MI355GQ_F16)
    return moe_gemv_impl(x, x_rows, q_weight, q_scale, expert_ids, top_k, num_experts, N, K, bits, group_size, out,
                         stream, paired);
  GQ_REQUIRE(!paired || (N & 1) == 0, "moe_gemv_silu_mul_dt: N=%lld must be even", (long long)N);
  if (paired && model_dtype != MI355GQ_BF16)
    return fail(MI355GQ_ERR_UNSUPPORTED, "moe_gemv_silu_mul_dt: no fused kernel for float32 models");
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(top_k >= 0 && top_k <= 65535 && N >= 0 && K >= 1 && N < kMaxDim && K < kMaxDim && num_experts > 0 &&
                 num_experts < kMaxDim,
             "moe_gemv_dt: bad shape");
  GQ_REQUIRE(x_rows == 1 || x_rows == top_k, "moe_gemv_dt: x has %lld rows, expected 1 or top_k=%lld",
             (long long)x_rows, (long long)top_k);
  if (top_k == 0 || N == 0) return MI355GQ_OK;
  GQ_REQUIRE(out && x && q_weight && q_scale && expert_ids, "moe_gemv_dt: null pointer");
  const bool f32 = model_dtype == MI355GQ_F32;
  GQ_REQUIRE(aligned16(q_weight) && aligned4(expert_ids) &&
                 (f32 ? aligned4(x) && aligned4(q_scale) && aligned4(out)
                      : aligned2(x) && aligned2(q_scale) && aligned2(out)),
             "moe_gemv_dt: q_weight must be 16-byte aligned, the other tensors naturally aligned");
  if (model_dtype == MI355GQ_BF16 && aligned16(x) && (x_rows == 1 || (K % 8) == 0)) {
    gq::GemvArgs a{};
    a.x = static_cast<const uint16_t*>(x);
    a.q_weight = static_cast<const uint32_t*>(q_weight);
    a.q_scale = static_cast<const uint16_t*>(q_scale);
    a.bias = nullptr;
    a.y = out;
    a.expert_ids = static_cast<const int32_t*>(expert_ids);
    a.M = 1; a.N = N; a.K = K; a.slots = top_k; a.x_slot_stride = x_rows == 1 ? 0 : K;
    a.num_experts = num_experts;
    a.bits = bits; a.group_size = group_size; a.out_f32 = 0;
    a.bf16 = 1;
    a.paired = paired;
    const hipError_t e = gq::launch_gemv(a, as_stream(stream));
    if (e != hipErrorNotSupported) return hip_result(e, "moe_gemv_dt gemv launch");
  }
  if (paired)
    return fail(MI355GQ_ERR_UNSUPPORTED, "moe_gemv_silu_mul_dt: no fused kernel for N=%lld K=%lld", (long long)N,
                (long long)K);
  return hip_result(gq::launch_moe_gemv_dt(x, x_rows == 1, static_cast<const uint32_t*>(q_weight), q_scale,
                                           static_cast<const int32_t*>(expert_ids), top_k, num_experts, N, K, bits,
                                           group_size, model_dtype, out, as_stream(stream)),
                    "moe_gemv_dt launch");
}

int mi355gq_moe_gemv_dt(const void* x, int64_t x_rows, const void* q_weight, const void* q_scale,
                        const void* expert_ids, int64_t top_k, int64_t num_experts, int64_t N, int64_t K, int bits,
                        int group_size, int model_dtype, void* out, mi355gq_stream_t stream) {
  return moe_gemv_dt_impl(x, x_rows, q_weight, q_scale, expert_ids, top_k, num_experts, N, K, bits, group_size,
                          model_dtype, out, stream, false);
}

int mi355gq_moe_gemv_silu_mul_dt(const void* x, int64_t x_rows, const void* q_weight, const void* q_scale,
                                 const void* expert_ids, int64_t top_k, int64_t num_experts, int64_t N, int64_t K,
                                 int bits, int group_size, int model_dtype, void* out, mi355gq_stream_t stream) {
  return moe_gemv_dt_impl(x, x_rows, q_weight, q_scale, expert_ids, top_k, num_experts, N, K, bits, group_size,
                          model_dtype, out, stream, true);
}

static int moe_group_gemm_dt_impl(const void* x, int64_t rows, const void* q_weight, const void* q_scale,
                                  const void* indptr, int indptr_dtype, int64_t num_experts, int64_t N, int64_t K,
                                  int bits, int group_size, int model_dtype, void* out, mi355gq_stream_t stream,
                                  bool paired, const void* x_row_index = nullptr, int64_t x_rows = 0) {
  GQ_CHECK(check_model_dtype(model_dtype, "moe_group_gemm_dt"));
  if (model_dtype == MI355GQ_F16)
    return moe_group_gemm_impl(x, rows, q_weight, q_scale, indptr, indptr_dtype, num_experts, N, K, bits,
                               group_size, out, stream, paired, x_row_index, x_rows);
  if (x_row_index != nullptr && model_dtype != MI355GQ_BF16)
    return fail(MI355GQ_ERR_UNSUPPORTED, "moe_experts_dt: the gather is folded in for float16 and bfloat16 models");
  GQ_REQUIRE(x_row_index == nullptr || (x_rows >= 1 && x_rows < kMaxDim && aligned4(x_row_index)),
             "moe_experts_dt: x has %lld rows", (long long)x_rows);
  GQ_REQUIRE(!paired || (N & 1) == 0, "moe_group_gemm_silu_mul_dt: N=%lld must be even", (long long)N);
  if (paired && model_dtype != MI355GQ_BF16)
    return fail(MI355GQ_ERR_UNSUPPORTED, "moe_group_gemm_silu_mul_dt: no fused kernel for float32 models");
  GQ_CHECK(check_scheme(bits, group_size));
  GQ_REQUIRE(rows >= 0 && N >= 0 && K >= 1 && rows < kMaxDim && N < kMaxDim && K < kMaxDim && num_experts > 0 &&
                 num_experts <= 65536,
             "moe_group_gemm_dt: bad shape");
  GQ_REQUIRE(indptr_dtype == MI355GQ_I32 || indptr_dtype == MI355GQ_I64, "moe_group_gemm_dt: indptr_dtype=%d",
             indptr_dtype);
  if (rows == 0 || N == 0) return MI355GQ_OK;
  GQ_REQUIRE(out && x && q_weight && q_scale && indptr, "moe_group_gemm_dt: null pointer");
  const bool f32 = model_dtype == MI355GQ_F32;
  GQ_REQUIRE(aligned16(q_weight) &&
                 (indptr_dtype == MI355GQ_I32 ? aligned4(indptr) : (reinterpret_cast<uintptr_t>(indptr) & 7u) == 0) &&
                 (f32 ? aligned4(x) && aligned4(q_scale) && aligned4(out)
                      : aligned2(x) && aligned2(q_scale) && aligned2(out)),
             "moe_group_gemm_dt: q_weight must be 16-byte aligned, the other tensors naturally aligned");
  if (model_dtype == MI355GQ_BF16 && rows > 1 && (K & 7) == 0 && aligned16(x) && aligned16(out)) {
    // the float16 grouped GEMM's tiles on the bf16 matrix instruction (as in linear_dt, faster than the
    // dot-product kernel from two rows on)
    gq::GemmArgs g{};
    g.x = static_cast<const uint16_t*>(x);
    g.q_weight = static_cast<const uint32_t*>(q_weight);
    g.q_scale = static_cast<const uint16_t*>(q_scale);
    g.y = out;
    g.indptr = indptr; g.indptr_i64 = indptr_dtype == MI355GQ_I64;
    g.rows = rows; g.N = N; g.K = K; g.num_experts = num_experts;
    g.bits = bits; g.group_size = group_size; g.out_f32 = 0;
    g.bf16 = 1;
    g.paired = paired;
    if (x_row_index != nullptr) {
      g.x_rows = static_cast<const int32_t*>(x_row_index);
      g.x_src_rows = x_rows;
    }
    if (gq::options().gemv_variant < 0 && moe_rows_by_gemv(g)) {  // about one row per expert (as in float16)
      const hipError_t e = moe_row_gemv(g, as_stream(stream));
      if (e != hipErrorNotSupported) return hip_result(e, "moe_group_gemm_dt row GEMV launch");
      if (paired) return fail(MI355GQ_ERR_UNSUPPORTED, "moe_group_gemm_silu_mul_dt: no fused GEMV for N=%lld K=%lld",
                              (long long)N, (long long)K);
    }
    // between the few-row kernel and the tiles: as in float16 (the bfloat16 instance)
    if (const int per_pass = midrow_rows_per_pass(rows, num_experts, K, bits)) {
      const hipError_t q = gq::launch_midrow(g, per_pass, as_stream(stream));
      if (q != hipErrorNotSupported) return hip_result(q, "moe_group_gemm_dt mid-row launch");
    }
    // few rows in total: every expert streams its weights for a handful of rows (as in float16)
    const int64_t quad_rows = 6 * num_experts > 32 ? 6 * num_experts : 32;
    if (rows <= quad_rows && rows <= 128) {
      const hipError_t q = gq::launch_quadrow(g, static_cast<int>(rows), as_stream(stream));
      if (q != hipErrorNotSupported) return hip_result(q, "moe_group_gemm_dt quad-row launch");
    }
    const hipError_t e = gq::launch_gemm(g, as_stream(stream));
    if (e != hipErrorNotSupported) return hip_result(e, "moe_group_gemm_dt gemm launch");
  }
  if (paired || x_row_index != nullptr)
    return fail(MI355GQ_ERR_UNSUPPORTED, "moe_group_gemm_dt: no fused kernel for N=%lld K=%lld (K %% 8 != 0?)",
                (long long)N, (long long)K);
  return hip_result(gq::launch_moe_group_gemm_dt(x, static_cast<const uint32_t*>(q_weight), q_scale, indptr,
                                                 indptr_dtype == MI355GQ_I64, rows, num_experts, N, K, bits,
                                                 group_size, model_dtype, out, as_stream(stream)),
                    "moe_group_gemm_dt launch");
}

int mi355gq_moe_group_gemm_dt(const void* x, int64_t rows, const void* q_weight, const void* q_scale,
                              const void* indptr, int indptr_dtype, int64_t num_experts, int64_t N, int64_t K,
                              int bits, int group_size, int model_dtype, void* out, mi355gq_stream_t stream) {
  return moe_group_gemm_dt_impl(x, rows, q_weight, q_scale, indptr, indptr_dtype, num_experts, N, K, bits,
                                group_size, model_dtype, out, stream, false);
}

int mi355gq_moe_group_gemm_silu_mul_dt(const void* x, int64_t rows, const void* q_weight, const void* q_scale,
                                       const void* indptr, int indptr_dtype, int64_t num_experts, int64_t N,
                                       int64_t K, int bits, int group_size, int model_dtype, void* out,
                                       mi355gq_stream_t stream) {
  return moe_group_gemm_dt_impl(x, rows, q_weight, q_scale, indptr, indptr_dtype, num_experts, N, K, bits,
                                group_size, model_dtype, out, stream, true);
}

static int gating_impl(const void* logits, int64_t T, int64_t num_experts, int64_t top_k, void* weights, void* ids,
                       int model_dtype, mi355gq_stream_t stream) {
  GQ_CHECK(check_model_dtype(model_dtype, "gating_softmax_topk"));
  GQ_REQUIRE(T >= 0 && T < kMaxDim, "gating_softmax_topk: bad T");
  GQ_REQUIRE(num_experts >= 1 && num_experts <= 256, "gating_softmax_topk: num_experts=%lld (1..256)",
             (long long)num_experts);
  GQ_REQUIRE(top_k >= 1 && top_k <= 8 && top_k <= num_experts,
             "gating_softmax_topk: top_k=%lld (1..min(8, num_experts))", (long long)top_k);
  if (T == 0) return MI355GQ_OK;
  GQ_REQUIRE(logits && weights && ids, "gating_softmax_topk: null pointer");
  return hip_result(gq::launch_topk_softmax(logits, T, static_cast<int>(num_experts), static_cast<int>(top_k), weights,
                                            static_cast<int32_t*>(ids), model_dtype, as_stream(stream)),
                    "gating_softmax_topk launch");
}

int mi355gq_moe_experts_dt(const void* x, int64_t x_rows, const void* x_row_index, int64_t rows, const void* q_weight,
                           const void* q_scale, const void* indptr, int indptr_dtype, int64_t num_experts, int64_t N,
                           int64_t K, int bits, int group_size, int epilogue, int model_dtype, void* out,
                           mi355gq_stream_t stream) {
  GQ_REQUIRE(epilogue == MI355GQ_EPILOGUE_NONE || epilogue == MI355GQ_EPILOGUE_SILU_MUL, "moe_experts_dt: epilogue=%d",
             epilogue);
  GQ_REQUIRE(x_row_index != nullptr || x_rows == rows, "moe_experts_dt: x has %lld rows, expected %lld",
             (long long)x_rows, (long long)rows);
  return moe_group_gemm_dt_impl(x, rows, q_weight, q_scale, indptr, indptr_dtype, num_experts, N, K, bits, group_size,
                                model_dtype, out, stream, epilogue == MI355GQ_EPILOGUE_SILU_MUL, x_row_index, x_rows);
}

int mi355gq_gating_softmax_topk(const void* logits, int64_t T, int64_t num_experts, int64_t top_k,
                                void* weights, void* ids, mi355gq_stream_t stream) {
  return gating_impl(logits, T, num_experts, top_k, weights, ids, MI355GQ_F16, stream);
}

int mi355gq_gating_softmax_topk_dt(const void* logits, int64_t T, int64_t num_experts, int64_t top_k, void* weights,
                                   void* ids, int model_dtype, mi355gq_stream_t stream) {
  return gating_impl(logits, T, num_experts, top_k, weights, ids, model_dtype, stream);
}

static int topk_scores_impl(const char* what, const void* x, int64_t T, int64_t num_experts, int64_t top_k,
                            void* out_scores, void* ids, int model_dtype, bool softmax_first,
                            mi355gq_stream_t stream) {
  GQ_CHECK(check_model_dtype(model_dtype, what));
  GQ_REQUIRE(T >= 0 && T < kMaxDim, "%s: bad T", what);
  GQ_REQUIRE(num_experts >= 1 && num_experts <= 65536, "%s: num_experts=%lld (1..65536)", what, (long long)num_experts);
  GQ_REQUIRE(top_k >= 1 && top_k <= 8 && top_k <= num_experts, "%s: top_k=%lld (1..min(8, num_experts))", what,
             (long long)top_k);
  if (T == 0) return MI355GQ_OK;
  GQ_REQUIRE(x && out_scores && ids, "%s: null pointer", what);
  GQ_REQUIRE(aligned4(ids) && (model_dtype == MI355GQ_F32 ? aligned4(x) && aligned4(out_scores)
                                                          : aligned2(x) && aligned2(out_scores)),
             "%s: misaligned tensor", what);
  return hip_result(gq::launch_topk_scores(x, T, static_cast<int>(num_experts), static_cast<int>(top_k), out_scores,
                                           static_cast<int32_t*>(ids), model_dtype, softmax_first, as_stream(stream)),
                    what);
}

int mi355gq_gating_topk(const void* scores, int64_t T, int64_t num_experts, int64_t top_k, void* out_scores,
                        void* ids, int model_dtype, mi355gq_stream_t stream) {
  return topk_scores_impl("gating_topk", scores, T, num_experts, top_k, out_scores, ids, model_dtype, false, stream);
}

int mi355gq_gating_softmax_topk_ex(const void* logits, int64_t T, int64_t num_experts, int64_t top_k,
                                   int norm_topk_prob, int model_dtype, void* weights, void* ids,
                                   mi355gq_stream_t stream) {
  if (norm_topk_prob) return gating_impl(logits, T, num_experts, top_k, weights, ids, model_dtype, stream);
  return topk_scores_impl("gating_softmax_topk_ex", logits, T, num_experts, top_k, weights, ids, model_dtype, true,
                          stream);
}

int mi355gq_moe_cumsum(const void* ids, int64_t T, int64_t top_k, int64_t num_experts,
                       void* cumsum, mi355gq_stream_t stream) {
  GQ_REQUIRE(T >= 0 && T < kMaxDim && top_k >= 1 && top_k <= 64, "moe_cumsum: bad shape");
  GQ_REQUIRE(num_experts >= 1 && num_experts <= 256, "moe_cumsum: num_experts=%lld (1..256)",
             (long long)num_experts);
  GQ_REQUIRE(T * num_experts < kMaxDim, "moe_cumsum: T * num_experts overflows int32");
  if (T == 0) return MI355GQ_OK;
  GQ_REQUIRE(ids && cumsum, "moe_cumsum: null pointer");
  return hip_result(gq::launch_moe_cumsum(static_cast<const int32_t*>(ids), T,
                                          static_cast<int>(top_k), static_cast<int>(num_experts),
                                          static_cast<int32_t*>(cumsum), as_stream(stream)),
                    "moe_cumsum launch");
}

int mi355gq_moe_get_indices(const void* cumsum, const void* ids, int64_t T, int64_t top_k,
                            int64_t num_experts, void* reverse_indices, void* token_indices,
                            mi355gq_stream_t stream) {
  GQ_REQUIRE(T >= 0 && T < kMaxDim && top_k >= 1 && top_k <= 64 && num_experts >= 1 &&
                 num_experts < kMaxDim && T * top_k < kMaxDim,
             "moe_get_indices: bad shape");
  if (T == 0) return MI355GQ_OK;
  GQ_REQUIRE(cumsum && ids && reverse_indices && token_indices, "moe_get_indices: null pointer");
  return hip_result(
      gq::launch_get_indices(static_cast<const int32_t*>(cumsum), static_cast<const int32_t*>(ids),
                             T, static_cast<int>(top_k), static_cast<int>(num_experts),
                             static_cast<int32_t*>(reverse_indices),
                             static_cast<int32_t*>(token_indices), as_stream(stream)),
      "moe_get_indices launch");
}

int mi355gq_moe_get_indptr(const void* cumsum, int64_t num_experts, int64_t T, int inclusive,
                           int out_dtype, void* indptr, mi355gq_stream_t stream) {
  GQ_REQUIRE(num_experts >= 1 && num_experts < kMaxDim && T >= 1 && T < kMaxDim,
             "moe_get_indptr: bad shape (needs T >= 1)");
  GQ_REQUIRE(out_dtype == MI355GQ_I32 || out_dtype == MI355GQ_I64, "moe_get_indptr: out_dtype=%d",
             out_dtype);
  GQ_REQUIRE(cumsum && indptr, "moe_get_indptr: null pointer");
  return hip_result(gq::launch_get_indptr(static_cast<const int32_t*>(cumsum), num_experts, T,
                                          inclusive != 0, out_dtype == MI355GQ_I64, indptr,
                                          as_stream(stream)),
                    "moe_get_indptr launch");
}

// rows of 2-byte elements are moved as they are; float32 rows as twice as many 2-byte units
static int move_rows_impl(const void* x, const void* indices, int64_t R, int64_t H, int64_t x_rows, void* out,
                          int scatter, int model_dtype, mi355gq_stream_t stream, const char* what) {
  GQ_CHECK(check_model_dtype(model_dtype, what));
  GQ_REQUIRE(R >= 0 && H >= 0 && x_rows >= 0 && R < kMaxDim && H < kMaxDim, "%s: bad shape", what);
  if (R == 0 || H == 0) return MI355GQ_OK;
  GQ_REQUIRE(x && indices && out, "%s: null pointer", what);
  const int64_t units = model_dtype == MI355GQ_F32 ? 2 * H : H;
  GQ_REQUIRE(model_dtype != MI355GQ_F32 || (aligned4(x) && aligned4(out)), "%s: misaligned float32 tensor", what);
  return hip_result(gq::launch_take_rows(static_cast<const uint16_t*>(x), static_cast<const int32_t*>(indices), R,
                                         units, x_rows, static_cast<uint16_t*>(out), scatter, as_stream(stream)),
                    what);
}

int mi355gq_take_rows(const void* x, const void* indices, int64_t R, int64_t H, int64_t x_rows,
                      void* out, mi355gq_stream_t stream) {
  return move_rows_impl(x, indices, R, H, x_rows, out, 0, MI355GQ_F16, stream, "take_rows");
}

int mi355gq_take_rows_dt(const void* x, const void* indices, int64_t R, int64_t H, int64_t x_rows, void* out,
                         int model_dtype, mi355gq_stream_t stream) {
  return move_rows_impl(x, indices, R, H, x_rows, out, 0, model_dtype, stream, "take_rows");
}

int mi355gq_moe_scatter_output(const void* x, const void* indices, int64_t R, int64_t H, void* out,
                               mi355gq_stream_t stream) {
  return move_rows_impl(x, indices, R, H, R, out, 1, MI355GQ_F16, stream, "moe_scatter_output");
}

int mi355gq_moe_scatter_output_dt(const void* x, const void* indices, int64_t R, int64_t H, void* out,
                                  int model_dtype, mi355gq_stream_t stream) {
  return move_rows_impl(x, indices, R, H, R, out, 1, model_dtype, stream, "moe_scatter_output");
}

static int silu_mul_impl(const void* x, int64_t R, int64_t I, void* out, int model_dtype, mi355gq_stream_t stream) {
  GQ_CHECK(check_model_dtype(model_dtype, "silu_mul"));
  GQ_REQUIRE(R >= 0 && I >= 0 && R < kMaxDim && I < kMaxDim, "silu_mul: bad shape");
  if (R == 0 || I == 0) return MI355GQ_OK;
  GQ_REQUIRE(x && out, "silu_mul: null pointer");
  return hip_result(gq::launch_silu_mul(x, R, I, out, model_dtype, as_stream(stream)), "silu_mul launch");
}

int mi355gq_silu_mul(const void* x, int64_t R, int64_t I, void* out, mi355gq_stream_t stream) {
  return silu_mul_impl(x, R, I, out, MI355GQ_F16, stream);
}

int mi355gq_silu_mul_dt(const void* x, int64_t R, int64_t I, void* out, int model_dtype, mi355gq_stream_t stream) {
  return silu_mul_impl(x, R, I, out, model_dtype, stream);
}

static int moe_combine_impl(const void* y, const void* weights, const void* positions, int64_t T,
                            int64_t top_k, int64_t H, void* out, int model_dtype, mi355gq_stream_t stream) {
  GQ_CHECK(check_model_dtype(model_dtype, "moe_combine"));
  GQ_REQUIRE(T >= 0 && H >= 0 && T < kMaxDim && H < kMaxDim && top_k >= 1 && top_k <= 64,
             "moe_combine: bad shape");
  if (T == 0 || H == 0) return MI355GQ_OK;
  GQ_REQUIRE(y && weights && out, "moe_combine: null pointer");
  return hip_result(gq::launch_moe_combine(y, weights, static_cast<const int32_t*>(positions), T,
                                           static_cast<int>(top_k), H, out, model_dtype, as_stream(stream)),
                    "moe_combine launch");
}

int mi355gq_moe_combine(const void* y, const void* weights, int64_t T, int64_t top_k, int64_t H,
                        void* out, mi355gq_stream_t stream) {
  return moe_combine_impl(y, weights, nullptr, T, top_k, H, out, MI355GQ_F16, stream);
}

int mi355gq_moe_combine_sorted(const void* y, const void* slot_positions, const void* weights, int64_t T,
                               int64_t top_k, int64_t H, void* out, mi355gq_stream_t stream) {
  GQ_REQUIRE(slot_positions != nullptr || T == 0, "moe_combine_sorted: slot_positions is null");
  return moe_combine_impl(y, weights, slot_positions, T, top_k, H, out, MI355GQ_F16, stream);
}

/* slot_positions null: y is in slot order (moe_combine); else the expert-sorted order (moe_combine_sorted) */
int mi355gq_moe_combine_dt(const void* y, const void* slot_positions, const void* weights, int64_t T, int64_t top_k,
                           int64_t H, void* out, int model_dtype, mi355gq_stream_t stream) {
  return moe_combine_impl(y, weights, slot_positions, T, top_k, H, out, model_dtype, stream);
}

static int moe_route_impl(const void* logits, int64_t T, int64_t num_experts, int64_t top_k, void* weights,
                          void* ids, void* token_indices, void* reverse_indices, void* slot_positions,
                          void* indptr, int indptr_dtype, int model_dtype, mi355gq_stream_t stream) {
  GQ_CHECK(check_model_dtype(model_dtype, "moe_route"));
  GQ_REQUIRE(T >= 0 && T < kMaxDim, "moe_route: bad T");
  GQ_REQUIRE(num_experts >= 1 && num_experts <= 256, "moe_route: num_experts=%lld (1..256)",
             (long long)num_experts);
  GQ_REQUIRE(top_k >= 1 && top_k <= 8 && top_k <= num_experts, "moe_route: top_k=%lld (1..min(8, num_experts))",
             (long long)top_k);
  GQ_REQUIRE(indptr_dtype == MI355GQ_I32 || indptr_dtype == MI355GQ_I64, "moe_route: indptr_dtype=%d",
             indptr_dtype);
  GQ_REQUIRE(indptr != nullptr, "moe_route: indptr is null");
  // one workgroup: by slot while the count table fits, else expert by expert while that is a handful of rounds
  const bool by_slot = gq::moe_route_by_slot(T, static_cast<int>(num_experts), static_cast<int>(top_k));
  if (!by_slot && (num_experts > 64 || T > 8192 || num_experts * ((T + 1023) / 1024) > 64))
    return fail(MI355GQ_ERR_UNSUPPORTED,
                "moe_route: T=%lld with %lld experts is past the single-workgroup form; run "
                "gating_softmax_topk, moe_cumsum, moe_get_indices and moe_get_indptr",
                (long long)T, (long long)num_experts);
  GQ_REQUIRE(T == 0 || (logits && weights && ids && token_indices && reverse_indices && slot_positions),
             "moe_route: null pointer");
  return hip_result(gq::launch_moe_route(logits, T, static_cast<int>(num_experts), static_cast<int>(top_k), weights,
                                         static_cast<int32_t*>(ids), static_cast<int32_t*>(token_indices),
                                         static_cast<int32_t*>(reverse_indices),
                                         static_cast<int32_t*>(slot_positions), indptr_dtype == MI355GQ_I64,
                                         indptr, model_dtype, as_stream(stream)),
                    "moe_route launch");
}

int mi355gq_moe_route(const void* logits, int64_t T, int64_t num_experts, int64_t top_k, void* weights,
                      void* ids, void* token_indices, void* reverse_indices, void* slot_positions,
                      void* indptr, int indptr_dtype, mi355gq_stream_t stream) {
  return moe_route_impl(logits, T, num_experts, top_k, weights, ids, token_indices, reverse_indices, slot_positions,
                        indptr, indptr_dtype, MI355GQ_F16, stream);
}

int mi355gq_moe_route_dt(const void* logits, int64_t T, int64_t num_experts, int64_t top_k, void* weights, void* ids,
                         void* token_indices, void* reverse_indices, void* slot_positions, void* indptr,
                         int indptr_dtype, int model_dtype, mi355gq_stream_t stream) {
  return moe_route_impl(logits, T, num_experts, top_k, weights, ids, token_indices, reverse_indices, slot_positions,
                        indptr, indptr_dtype, model_dtype, stream);
}

}  // extern "C"
