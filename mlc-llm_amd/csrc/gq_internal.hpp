// Internal launcher interface between the C ABI layer (gq_api.hip) and the kernel files.
// Launchers assume validated arguments and return the hipError_t of the launch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gq {

// Kernel forcing for tests and tuning sweeps.  The state is thread-local and defaults to "heuristics": only the
// thread that called the test hook (mi355gq_testing_set_option, declared in gq_testing.h and absent from the
// public header) ever sees anything else, so calls arriving on other threads cannot be steered by it.
struct Options {
  int gemv_rows_per_wave = -1;  // -1: heuristic
  int gemm_fast_loop = -1;      // 0: the pipelined GEMM always runs its general K loop (with the zero-selects and clamps)
  int quad_pairs = -1;          // -1: heuristic, 1 | 2: quads per item of the quad-row kernel
  int gemv_ksplit = -1;         // -1: heuristic, 0: never, 1: wherever it applies (register GEMV: two waves share a row's K)
  int quad_ksplit = -1;         // -1: heuristic, 0 | 1 | 2: log2 of the waves that share a quad set's K range
  int gemv_variant = -1;        // -1: heuristic, 0: LDS GEMV, 1: register GEMV, 2..5 skinny forms, 6..8 quad-row forms (x in LDS), 9: quad-row with x in registers
  int gemm_variant = -1;
  int gemv_waves = -1;          // total waves of a persistent GEMV / quad-row / skinny grid
  int gemm_split_k = -1;        // wanted workgroups of the few-row GEMM's split along K
};
Options& options();

// Records which kernel instantiation the calling thread launched last (thread-local text, read back through the
// test hook mi355gq_testing_last_kernel): measurement code names the kernel it timed from the run itself.
void note_kernel(const char* fmt, ...);

// hipFuncAttributeMaxDynamicSharedMemorySize = the CU's whole LDS, set once per (kernel, device) and remembered;
// kernels whose dynamic LDS may exceed 64 KiB call it before launching.
hipError_t allow_large_lds(const void* kernel);

struct GemvArgs {
  const uint16_t* x;        // [x_rows, K] fp16
  const uint32_t* q_weight; // [experts?, N, nw]
  const uint16_t* q_scale;  // [experts?, N, ng]
  const uint16_t* bias;     // [N] or null
  const uint16_t* residual = nullptr;  // [M, N] fp16 added to the result, or null (plain linear only)
  void* y;                  // [M or slots, N]
  const int32_t* expert_ids;  // null for a plain linear; else [slots]
  int64_t M;                // batch rows of a plain linear (1..8); 1 for MoE slots
  int64_t N, K;
  int64_t slots;            // 1 for a plain linear, top_k for MoE
  int64_t x_slot_stride;    // elements between x rows of consecutive slots (0 or K)
  int64_t num_experts;
  int bits, group_size;
  int out_f32;
  int paired = 0;           // fused gate/up form (see gate_up_row): y is [M or slots, N / 2] fp16; N even, no bias / residual
  int bf16 = 0;             // bfloat16 model: x, q_scale, bias, residual and a 16-bit y are bf16 (M <= 2, no fused form)
  // expert-sorted rows (slots = rows, M = 1, expert_ids null): the expert of a row comes from indptr
  // [num_experts + 1], its x row from x_row_index (null: the row itself)
  const void* indptr = nullptr;
  int indptr_i64 = 0;
  const int32_t* x_row_index = nullptr;
  int64_t x_src_rows = 0;
  // the token routes itself (expert_ids null, slots = top_k <= 2, num_experts <= 64): router logits in the model dtype,
  // and where the chosen ids / softmax weights go
  const void* gate = nullptr;
  void* route_w = nullptr;
  int32_t* route_ids = nullptr;
  // one token's two expert slots summed with their routing weights in the same launch (slots = 2, expert_ids set, y is
  // [1, N] in the model dtype): the two weights, model dtype
  const void* sum_weights = nullptr;
};
hipError_t launch_gemv(const GemvArgs& a, hipStream_t s);

struct GemmArgs {
  const uint16_t* x;        // [rows, K]
  const uint32_t* q_weight; // [experts, N, nw]
  const uint16_t* q_scale;  // [experts, N, ng]
  const uint16_t* bias;     // [N] or null (plain linear only)
  const uint16_t* residual = nullptr;  // [rows, N] fp16 added to the result, or null (plain linear only)
  void* y;                  // [rows, N]
  const void* indptr;       // null for a plain linear
  int indptr_i64;
  int64_t rows, N, K, num_experts;
  int bits, group_size, out_f32;
  void* workspace = nullptr;       // caller's scratch for split-K partial sums (may be null)
  int64_t workspace_bytes = 0;
  int paired = 0;                  // fused gate/up form: y is [rows, N / 2] fp16; N even, no bias / residual
  const int32_t* x_rows = nullptr; // the MoE gather folded in: activation row r reads x[x_rows[r]] (x has x_src_rows rows)
  int64_t x_src_rows = 0;
  int bf16 = 0;                    // bfloat16 model: x, q_scale, bias and a 16-bit y are bf16 (plain linear only)
};
hipError_t launch_gemm(const GemmArgs& a, hipStream_t s);
// scratch the split-K form of the GEMM wants for this shape (0 when it does not split)
int64_t gemm_workspace_bytes(int64_t rows, int64_t N, int64_t K, int bits, int group_size);
// MFMA kernel for few activation rows per segment (q4 only; hipErrorNotSupported otherwise).
// rows_max bounds the rows of any one segment.
hipError_t launch_skinny(const GemmArgs& a, int rows_max, hipStream_t s);
// 4x4x4-MFMA kernel with GEMV-like weight streaming (q4, activations resident in LDS);
// hipErrorNotSupported when the shape does not fit.
hipError_t launch_quadrow(const GemmArgs& a, int rows_max, hipStream_t s);

// the same matrix instruction with the activations resident in registers (plain linears of up to 8 float16 rows);
// hipErrorNotSupported when the shape does not fit.
hipError_t launch_quadreg(const GemmArgs& a, int rows_max, hipStream_t s);

// 16x16x32 matrix instruction on unscaled weight operands, the scale applied per group afterwards (q4f16_1, K % 256 == 0;
// plain linears and expert segments); rows_max bounds the rows of any one segment; hipErrorNotSupported when the shape
// does not fit.
hipError_t launch_midrow(const GemmArgs& a, int rows_max, hipStream_t s);
int64_t midrow_workspace_bytes(int64_t rows, int64_t N, int64_t K);

// KN-layout tensors (q_weight [nw, N], q_scale [ng, N]): both tensors transposed in one call (src_rows_w / src_rows_s rows
// of src_cols columns each), the dequantisation to [K, N], and the decode GEMV (M <= 8, N % 4 == 0) with its workspace
hipError_t launch_kn_transpose(const uint32_t* qw_src, const uint16_t* qs_src, int64_t src_rows_w, int64_t src_rows_s,
                               int64_t src_cols, uint32_t* qw_dst, uint16_t* qs_dst, hipStream_t s);
hipError_t launch_dequantize_kn(const uint32_t* qw, const uint16_t* qs, int64_t N, int64_t K, int bits, uint16_t* out,
                                hipStream_t s);
int64_t gemv_kn_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits);
hipError_t launch_gemv_kn(const uint16_t* x, const uint32_t* qw, const uint16_t* qs, const uint16_t* bias, int64_t M,
                          int64_t N, int64_t K, int bits, int out_f32, void* y, void* workspace, int64_t workspace_bytes,
                          hipStream_t s);

// plain streaming read of two byte ranges (multiples of 16 bytes, 16-byte aligned)
hipError_t launch_stream_read(const void* a, int64_t a_bytes, const void* b, int64_t b_bytes,
                              void* sink, hipStream_t s);

// model dtypes beyond float16 (values of the public enum: MI355GQ_F16 = 0, MI355GQ_F32 = 1, MI355GQ_BF16 = 2)
constexpr int MODEL_F16 = 0, MODEL_F32 = 1, MODEL_BF16 = 2;
hipError_t launch_quantize_dt(const void* w, int64_t rows, int64_t K, int bits, int group_size, int round_mode,
                              int model_dtype, uint32_t* qw, void* qs, hipStream_t s);
hipError_t launch_dequantize_dt(const int32_t* ids, int64_t out_rows, const uint32_t* qw, const void* qs,
                                int64_t table_rows, int64_t K, int bits, int group_size, int model_dtype,
                                void* out, hipStream_t s);
// out_kind: MODEL_F32 or MODEL_BF16
hipError_t launch_linear_dt(const void* x, const uint32_t* qw, const void* qs, const void* bias, const void* residual,
                            int64_t M, int64_t N, int64_t K, int bits, int group_size, int model_dtype, int out_kind,
                            void* y, hipStream_t s);
// the two expert matmuls over stacked q_weight / q_scale, everything else in model_dtype
hipError_t launch_moe_gemv_dt(const void* x, bool x_one_row, const uint32_t* qw, const void* qs, const int32_t* ids,
                              int64_t slots, int64_t num_experts, int64_t N, int64_t K, int bits, int group_size,
                              int model_dtype, void* y, hipStream_t s);
hipError_t launch_moe_group_gemm_dt(const void* x, const uint32_t* qw, const void* qs, const void* indptr,
                                    bool indptr_i64, int64_t rows, int64_t num_experts, int64_t N, int64_t K,
                                    int bits, int group_size, int model_dtype, void* y, hipStream_t s);
hipError_t launch_quantize(const uint16_t* w, int64_t rows, int64_t K, int bits, int group_size,
                           int round_mode, uint32_t* qw, uint16_t* qs, hipStream_t s);
hipError_t launch_dequantize(const int32_t* ids, int64_t out_rows, const uint32_t* qw,
                             const uint16_t* qs, int64_t table_rows, int64_t K, int bits,
                             int group_size, uint16_t* out, hipStream_t s);

// (logits, weights, activations of the routing glue carry model_dtype: MODEL_F16 | MODEL_F32 | MODEL_BF16)
hipError_t launch_topk_softmax(const void* logits, int64_t T, int ne, int k, void* w, int32_t* ids, int model_dtype,
                               hipStream_t s);
// gating_topk on given scores, or (softmax_first) fp32 softmax over all experts rounded to the dtype, then that top-k
hipError_t launch_topk_scores(const void* x, int64_t T, int ne, int k, void* w, int32_t* ids, int model_dtype,
                              bool softmax_first, hipStream_t s);
hipError_t launch_moe_cumsum(const int32_t* ids, int64_t T, int k, int ne, int32_t* cumsum,
                             hipStream_t s);
hipError_t launch_get_indices(const int32_t* cumsum, const int32_t* ids, int64_t T, int k, int ne,
                              int32_t* rev, int32_t* tok, hipStream_t s);
hipError_t launch_get_indptr(const int32_t* cumsum, int64_t ne, int64_t T, int inclusive,
                             int out_i64, void* indptr, hipStream_t s);
hipError_t launch_take_rows(const uint16_t* x, const int32_t* idx, int64_t R, int64_t H,
                            int64_t x_rows, uint16_t* out, int scatter, hipStream_t s);
hipError_t launch_silu_mul(const void* x, int64_t R, int64_t I, void* out, int model_dtype, hipStream_t s);
hipError_t launch_moe_combine(const void* y, const void* w, const int32_t* pos, int64_t T, int k, int64_t H,
                              void* out, int model_dtype, hipStream_t s);
// fused routing for batches one workgroup can scan (the caller checks T and the expert count)
bool moe_route_by_slot(int64_t T, int ne, int k);  // the single-workgroup route step has its slot-organised form
hipError_t launch_moe_route(const void* logits, int64_t T, int ne, int k, void* w, int32_t* ids, int32_t* tok,
                            int32_t* rev, int32_t* pos_of_slot, int out_i64, void* indptr, int model_dtype,
                            hipStream_t s);

}  // namespace gq
