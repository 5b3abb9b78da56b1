/*
 * mi355gq — MI355X (gfx950) kernels for MLC-LLM group-quantized weights, C ABI.
 *
 * Every entry point takes raw device pointers, sizes and a hipStream_t (passed
 * as void*), launches asynchronously on that stream and returns MI355GQ_OK or a
 * negative code; mi355gq_last_error() then holds a thread-local message.
 * The library holds no process-wide mutable state (a per-device record of kernel attributes already set aside):
 * entry points may be called from any thread.
 * Nothing allocates, nothing retains pointers, nothing synchronises: outputs
 * (and workspaces, where named) are owned by the caller, exactly as Relax
 * `call_dps_packed` hands them over (destination-passing style, see the
 * reference's python/mlc_llm/op/ft_gemm.py:72-92 and op/cutlass.py:71-77).
 *
 * Layouts are the reference's, unchanged (python/mlc_llm/quantization/
 * group_quantization.py:342-347, 574-580): NK layout,
 *   q_weight uint32 [N, nw]  nw = (G / E) * ceil(K / G),  E = 32 / bits
 *   q_scale  fp16   [N, ng]  ng = ceil(K / G)
 * q4f16_1: bits = 4, G = 32;  q3f16_1: bits = 3, G = 40.  fp16 = IEEE binary16.
 * All tensors are dense row-major; q_weight rows must be 16-byte aligned
 * (always true for a 16-byte aligned base because nw is a multiple of 4).
 */
#ifndef MI355GQ_H_
#define MI355GQ_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define MI355GQ_API __attribute__((visibility("default")))
#else
#define MI355GQ_API
#endif

#define MI355GQ_VERSION 100

enum {
  MI355GQ_OK = 0,
  MI355GQ_ERR_ARG = -1,         /* bad pointer / size / scheme / alignment */
  MI355GQ_ERR_HIP = -2,         /* a HIP call failed; message holds hipGetErrorString */
  MI355GQ_ERR_UNSUPPORTED = -3, /* valid request this build has no kernel for */
  MI355GQ_ERR_WORKSPACE = -4    /* caller's workspace is too small */
};

enum { MI355GQ_F16 = 0, MI355GQ_F32 = 1, MI355GQ_BF16 = 2 }; /* output dtype (F16 / F32); model dtype of the *_dt entry points */
enum { MI355GQ_ROUND_HALF_AWAY = 0, MI355GQ_ROUND_HALF_EVEN = 1 };
enum { MI355GQ_I32 = 0, MI355GQ_I64 = 1 };             /* indptr dtype */

typedef void* mi355gq_stream_t; /* hipStream_t */

MI355GQ_API int mi355gq_version(void);
/* Thread-local message of the last failing call on this thread ("" if none). */
MI355GQ_API const char* mi355gq_last_error(void);
/* 0 when the current HIP device is gfx950, MI355GQ_ERR_UNSUPPORTED otherwise. */
MI355GQ_API int mi355gq_check_device(void);

/*
 * GroupQuantize.quantize_weight, NK layout (replaces the Relax function built at
 * python/mlc_llm/quantization/group_quantization.py:188-306 and utils.py:136-188).
 * w fp16 [rows, K] -> q_weight uint32 [rows, nw], q_scale fp16 [rows, ng]. Bit-exact.
 */
MI355GQ_API int mi355gq_quantize(const void* w, int64_t rows, int64_t K, int bits, int group_size,
                     int round_mode, void* q_weight, void* q_scale, mi355gq_stream_t stream);

/*
 * GroupQuantize._dequantize (group_quantization.py:155-186, utils.py:15-48):
 * out fp16 [rows, K] = (unpack(q_weight) - m) * q_scale, evaluated for k < K only. Bit-exact.
 */
MI355GQ_API int mi355gq_dequantize(const void* q_weight, const void* q_scale, int64_t rows, int64_t K,
                       int bits, int group_size, void* out, mi355gq_stream_t stream);

/*
 * GroupQuantizeEmbedding.forward (group_quantization.py:486-522, fused by
 * compiler_pass/fuse_dequantize_take.py:14-49): out fp16 [T, K] = dequantize(row ids[t]).
 * ids int32 [T], each in [0, num_rows) (not checked on the device: out-of-range ids are
 * clamped to the table like a safe gather, never read out of bounds).
 */
MI355GQ_API int mi355gq_embedding_take(const void* ids, int64_t T, const void* q_weight, const void* q_scale,
                           int64_t num_rows, int64_t K, int bits, int group_size, void* out,
                           mi355gq_stream_t stream);

/*
 * The three packing entry points above for the other model dtypes of the reference registry
 * (quantization/quantization.py:91-123: q4bf16_0 / q4bf16_1 with model_dtype bfloat16, q4f32_1 with
 * float32): `GroupQuantize` carries `model_dtype` through _quantize / _dequantize
 * (group_quantization.py:235-306, 155-186), so w, q_scale, out and every intermediate have that type.
 * model_dtype MI355GQ_F16 forwards to the float16 entry points; MI355GQ_F32 is IEEE single arithmetic
 * op for op; MI355GQ_BF16 does each operation in float32 and rounds the result to nearest-even
 * bfloat16 (TVM's bf16 legalisation).  q_weight layout is that of the float16 schemes.  Tensors need
 * only their natural alignment.
 */
MI355GQ_API int mi355gq_quantize_dt(const void* w, int64_t rows, int64_t K, int bits, int group_size,
                        int round_mode, int model_dtype, void* q_weight, void* q_scale,
                        mi355gq_stream_t stream);
MI355GQ_API int mi355gq_dequantize_dt(const void* q_weight, const void* q_scale, int64_t rows, int64_t K,
                          int bits, int group_size, int model_dtype, void* out, mi355gq_stream_t stream);
MI355GQ_API int mi355gq_embedding_take_dt(const void* ids, int64_t T, const void* q_weight,
                              const void* q_scale, int64_t num_rows, int64_t K, int bits, int group_size,
                              int model_dtype, void* out, mi355gq_stream_t stream);

/*
 * GroupQuantizeLinear.forward / GroupQuantizeEmbedding.lm_head_forward
 * (group_quantization.py:390-437, 524-556), i.e. the fused_dequantize*_NT_matmul kernels
 * (compiler_pass/fuse_dequantize_matmul_ewise.py, fuse_transpose_matmul.py:64-143):
 *   y[M, N] = x[M, K] . dequantize(q_weight, q_scale)[N, K]^T (+ bias[N])
 * x fp16, bias fp16 or NULL, y fp16 (MI355GQ_F16) or fp32 (MI355GQ_F32); fp32 accumulation.
 * M <= 8 runs the decode GEMV / few-row kernels, larger M the MFMA GEMM (the regime split of
 * compiler_pass/low_batch_specialization.py:22-57).
 * workspace: device scratch, 16-byte aligned, of at least mi355gq_linear_workspace_bytes()
 * bytes for the shape; the GEMM with 17..256 rows asks for some (fp32 partial sums of its
 * split along K), and so does q4 at 9..32 rows with K beyond 4096 and at 5..8 rows with K beyond
 * 8192 (partial sums of K slices that run on separate workgroups).  NULL or too small is not an error: the shape runs unsplit, slower.
 * Its contents are undefined afterwards; calls that share a workspace must be stream-ordered.
 */
MI355GQ_API int64_t mi355gq_linear_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits, int group_size);
MI355GQ_API int mi355gq_linear(const void* x, const void* q_weight, const void* q_scale, const void* bias,
                   int64_t M, int64_t N, int64_t K, int bits, int group_size, int out_dtype,
                   void* y, void* workspace, int64_t workspace_bytes, mi355gq_stream_t stream);

/*
 * mi355gq_linear for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose VM allocates workspaces
 * itself.  Same arguments and results as mi355gq_linear without the workspace: the partial sums of a split
 * along K go to a device array inside the library (mi355gq_linear_static_scratch_max_bytes() = 32 MiB, held
 * by every GPU the library runs on until the process ends), so the call allocates nothing.  Shapes whose split
 * would want more return MI355GQ_ERR_WORKSPACE (nothing is launched); the K slices of 5..32 rows are dropped first
 * where only their sums do not fit (the shape then runs as it does without a workspace for them).  All calls on one GPU share the array:
 * calls that overlap on one GPU (different streams, different threads) race on it; stream-ordered calls do not.
 * The first use on a device looks the array's address up (and may load it with the code object): call
 * mi355gq_linear_static_scratch_init() once per device, with that device current, before a region that must not
 * allocate or that is being captured; later calls only read the kept address.
 */
MI355GQ_API int64_t mi355gq_linear_static_scratch_max_bytes(void);
MI355GQ_API int mi355gq_linear_static_scratch_init(void);
MI355GQ_API int mi355gq_linear_static_scratch(const void* x, const void* q_weight, const void* q_scale,
                                  const void* bias, int64_t M, int64_t N, int64_t K, int bits, int group_size,
                                  int out_dtype, void* y, mi355gq_stream_t stream);

/*
 * KN-layout schemes (q4f16_0, q3f16_0, q4bf16_0 of quantization/quantization.py:47-57, 69-79): quantize_weight with
 * output_transpose stores the transposed tensors (group_quantization.py:125-130, 299-305),
 *   q_weight uint32 [nw, N],  q_scale fp16 [ng, N],
 * and GroupQuantizeLinear.forward dequantises along axis 0 and multiplies without a transpose (:404-437).
 * mi355gq_linear_kn is mi355gq_linear on those tensors as stored: up to 8 rows (N a multiple of 4) run a GEMV that
 * streams them in place (its split along K keeps fp32 partial sums in the workspace; without one it runs unsplit,
 * slower); every other shape runs the NK kernels on an NK copy made in the workspace, which must then hold
 * mi355gq_linear_kn_workspace_bytes() bytes, 16-byte aligned (MI355GQ_ERR_WORKSPACE otherwise).
 * mi355gq_kn_to_nk / mi355gq_nk_to_kn move both tensors between the layouts (bit moves: a caller that keeps converted
 * q4f16_0 weights can make the NK tensors once and use every other entry point); mi355gq_dequantize_kn is
 * GroupQuantize._dequantize with axis 0: out fp16 [K, N].  float16 models.
 */
MI355GQ_API int mi355gq_kn_to_nk(const void* q_weight_kn, const void* q_scale_kn, int64_t N, int64_t K, int bits,
                     int group_size, void* q_weight_nk, void* q_scale_nk, mi355gq_stream_t stream);
MI355GQ_API int mi355gq_nk_to_kn(const void* q_weight_nk, const void* q_scale_nk, int64_t N, int64_t K, int bits,
                     int group_size, void* q_weight_kn, void* q_scale_kn, mi355gq_stream_t stream);
MI355GQ_API int mi355gq_dequantize_kn(const void* q_weight, const void* q_scale, int64_t N, int64_t K, int bits,
                          int group_size, void* out, mi355gq_stream_t stream);
MI355GQ_API int64_t mi355gq_linear_kn_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits, int group_size);
MI355GQ_API int mi355gq_linear_kn(const void* x, const void* q_weight, const void* q_scale, const void* bias, int64_t M,
                      int64_t N, int64_t K, int bits, int group_size, int out_dtype, void* y, void* workspace,
                      int64_t workspace_bytes, mi355gq_stream_t stream);

/*
 * The same linear with the element-wise tail the reference folds into the matmul kernel:
 * FuseDequantizeMatmulEwise (compiler_pass/fuse_dequantize_matmul_ewise.py:19-32) fuses the
 * dequantize + matmul pair together with up to three element-wise operands that operator fusion
 * attached to the matmul, which for a decoder layer is the residual addition after o_proj and
 * after down_proj (model/llama/llama_model.py:204-215):
 *   y[M, N] = x . W^T (+ bias[N]) + residual[M, N]
 * residual is fp16; it may be y itself when y is fp16 (hidden += proj(x)): every element is read
 * before it is written, by the same lane.  Accumulation and both additions are fp32, rounded once.
 */
MI355GQ_API int mi355gq_linear_residual(const void* x, const void* q_weight, const void* q_scale,
                            const void* bias, const void* residual, int64_t M, int64_t N, int64_t K,
                            int bits, int group_size, int out_dtype, void* y, void* workspace,
                            int64_t workspace_bytes, mi355gq_stream_t stream);

/*
 * mi355gq_linear for the other model dtypes (see mi355gq_quantize_dt): x, q_scale and bias carry
 * model_dtype (MI355GQ_F32 or MI355GQ_BF16; MI355GQ_F16 forwards to mi355gq_linear), y carries
 * out_dtype = model_dtype or MI355GQ_F32.  Weights are dequantised as GroupQuantize._dequantize does
 * ((q - m) * scale rounded to the model dtype) and accumulated in fp32.  Exception: up to 8 bfloat16 rows run the
 * float16 path's register GEMV / quad-row kernel, which scale each group's integer dot product in fp32 and so skip
 * that per-weight rounding (as mi355gq_linear does for float16).  No SiLU epilogue.
 * workspace: device scratch of at least mi355gq_linear_dt_workspace_bytes(M, N, K, ...) bytes, 16-byte aligned,
 * or null (then few-row bfloat16 matmuls run unsplit: slower, same result up to summation order).
 */
/* mi355gq_linear_residual for the other model dtypes: residual [M, N] carries model_dtype (it may be y itself when
 * out_dtype == model_dtype). */
MI355GQ_API int mi355gq_linear_residual_dt(const void* x, const void* q_weight, const void* q_scale, const void* bias,
                               const void* residual, int64_t M, int64_t N, int64_t K, int bits,
                               int group_size, int model_dtype, int out_dtype, void* y, void* workspace,
                               int64_t workspace_bytes, mi355gq_stream_t stream);
MI355GQ_API int64_t mi355gq_linear_dt_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits, int group_size,
                                          int model_dtype);
MI355GQ_API int mi355gq_linear_dt(const void* x, const void* q_weight, const void* q_scale, const void* bias,
                      int64_t M, int64_t N, int64_t K, int bits, int group_size, int model_dtype,
                      int out_dtype, void* y, void* workspace, int64_t workspace_bytes,
                      mi355gq_stream_t stream);

/*
 * gate_up projection with the activation folded in: the sequence
 *   x1, x2 = split(gate_up_proj(x), 2, axis=-1); silu(x1) * x2
 * of the MLP (model/llama/llama_model.py:122-125; for the experts model/mixtral/mixtral_model.py:64-68),
 * the element-wise tail the FasterTransformer precedent folds into its matmul as an `activation`
 * argument (op/ft_gemm.py:72-92).  q_weight / q_scale are the unchanged [N, ...] tensors whose first
 * N / 2 rows are the gate and last N / 2 rows the up projection:
 *   y[M, N / 2] = silu(x . W[j]^T) * (x . W[N / 2 + j]^T),  y fp16
 * with the rounding points of the unfused sequence (fp16 matmul outputs, silu evaluated in fp32 and
 * rounded to fp16, fp16 product), so the result equals mi355gq_linear followed by mi355gq_silu_mul
 * bit for bit while the [M, N] intermediate never reaches memory.  N must be even.
 * Returns MI355GQ_ERR_UNSUPPORTED for shapes no fused kernel takes (K not a multiple of 8; the
 * caller then runs the two calls).  workspace as for mi355gq_linear, sized by
 * mi355gq_linear_silu_mul_workspace_bytes().
 */
MI355GQ_API int64_t mi355gq_linear_silu_mul_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits,
                                                            int group_size);
MI355GQ_API int mi355gq_linear_silu_mul(const void* x, const void* q_weight, const void* q_scale, int64_t M,
                            int64_t N, int64_t K, int bits, int group_size, void* y, void* workspace,
                            int64_t workspace_bytes, mi355gq_stream_t stream);

/*
 * moe_matmul.dequantize_gemv (python/mlc_llm/op/moe_matmul.py:77-176), single-token MoE:
 *   out[e, :] = x[x_rows == 1 ? 0 : e, :] . dequantize(W[expert_ids[e]])^T,  e < top_k
 * x fp16 [x_rows, K] with x_rows in {1, top_k}; expert_ids int32 [1, top_k];
 * q_weight uint32 [num_experts, N, nw]; q_scale fp16 [num_experts, N, ng]; out fp16 [top_k, N].
 */
MI355GQ_API int mi355gq_moe_gemv(const void* x, int64_t x_rows, const void* q_weight, const void* q_scale,
                     const void* expert_ids, int64_t top_k, int64_t num_experts, int64_t N,
                     int64_t K, int bits, int group_size, void* out, mi355gq_stream_t stream);

/*
 * moe_matmul.dequantize_group_gemm (op/moe_matmul.py:562-768):
 *   out[r, :] = x[r, :] . dequantize(W[e])^T  for indptr[e] <= r < indptr[e+1]
 * x fp16 [rows, K] already gathered in expert order; indptr [num_experts + 1], int32 or int64
 * (indptr[0] = 0); out fp16 [rows, N].  Rows outside every segment are left untouched.
 */
MI355GQ_API int mi355gq_moe_group_gemm(const void* x, int64_t rows, const void* q_weight, const void* q_scale,
                           const void* indptr, int indptr_dtype, int64_t num_experts, int64_t N,
                           int64_t K, int bits, int group_size, void* out,
                           mi355gq_stream_t stream);

/*
 * mi355gq_moe_gemv / mi355gq_moe_group_gemm for the other model dtypes (GroupQuantizeMixtralExperts.forward,
 * quantization/group_quantization.py:619-660, under q4f32_1 / q4bf16_*): x, q_scale and out carry model_dtype
 * (MI355GQ_F32 or MI355GQ_BF16; MI355GQ_F16 forwards to the entries above); weights are dequantised as
 * GroupQuantize._dequantize does and accumulated in fp32.  K >= 1.
 */
MI355GQ_API int mi355gq_moe_gemv_dt(const void* x, int64_t x_rows, const void* q_weight, const void* q_scale,
                        const void* expert_ids, int64_t top_k, int64_t num_experts, int64_t N, int64_t K,
                        int bits, int group_size, int model_dtype, void* out, mi355gq_stream_t stream);
MI355GQ_API int mi355gq_moe_group_gemm_dt(const void* x, int64_t rows, const void* q_weight, const void* q_scale,
                              const void* indptr, int indptr_dtype, int64_t num_experts, int64_t N,
                              int64_t K, int bits, int group_size, int model_dtype, void* out,
                              mi355gq_stream_t stream);

/*
 * The e1_e3 expert matmul of MixtralMoE with its activation folded in (mixtral_model.py:64-68:
 * x1, x3 = split(e1_e3(x, indptr), 2, axis=-1); silu(x1) * x3), in both forms of the expert matmul.
 * Same arguments as mi355gq_moe_gemv / mi355gq_moe_group_gemm; N is the stored row count of an
 * expert (gate rows then up rows, N even) and out is fp16 [top_k | rows, N / 2]; results equal the
 * unfused call followed by mi355gq_silu_mul bit for bit.  MI355GQ_ERR_UNSUPPORTED when no fused
 * kernel takes the shape.
 */
MI355GQ_API int mi355gq_moe_gemv_silu_mul(const void* x, int64_t x_rows, const void* q_weight,
                              const void* q_scale, const void* expert_ids, int64_t top_k,
                              int64_t num_experts, int64_t N, int64_t K, int bits, int group_size,
                              void* out, mi355gq_stream_t stream);
/*
 * One token through the router and the e1_e3 expert matmul in one launch (MixtralMoE.forward with one token,
 * mixtral_model.py:76-95: gating_softmax_topk of moe_misc.py:135-235, then dequantize_gemv of moe_matmul.py:77-176
 * with silu(x1) * x3 folded in as above).  x [1, K] and gate_logits [num_experts] in the model dtype; every
 * workgroup picks the top_k experts from the logits itself, so no routing kernel runs in front.  Writes
 * expert_weights [top_k] (model dtype) and expert_ids int32 [top_k], bit for bit what mi355gq_gating_softmax_topk
 * returns, for the operators that follow (the e2 matmul, the combine), and out [top_k, N / 2], bit for bit what
 * mi355gq_moe_gemv_silu_mul_dt returns for those ids.  float16 / bfloat16 models, top_k <= 2, at most 64 experts;
 * MI355GQ_ERR_UNSUPPORTED otherwise (the caller then runs the two operators).
 */
MI355GQ_API int mi355gq_moe_gemv_routed_silu_mul(const void* x, const void* gate_logits, int64_t num_experts,
                                     int64_t top_k, const void* q_weight, const void* q_scale, int64_t N, int64_t K,
                                     int bits, int group_size, int model_dtype, void* expert_weights,
                                     void* expert_ids, void* out, mi355gq_stream_t stream);
/*
 * One token's e2 expert matmul and the weighted sum over its experts in one launch (MixtralMoE.forward with one token,
 * mixtral_model.py:96-117: dequantize_gemv of moe_matmul.py:77-176 on the top_k rows of x, each against its expert,
 * then x * expert_weights and moe_sum of moe_misc.py:14-32).  x [top_k, K], expert_ids int32 [top_k], expert_weights
 * [top_k] and out [1, N] in the model dtype; out equals, bit for bit in its roundings (matmul result, product, sum, each
 * rounded to the model dtype), mi355gq_moe_gemv_dt followed by mi355gq_moe_combine_dt up to the order in which a row's
 * K is summed (two halves).  float16 / bfloat16 models, top_k = 2, K of 3 to 12 groups per lane (q4: 4097..24576 while
 * both rows of x fit 63 KiB of LDS); MI355GQ_ERR_UNSUPPORTED otherwise (the caller then runs the two operators).
 */
MI355GQ_API int mi355gq_moe_gemv_combine(const void* x, const void* q_weight, const void* q_scale, int64_t N, int64_t K,
                             int bits, int group_size, int model_dtype, int64_t num_experts,
                             const void* expert_ids, const void* expert_weights, int64_t top_k, void* out,
                             mi355gq_stream_t stream);
MI355GQ_API int mi355gq_moe_group_gemm_silu_mul(const void* x, int64_t rows, const void* q_weight,
                                    const void* q_scale, const void* indptr, int indptr_dtype,
                                    int64_t num_experts, int64_t N, int64_t K, int bits, int group_size,
                                    void* out, mi355gq_stream_t stream);

/*
 * The grouped expert matmul with the steps MixtralMoE.forward wraps around it folded in
 * (mixtral_model.py:99-109): the gather `x = take(x, token_indices)` becomes an index on the
 * activation rows (row r of the expert-sorted order reads x[x_row_index[r]]; x_row_index int32 [rows]
 * or NULL for x already gathered, x has x_rows rows), and epilogue MI355GQ_EPILOGUE_SILU_MUL gives
 * silu(x1) * x3 of the two halves as in mi355gq_moe_group_gemm_silu_mul.  Same kernels and bits as
 * mi355gq_take_rows followed by mi355gq_moe_group_gemm(_silu_mul).
 */
#define MI355GQ_EPILOGUE_NONE 0
#define MI355GQ_EPILOGUE_SILU_MUL 1
MI355GQ_API int mi355gq_moe_experts(const void* x, int64_t x_rows, const void* x_row_index, int64_t rows,
                        const void* q_weight, const void* q_scale, const void* indptr, int indptr_dtype,
                        int64_t num_experts, int64_t N, int64_t K, int bits, int group_size, int epilogue,
                        void* out, mi355gq_stream_t stream);

/* ---- routing glue of the MoE layer (python/mlc_llm/op/moe_misc.py) ---- */

/*
 * The routing of one MoE layer in one launch: gating_softmax_topk, moe_cumsum, get_indices and
 * get_indptr (moe_misc.py:135-235, 371-605; the sequence of mixtral_model.py:77-106) for batches one
 * workgroup can scan (T * top_k <= 8192 with num_experts * ceil(T * top_k / 64) <= 8192, or else
 * num_experts <= 64 and T <= 8192 with num_experts * ceil(T / 1024) <= 64; otherwise
 * MI355GQ_ERR_UNSUPPORTED and the four calls below do the same work).  Outputs as those calls give
 * them: weights fp16 [T, top_k], ids int32 [T, top_k], token_indices / reverse_indices int32
 * [T * top_k], indptr [num_experts + 1] (exclusive form, indptr[0] = 0); plus slot_positions int32
 * [T * top_k], the inverse of reverse_indices (slot t * top_k + j is row slot_positions[...] of the
 * expert-sorted order), which lets mi355gq_moe_combine_sorted read the experts' output where it lies.
 * The [num_experts, T] cumsum table is not materialised.
 */
MI355GQ_API int mi355gq_moe_route(const void* logits, int64_t T, int64_t num_experts, int64_t top_k,
                      void* weights, void* ids, void* token_indices, void* reverse_indices,
                      void* slot_positions, void* indptr, int indptr_dtype, mi355gq_stream_t stream);

/* gating_softmax_topk, norm_topk_prob = True (moe_misc.py:135-235): logits fp16 [T, num_experts]
 * -> weights fp16 [T, top_k] (softmax over the selected logits, fp32 maths), ids int32 [T, top_k].
 * Ties keep the lower expert index. top_k <= 8, num_experts <= 256. */
MI355GQ_API int mi355gq_gating_softmax_topk(const void* logits, int64_t T, int64_t num_experts, int64_t top_k,
                                void* weights, void* ids, mi355gq_stream_t stream);

/* gating_topk (moe_misc.py:63-132): scores [T, num_experts] in model_dtype -> the top_k scores as they are
 * [T, top_k] and their expert ids int32 [T, top_k], by the same insertion (ties keep the lower index). top_k <= 8. */
MI355GQ_API int mi355gq_gating_topk(const void* scores, int64_t T, int64_t num_experts, int64_t top_k,
                        void* out_scores, void* ids, int model_dtype, mi355gq_stream_t stream);

/* gating_softmax_topk with its norm_topk_prob argument (moe_misc.py:135-235).  norm_topk_prob != 0 is
 * mi355gq_gating_softmax_topk(_dt).  norm_topk_prob == 0 is the branch of :234-235: softmax over ALL experts in
 * fp32, cast to the model dtype, then gating_topk of those rounded scores; the weights are the selected scores,
 * not renormalised. */
/* (The reference leaves the order of the fp32 sum over all experts to TVM's reduction; this entry sums left to right,
 * so a score may differ from the reference's in the last place of the model dtype and, with it, a near-tie's winner.) */
MI355GQ_API int mi355gq_gating_softmax_topk_ex(const void* logits, int64_t T, int64_t num_experts, int64_t top_k,
                                   int norm_topk_prob, int model_dtype, void* weights, void* ids,
                                   mi355gq_stream_t stream);

/* moe_cumsum (moe_misc.py:371-450): ids int32 [T, top_k] -> cumsum int32 [num_experts * T],
 * inclusive prefix sum of the expert-major token mask. */
MI355GQ_API int mi355gq_moe_cumsum(const void* ids, int64_t T, int64_t top_k, int64_t num_experts,
                       void* cumsum, mi355gq_stream_t stream);

/* get_indices (moe_misc.py:453-525): cumsum int32 [num_experts * T], ids int32 [T, top_k]
 * -> reverse_indices, token_indices int32 [T * top_k]. */
MI355GQ_API int mi355gq_moe_get_indices(const void* cumsum, const void* ids, int64_t T, int64_t top_k,
                            int64_t num_experts, void* reverse_indices, void* token_indices, mi355gq_stream_t stream);

/* get_indptr (moe_misc.py:528-605): inclusive = 0 -> [num_experts + 1] with leading 0,
 * inclusive = 1 -> [num_experts]; out_dtype MI355GQ_I32 or MI355GQ_I64. */
MI355GQ_API int mi355gq_moe_get_indptr(const void* cumsum, int64_t num_experts, int64_t T, int inclusive,
                           int out_dtype, void* indptr, mi355gq_stream_t stream);

/* relax take(x, indices, axis=0) as used at model/mixtral/mixtral_model.py:107:
 * out fp16 [R, H] = x[indices[r], :]. */
MI355GQ_API int mi355gq_take_rows(const void* x, const void* indices, int64_t R, int64_t H, int64_t x_rows,
                      void* out, mi355gq_stream_t stream);

/* scatter_output (moe_misc.py:608-645): out[indices[r], :] = x[r, :], fp16 [R, H]. */
MI355GQ_API int mi355gq_moe_scatter_output(const void* x, const void* indices, int64_t R, int64_t H,
                               void* out, mi355gq_stream_t stream);

/* split + silu(x1) * x3 (mixtral_model.py:66-68): x fp16 [R, 2I] -> out fp16 [R, I]. */
MI355GQ_API int mi355gq_silu_mul(const void* x, int64_t R, int64_t I, void* out, mi355gq_stream_t stream);

/* weights * experts' outputs, summed over top_k (mixtral_model.py:111-115, moe_misc.moe_sum
 * :14-32): y fp16 [T, top_k, H], weights fp16 [T, top_k] -> out fp16 [T, H]; fp16 product,
 * fp16 left-to-right sum, as the reference's elementwise ops do. */
MI355GQ_API int mi355gq_moe_combine(const void* y, const void* weights, int64_t T, int64_t top_k, int64_t H,
                        void* out, mi355gq_stream_t stream);

/* scatter_output (moe_misc.py:608-645) + the combine above in one pass: y fp16 [T * top_k, H] still in
 * expert-sorted order, slot_positions from mi355gq_moe_route; out[t] = sum_j w[t, j] * y[slot_positions[t * top_k + j]]. */
MI355GQ_API int mi355gq_moe_combine_sorted(const void* y, const void* slot_positions, const void* weights,
                               int64_t T, int64_t top_k, int64_t H, void* out, mi355gq_stream_t stream);

/*
 * The folded gate/up activation (mi355gq_linear_silu_mul, mi355gq_moe_gemv_silu_mul, mi355gq_moe_group_gemm_silu_mul)
 * for bfloat16 models: y / out in bfloat16 [.., N / 2], equal bit for bit to the plain entry followed by
 * mi355gq_silu_mul_dt.  MI355GQ_F16 forwards to the float16 entries; MI355GQ_F32 and shapes without a fused kernel
 * return MI355GQ_ERR_UNSUPPORTED (run the two steps).
 */
MI355GQ_API int64_t mi355gq_linear_silu_mul_dt_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits,
                                                   int group_size, int model_dtype);
MI355GQ_API int mi355gq_linear_silu_mul_dt(const void* x, const void* q_weight, const void* q_scale, int64_t M,
                               int64_t N, int64_t K, int bits, int group_size, int model_dtype, void* y,
                               void* workspace, int64_t workspace_bytes, mi355gq_stream_t stream);
MI355GQ_API int mi355gq_moe_gemv_silu_mul_dt(const void* x, int64_t x_rows, const void* q_weight, const void* q_scale,
                                 const void* expert_ids, int64_t top_k, int64_t num_experts, int64_t N,
                                 int64_t K, int bits, int group_size, int model_dtype, void* out,
                                 mi355gq_stream_t stream);
MI355GQ_API int mi355gq_moe_group_gemm_silu_mul_dt(const void* x, int64_t rows, const void* q_weight,
                                       const void* q_scale, const void* indptr, int indptr_dtype,
                                       int64_t num_experts, int64_t N, int64_t K, int bits, int group_size,
                                       int model_dtype, void* out, mi355gq_stream_t stream);

/* mi355gq_moe_experts for bfloat16 models (float32: MI355GQ_ERR_UNSUPPORTED when x_row_index is given). */
MI355GQ_API int mi355gq_moe_experts_dt(const void* x, int64_t x_rows, const void* x_row_index, int64_t rows,
                           const void* q_weight, const void* q_scale, const void* indptr, int indptr_dtype,
                           int64_t num_experts, int64_t N, int64_t K, int bits, int group_size, int epilogue,
                           int model_dtype, void* out, mi355gq_stream_t stream);

/*
 * The routing glue for the other model dtypes (logits, weights, activations and results in model_dtype =
 * MI355GQ_F32 or MI355GQ_BF16; MI355GQ_F16 is the entries above): the same operations with every
 * intermediate the reference stores rounded to that dtype (softmax in fp32 as in moe_misc.py:205-219; silu in
 * fp32, rounded, then the product rounded; the combine's product and left-to-right sums rounded).  take_rows /
 * moe_scatter_output move rows of the dtype's element size.  mi355gq_moe_combine_dt: slot_positions null for y in
 * slot order (mi355gq_moe_combine), else the expert-sorted order (mi355gq_moe_combine_sorted).
 */
MI355GQ_API int mi355gq_gating_softmax_topk_dt(const void* logits, int64_t T, int64_t num_experts, int64_t top_k,
                                   void* weights, void* ids, int model_dtype, mi355gq_stream_t stream);
MI355GQ_API int mi355gq_moe_route_dt(const void* logits, int64_t T, int64_t num_experts, int64_t top_k, void* weights,
                         void* ids, void* token_indices, void* reverse_indices, void* slot_positions,
                         void* indptr, int indptr_dtype, int model_dtype, mi355gq_stream_t stream);
MI355GQ_API int mi355gq_take_rows_dt(const void* x, const void* indices, int64_t R, int64_t H, int64_t x_rows,
                         void* out, int model_dtype, mi355gq_stream_t stream);
MI355GQ_API int mi355gq_moe_scatter_output_dt(const void* x, const void* indices, int64_t R, int64_t H, void* out,
                                  int model_dtype, mi355gq_stream_t stream);
MI355GQ_API int mi355gq_silu_mul_dt(const void* x, int64_t R, int64_t I, void* out, int model_dtype,
                        mi355gq_stream_t stream);
MI355GQ_API int mi355gq_moe_combine_dt(const void* y, const void* slot_positions, const void* weights, int64_t T,
                           int64_t top_k, int64_t H, void* out, int model_dtype, mi355gq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355GQ_H_ */
