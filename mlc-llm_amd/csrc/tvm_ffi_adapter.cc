// TVM-FFI adapter: registers the C ABI of include/mi355gq.h as global packed functions, so that
// a Relax module can reach the kernels through
//     R.call_dps_packed("mlc.gq.linear", (x, q_weight, q_scale, bias, bits, group_size, workspace), out_sinfo=...)
// the same way the reference reaches "fastertransformer.gemm_fp16_int"
// (python/mlc_llm/op/ft_gemm.py:72-92) or "cutlass.group_gemm" (op/cutlass.py:71-77).
// Registration follows the reference's own idiom (cpp/multi_gpu/builtin.cc:89-94).
//
// NOT COMPILED IN THIS TREE BY DEFAULT: build.py adds this file only when the `tvm_ffi` Python
// package (which ships the tvm/ffi headers) is importable.  The container this library was
// developed in has no TVM, so this file has never been compiled; it is the binding a maintainer
// adds, kept next to the code it binds.  Everything it calls is the verified C ABI.
//
// DPS convention: the destination tensor(s) come last.  Tensors arrive as DLTensor views; ints as
// int64.  Errors of the C ABI are rethrown as TVM errors carrying mi355gq_last_error().
#include <tvm/ffi/container/tensor.h>
#include <tvm/ffi/error.h>
#include <tvm/ffi/extra/c_env_api.h>
#include <tvm/ffi/function.h>
#include <tvm/ffi/optional.h>
#include <tvm/ffi/reflection/registry.h>

#include "../../include/mi355gq.h"

namespace mlc {
namespace llm {
namespace gq {

using tvm::ffi::Optional;
using tvm::ffi::TensorView;

namespace {

inline void* Ptr(const TensorView& t) {
  return static_cast<char*>(t.data_ptr()) + t.byte_offset();
}

inline void* StreamOf(const TensorView& t) {
  const DLDevice dev = t.device();
  TVM_FFI_ICHECK(dev.device_type == kDLROCM) << "mlc.gq.*: tensors must live on a ROCm device";
  return TVMFFIEnvGetStream(dev.device_type, dev.device_id);
}

inline void Check(int rc, const char* what) {
  if (rc != MI355GQ_OK) TVM_FFI_THROW(RuntimeError) << what << ": " << mi355gq_last_error();
}

inline int64_t Rows(const TensorView& t) {  // product of all dims but the last
  int64_t m = 1;
  for (int i = 0; i + 1 < t.ndim(); ++i) m *= t.shape()[i];
  return m;
}

inline int OutDtype(const TensorView& y) { return y.dtype().bits == 32 ? MI355GQ_F32 : MI355GQ_F16; }

}  // namespace

// y = x . dequantize(q_weight, q_scale)^T (+ bias).  `workspace` is an optional uint8 scratch
// tensor of at least mlc.gq.linear_workspace_bytes(M, N, K, bits, group_size) bytes (the few-row
// GEMM splits K through it); without it the call is still correct, only slower for 17..256 rows.
void Linear(TensorView x, TensorView q_weight, TensorView q_scale, Optional<TensorView> bias,
            int64_t bits, int64_t group_size, Optional<TensorView> workspace, TensorView y) {
  const int64_t K = x.shape()[x.ndim() - 1], N = q_weight.shape()[0];
  void* ws = workspace.has_value() ? Ptr(workspace.value()) : nullptr;
  int64_t ws_bytes = 0;
  if (workspace.has_value()) {
    ws_bytes = (workspace.value().dtype().bits + 7) / 8;
    for (int i = 0; i < workspace.value().ndim(); ++i) ws_bytes *= workspace.value().shape()[i];
  }
  Check(mi355gq_linear(Ptr(x), Ptr(q_weight), Ptr(q_scale),
                       bias.has_value() ? Ptr(bias.value()) : nullptr, Rows(x), N, K,
                       static_cast<int>(bits), static_cast<int>(group_size), OutDtype(y), Ptr(y),
                       ws, ws_bytes, StreamOf(x)),
        "mlc.gq.linear");
}

// y = x . dequantize(q_weight, q_scale)^T (+ bias) + residual; residual may be y itself
void LinearResidual(TensorView x, TensorView q_weight, TensorView q_scale, Optional<TensorView> bias,
                    TensorView residual, int64_t bits, int64_t group_size, Optional<TensorView> workspace,
                    TensorView y) {
  const int64_t K = x.shape()[x.ndim() - 1], N = q_weight.shape()[0];
  void* ws = workspace.has_value() ? Ptr(workspace.value()) : nullptr;
  int64_t ws_bytes = 0;
  if (workspace.has_value()) {
    ws_bytes = (workspace.value().dtype().bits + 7) / 8;
    for (int i = 0; i < workspace.value().ndim(); ++i) ws_bytes *= workspace.value().shape()[i];
  }
  Check(mi355gq_linear_residual(Ptr(x), Ptr(q_weight), Ptr(q_scale),
                                bias.has_value() ? Ptr(bias.value()) : nullptr, Ptr(residual), Rows(x),
                                N, K, static_cast<int>(bits), static_cast<int>(group_size), OutDtype(y),
                                Ptr(y), ws, ws_bytes, StreamOf(x)),
        "mlc.gq.linear_residual");
}

int64_t LinearWorkspaceBytes(int64_t M, int64_t N, int64_t K, int64_t bits, int64_t group_size) {
  return mi355gq_linear_workspace_bytes(M, N, K, static_cast<int>(bits), static_cast<int>(group_size));
}

// y[M, N / 2] = silu(x1) * x2 with x1, x2 = split(x . dequantize(q_weight, q_scale)^T, 2, axis=-1): the
// gate_up projection of an MLP with its activation folded in.  There is no fused kernel when K is
// not a multiple of 8 (an error here): the pass that rewrites matmul + split + silu + multiply into
// this call must leave such layers as they are.
void LinearSiluMul(TensorView x, TensorView q_weight, TensorView q_scale, int64_t bits, int64_t group_size,
                   Optional<TensorView> workspace, TensorView y) {
  const int64_t K = x.shape()[x.ndim() - 1], N = q_weight.shape()[0];
  void* ws = workspace.has_value() ? Ptr(workspace.value()) : nullptr;
  int64_t ws_bytes = 0;
  if (workspace.has_value()) {
    ws_bytes = (workspace.value().dtype().bits + 7) / 8;
    for (int i = 0; i < workspace.value().ndim(); ++i) ws_bytes *= workspace.value().shape()[i];
  }
  Check(mi355gq_linear_silu_mul(Ptr(x), Ptr(q_weight), Ptr(q_scale), Rows(x), N, K, static_cast<int>(bits),
                                static_cast<int>(group_size), Ptr(y), ws, ws_bytes, StreamOf(x)),
        "mlc.gq.linear_silu_mul");
}

int64_t LinearSiluMulWorkspaceBytes(int64_t M, int64_t N, int64_t K, int64_t bits, int64_t group_size) {
  return mi355gq_linear_silu_mul_workspace_bytes(M, N, K, static_cast<int>(bits), static_cast<int>(group_size));
}

void EmbeddingTake(TensorView ids, TensorView q_weight, TensorView q_scale, int64_t bits,
                   int64_t group_size, TensorView out) {
  const int64_t K = out.shape()[out.ndim() - 1];
  Check(mi355gq_embedding_take(Ptr(ids), Rows(out), Ptr(q_weight), Ptr(q_scale),
                               q_weight.shape()[0], K, static_cast<int>(bits),
                               static_cast<int>(group_size), Ptr(out), StreamOf(out)),
        "mlc.gq.embedding_take");
}

void MoeGemv(TensorView x, TensorView q_weight, TensorView q_scale, TensorView expert_ids,
             int64_t bits, int64_t group_size, TensorView out) {
  Check(mi355gq_moe_gemv(Ptr(x), x.shape()[0], Ptr(q_weight), Ptr(q_scale), Ptr(expert_ids),
                         expert_ids.shape()[1], q_weight.shape()[0], q_weight.shape()[1],
                         x.shape()[1], static_cast<int>(bits), static_cast<int>(group_size), Ptr(out),
                         StreamOf(x)),
        "mlc.gq.moe_gemv");
}

void MoeGroupGemm(TensorView x, TensorView q_weight, TensorView q_scale, TensorView indptr,
                  int64_t bits, int64_t group_size, TensorView out) {
  Check(mi355gq_moe_group_gemm(Ptr(x), x.shape()[0], Ptr(q_weight), Ptr(q_scale), Ptr(indptr),
                               indptr.dtype().bits == 64 ? MI355GQ_I64 : MI355GQ_I32,
                               q_weight.shape()[0], q_weight.shape()[1], x.shape()[1],
                               static_cast<int>(bits), static_cast<int>(group_size), Ptr(out),
                               StreamOf(x)),
        "mlc.gq.moe_group_gemm");
}

// the e1_e3 expert matmuls with silu(x1) * x3 folded in: out is [top_k | rows, N / 2]
void MoeGemvSiluMul(TensorView x, TensorView q_weight, TensorView q_scale, TensorView expert_ids,
                    int64_t bits, int64_t group_size, TensorView out) {
  Check(mi355gq_moe_gemv_silu_mul(Ptr(x), x.shape()[0], Ptr(q_weight), Ptr(q_scale), Ptr(expert_ids),
                                  expert_ids.shape()[1], q_weight.shape()[0], q_weight.shape()[1],
                                  x.shape()[1], static_cast<int>(bits), static_cast<int>(group_size),
                                  Ptr(out), StreamOf(x)),
        "mlc.gq.moe_gemv_silu_mul");
}

void MoeGroupGemmSiluMul(TensorView x, TensorView q_weight, TensorView q_scale, TensorView indptr,
                         int64_t bits, int64_t group_size, TensorView out) {
  Check(mi355gq_moe_group_gemm_silu_mul(Ptr(x), x.shape()[0], Ptr(q_weight), Ptr(q_scale), Ptr(indptr),
                                        indptr.dtype().bits == 64 ? MI355GQ_I64 : MI355GQ_I32,
                                        q_weight.shape()[0], q_weight.shape()[1], x.shape()[1],
                                        static_cast<int>(bits), static_cast<int>(group_size), Ptr(out),
                                        StreamOf(x)),
        "mlc.gq.moe_group_gemm_silu_mul");
}

// group gemm over x[x_row_index] (x_row_index: the layer's token_indices, or absent for gathered x);
// silu_mul != 0 folds silu(x1) * x3 of the output halves in
void MoeExperts(TensorView x, Optional<TensorView> x_row_index, TensorView q_weight, TensorView q_scale,
                TensorView indptr, int64_t bits, int64_t group_size, int64_t silu_mul, TensorView out) {
  Check(mi355gq_moe_experts(Ptr(x), x.shape()[0], x_row_index.has_value() ? Ptr(x_row_index.value()) : nullptr,
                            out.shape()[0], Ptr(q_weight), Ptr(q_scale), Ptr(indptr),
                            indptr.dtype().bits == 64 ? MI355GQ_I64 : MI355GQ_I32, q_weight.shape()[0],
                            q_weight.shape()[1], x.shape()[1], static_cast<int>(bits),
                            static_cast<int>(group_size),
                            silu_mul ? MI355GQ_EPILOGUE_SILU_MUL : MI355GQ_EPILOGUE_NONE, Ptr(out), StreamOf(x)),
        "mlc.gq.moe_experts");
}

// routing of one MoE layer; six destinations
void MoeRoute(TensorView logits, int64_t top_k, TensorView weights, TensorView ids, TensorView token_indices,
              TensorView reverse_indices, TensorView slot_positions, TensorView indptr) {
  Check(mi355gq_moe_route(Ptr(logits), logits.shape()[0], logits.shape()[1], top_k, Ptr(weights), Ptr(ids),
                          Ptr(token_indices), Ptr(reverse_indices), Ptr(slot_positions), Ptr(indptr),
                          indptr.dtype().bits == 64 ? MI355GQ_I64 : MI355GQ_I32, StreamOf(logits)),
        "mlc.gq.moe_route");
}

void MoeCombineSorted(TensorView y, TensorView slot_positions, TensorView weights, TensorView out) {
  Check(mi355gq_moe_combine_sorted(Ptr(y), Ptr(slot_positions), Ptr(weights), weights.shape()[0],
                                   weights.shape()[1], y.shape()[1], Ptr(out), StreamOf(y)),
        "mlc.gq.moe_combine_sorted");
}

// quantize has two destinations: (q_weight, q_scale)
void Quantize(TensorView w, int64_t bits, int64_t group_size, int64_t round_mode,
              TensorView q_weight, TensorView q_scale) {
  const int64_t K = w.shape()[w.ndim() - 1];
  Check(mi355gq_quantize(Ptr(w), Rows(w), K, static_cast<int>(bits), static_cast<int>(group_size),
                         static_cast<int>(round_mode), Ptr(q_weight), Ptr(q_scale), StreamOf(w)),
        "mlc.gq.quantize");
}

void Dequantize(TensorView q_weight, TensorView q_scale, int64_t bits, int64_t group_size,
                TensorView out) {
  const int64_t K = out.shape()[out.ndim() - 1];
  Check(mi355gq_dequantize(Ptr(q_weight), Ptr(q_scale), Rows(out), K, static_cast<int>(bits),
                           static_cast<int>(group_size), Ptr(out), StreamOf(out)),
        "mlc.gq.dequantize");
}

// the same four for the other model dtypes: model_dtype is MI355GQ_F16 / MI355GQ_F32 / MI355GQ_BF16
void QuantizeDt(TensorView w, int64_t bits, int64_t group_size, int64_t round_mode, int64_t model_dtype,
                TensorView q_weight, TensorView q_scale) {
  const int64_t K = w.shape()[w.ndim() - 1];
  Check(mi355gq_quantize_dt(Ptr(w), Rows(w), K, static_cast<int>(bits), static_cast<int>(group_size),
                            static_cast<int>(round_mode), static_cast<int>(model_dtype), Ptr(q_weight),
                            Ptr(q_scale), StreamOf(w)),
        "mlc.gq.quantize_dt");
}

void DequantizeDt(TensorView q_weight, TensorView q_scale, int64_t bits, int64_t group_size, int64_t model_dtype,
                  TensorView out) {
  const int64_t K = out.shape()[out.ndim() - 1];
  Check(mi355gq_dequantize_dt(Ptr(q_weight), Ptr(q_scale), Rows(out), K, static_cast<int>(bits),
                              static_cast<int>(group_size), static_cast<int>(model_dtype), Ptr(out),
                              StreamOf(out)),
        "mlc.gq.dequantize_dt");
}

void EmbeddingTakeDt(TensorView ids, TensorView q_weight, TensorView q_scale, int64_t bits, int64_t group_size,
                     int64_t model_dtype, TensorView out) {
  const int64_t K = out.shape()[out.ndim() - 1];
  Check(mi355gq_embedding_take_dt(Ptr(ids), Rows(out), Ptr(q_weight), Ptr(q_scale), q_weight.shape()[0], K,
                                  static_cast<int>(bits), static_cast<int>(group_size),
                                  static_cast<int>(model_dtype), Ptr(out), StreamOf(out)),
        "mlc.gq.embedding_take_dt");
}

int64_t LinearDtWorkspaceBytes(int64_t M, int64_t N, int64_t K, int64_t bits, int64_t group_size,
                               int64_t model_dtype) {
  return mi355gq_linear_dt_workspace_bytes(M, N, K, static_cast<int>(bits), static_cast<int>(group_size),
                                           static_cast<int>(model_dtype));
}

void LinearDt(TensorView x, TensorView q_weight, TensorView q_scale, Optional<TensorView> bias, int64_t bits,
              int64_t group_size, int64_t model_dtype, Optional<TensorView> workspace, TensorView y) {
  const int64_t K = x.shape()[x.ndim() - 1], N = q_weight.shape()[0];
  const int out_dtype = y.dtype().bits == 32 ? MI355GQ_F32 : static_cast<int>(model_dtype);
  void* ws = workspace.has_value() ? Ptr(workspace.value()) : nullptr;
  int64_t ws_bytes = 0;
  if (workspace.has_value()) {
    ws_bytes = (workspace.value().dtype().bits + 7) / 8;
    for (int i = 0; i < workspace.value().ndim(); ++i) ws_bytes *= workspace.value().shape()[i];
  }
  Check(mi355gq_linear_dt(Ptr(x), Ptr(q_weight), Ptr(q_scale), bias.has_value() ? Ptr(bias.value()) : nullptr,
                          Rows(x), N, K, static_cast<int>(bits), static_cast<int>(group_size),
                          static_cast<int>(model_dtype), out_dtype, Ptr(y), ws, ws_bytes, StreamOf(x)),
        "mlc.gq.linear_dt");
}

void LinearResidualDt(TensorView x, TensorView q_weight, TensorView q_scale, Optional<TensorView> bias,
                      TensorView residual, int64_t bits, int64_t group_size, int64_t model_dtype,
                      Optional<TensorView> workspace, TensorView y) {
  const int64_t K = x.shape()[x.ndim() - 1], N = q_weight.shape()[0];
  const int out_dtype = y.dtype().bits == 32 ? MI355GQ_F32 : static_cast<int>(model_dtype);
  void* ws = workspace.has_value() ? Ptr(workspace.value()) : nullptr;
  int64_t ws_bytes = 0;
  if (workspace.has_value()) {
    ws_bytes = (workspace.value().dtype().bits + 7) / 8;
    for (int i = 0; i < workspace.value().ndim(); ++i) ws_bytes *= workspace.value().shape()[i];
  }
  Check(mi355gq_linear_residual_dt(Ptr(x), Ptr(q_weight), Ptr(q_scale),
                                   bias.has_value() ? Ptr(bias.value()) : nullptr, Ptr(residual), Rows(x), N, K,
                                   static_cast<int>(bits), static_cast<int>(group_size),
                                   static_cast<int>(model_dtype), out_dtype, Ptr(y), ws, ws_bytes, StreamOf(x)),
        "mlc.gq.linear_residual_dt");
}

void MoeGemvDt(TensorView x, TensorView q_weight, TensorView q_scale, TensorView expert_ids, int64_t bits,
               int64_t group_size, int64_t model_dtype, TensorView out) {
  Check(mi355gq_moe_gemv_dt(Ptr(x), x.shape()[0], Ptr(q_weight), Ptr(q_scale), Ptr(expert_ids),
                            expert_ids.shape()[1], q_weight.shape()[0], q_weight.shape()[1], x.shape()[1],
                            static_cast<int>(bits), static_cast<int>(group_size), static_cast<int>(model_dtype),
                            Ptr(out), StreamOf(x)),
        "mlc.gq.moe_gemv_dt");
}

void MoeGroupGemmDt(TensorView x, TensorView q_weight, TensorView q_scale, TensorView indptr, int64_t bits,
                    int64_t group_size, int64_t model_dtype, TensorView out) {
  Check(mi355gq_moe_group_gemm_dt(Ptr(x), x.shape()[0], Ptr(q_weight), Ptr(q_scale), Ptr(indptr),
                                  indptr.dtype().bits == 64 ? MI355GQ_I64 : MI355GQ_I32, q_weight.shape()[0],
                                  q_weight.shape()[1], x.shape()[1], static_cast<int>(bits),
                                  static_cast<int>(group_size), static_cast<int>(model_dtype), Ptr(out),
                                  StreamOf(x)),
        "mlc.gq.moe_group_gemm_dt");
}

// the folded gate/up activation for bfloat16 models (y / out are [.., N / 2] in the model dtype)
void LinearSiluMulDt(TensorView x, TensorView q_weight, TensorView q_scale, int64_t bits, int64_t group_size,
                     int64_t model_dtype, Optional<TensorView> workspace, TensorView y) {
  const int64_t K = x.shape()[x.ndim() - 1], N = q_weight.shape()[0];
  void* ws = workspace.has_value() ? Ptr(workspace.value()) : nullptr;
  int64_t ws_bytes = 0;
  if (workspace.has_value()) {
    ws_bytes = (workspace.value().dtype().bits + 7) / 8;
    for (int i = 0; i < workspace.value().ndim(); ++i) ws_bytes *= workspace.value().shape()[i];
  }
  Check(mi355gq_linear_silu_mul_dt(Ptr(x), Ptr(q_weight), Ptr(q_scale), Rows(x), N, K, static_cast<int>(bits),
                                   static_cast<int>(group_size), static_cast<int>(model_dtype), Ptr(y), ws,
                                   ws_bytes, StreamOf(x)),
        "mlc.gq.linear_silu_mul_dt");
}

void MoeGemvSiluMulDt(TensorView x, TensorView q_weight, TensorView q_scale, TensorView expert_ids, int64_t bits,
                      int64_t group_size, int64_t model_dtype, TensorView out) {
  Check(mi355gq_moe_gemv_silu_mul_dt(Ptr(x), x.shape()[0], Ptr(q_weight), Ptr(q_scale), Ptr(expert_ids),
                                     expert_ids.shape()[1], q_weight.shape()[0], q_weight.shape()[1], x.shape()[1],
                                     static_cast<int>(bits), static_cast<int>(group_size),
                                     static_cast<int>(model_dtype), Ptr(out), StreamOf(x)),
        "mlc.gq.moe_gemv_silu_mul_dt");
}

void MoeGroupGemmSiluMulDt(TensorView x, TensorView q_weight, TensorView q_scale, TensorView indptr, int64_t bits,
                           int64_t group_size, int64_t model_dtype, TensorView out) {
  Check(mi355gq_moe_group_gemm_silu_mul_dt(Ptr(x), x.shape()[0], Ptr(q_weight), Ptr(q_scale), Ptr(indptr),
                                           indptr.dtype().bits == 64 ? MI355GQ_I64 : MI355GQ_I32,
                                           q_weight.shape()[0], q_weight.shape()[1], x.shape()[1],
                                           static_cast<int>(bits), static_cast<int>(group_size),
                                           static_cast<int>(model_dtype), Ptr(out), StreamOf(x)),
        "mlc.gq.moe_group_gemm_silu_mul_dt");
}

void MoeExpertsDt(TensorView x, Optional<TensorView> x_row_index, TensorView q_weight, TensorView q_scale,
                  TensorView indptr, int64_t bits, int64_t group_size, int64_t epilogue, int64_t model_dtype,
                  TensorView out) {
  Check(mi355gq_moe_experts_dt(Ptr(x), x.shape()[0], x_row_index.has_value() ? Ptr(x_row_index.value()) : nullptr,
                               out.shape()[0], Ptr(q_weight), Ptr(q_scale), Ptr(indptr),
                               indptr.dtype().bits == 64 ? MI355GQ_I64 : MI355GQ_I32, q_weight.shape()[0],
                               q_weight.shape()[1], x.shape()[1], static_cast<int>(bits),
                               static_cast<int>(group_size), static_cast<int>(epilogue),
                               static_cast<int>(model_dtype), Ptr(out), StreamOf(x)),
        "mlc.gq.moe_experts_dt");
}

// routing glue with logits, weights and activations in model_dtype
void GatingSoftmaxTopkDt(TensorView logits, int64_t top_k, int64_t model_dtype, TensorView weights, TensorView ids) {
  Check(mi355gq_gating_softmax_topk_dt(Ptr(logits), logits.shape()[0], logits.shape()[1], top_k, Ptr(weights),
                                       Ptr(ids), static_cast<int>(model_dtype), StreamOf(logits)),
        "mlc.gq.gating_softmax_topk_dt");
}

void TakeRowsDt(TensorView x, TensorView indices, int64_t model_dtype, TensorView out) {
  Check(mi355gq_take_rows_dt(Ptr(x), Ptr(indices), out.shape()[0], x.shape()[1], x.shape()[0], Ptr(out),
                             static_cast<int>(model_dtype), StreamOf(x)),
        "mlc.gq.take_rows_dt");
}

void ScatterOutputDt(TensorView x, TensorView indices, int64_t model_dtype, TensorView out) {
  Check(mi355gq_moe_scatter_output_dt(Ptr(x), Ptr(indices), x.shape()[0], x.shape()[1], Ptr(out),
                                      static_cast<int>(model_dtype), StreamOf(x)),
        "mlc.gq.moe_scatter_output_dt");
}

void SiluMulDt(TensorView x, int64_t model_dtype, TensorView out) {
  Check(mi355gq_silu_mul_dt(Ptr(x), x.shape()[0], x.shape()[1] / 2, Ptr(out), static_cast<int>(model_dtype),
                            StreamOf(x)),
        "mlc.gq.silu_mul_dt");
}

void MoeCombineDt(TensorView y, Optional<TensorView> slot_positions, TensorView weights, int64_t model_dtype,
                  TensorView out) {
  Check(mi355gq_moe_combine_dt(Ptr(y), slot_positions.has_value() ? Ptr(slot_positions.value()) : nullptr,
                               Ptr(weights), weights.shape()[0], weights.shape()[1], out.shape()[1], Ptr(out),
                               static_cast<int>(model_dtype), StreamOf(y)),
        "mlc.gq.moe_combine_dt");
}

TVM_FFI_STATIC_INIT_BLOCK() {
  namespace refl = tvm::ffi::reflection;
  refl::GlobalDef()
      .def("mlc.gq.linear", Linear)
      .def("mlc.gq.linear_residual", LinearResidual)
      .def("mlc.gq.linear_workspace_bytes", LinearWorkspaceBytes)
      .def("mlc.gq.linear_silu_mul", LinearSiluMul)
      .def("mlc.gq.linear_silu_mul_workspace_bytes", LinearSiluMulWorkspaceBytes)
      .def("mlc.gq.embedding_take", EmbeddingTake)
      .def("mlc.gq.moe_gemv", MoeGemv)
      .def("mlc.gq.moe_group_gemm", MoeGroupGemm)
      .def("mlc.gq.moe_gemv_silu_mul", MoeGemvSiluMul)
      .def("mlc.gq.moe_group_gemm_silu_mul", MoeGroupGemmSiluMul)
      .def("mlc.gq.moe_experts", MoeExperts)
      .def("mlc.gq.moe_route", MoeRoute)
      .def("mlc.gq.moe_combine_sorted", MoeCombineSorted)
      .def("mlc.gq.quantize", Quantize)
      .def("mlc.gq.dequantize", Dequantize)
      .def("mlc.gq.quantize_dt", QuantizeDt)
      .def("mlc.gq.dequantize_dt", DequantizeDt)
      .def("mlc.gq.embedding_take_dt", EmbeddingTakeDt)
      .def("mlc.gq.linear_dt", LinearDt)
      .def("mlc.gq.linear_dt_workspace_bytes", LinearDtWorkspaceBytes)
      .def("mlc.gq.linear_residual_dt", LinearResidualDt)
      .def("mlc.gq.linear_silu_mul_dt", LinearSiluMulDt)
      .def("mlc.gq.moe_gemv_silu_mul_dt", MoeGemvSiluMulDt)
      .def("mlc.gq.moe_group_gemm_silu_mul_dt", MoeGroupGemmSiluMulDt)
      .def("mlc.gq.moe_experts_dt", MoeExpertsDt)
      .def("mlc.gq.gating_softmax_topk_dt", GatingSoftmaxTopkDt)
      .def("mlc.gq.take_rows_dt", TakeRowsDt)
      .def("mlc.gq.moe_scatter_output_dt", ScatterOutputDt)
      .def("mlc.gq.silu_mul_dt", SiluMulDt)
      .def("mlc.gq.moe_combine_dt", MoeCombineDt)
      .def("mlc.gq.moe_gemv_dt", MoeGemvDt)
      .def("mlc.gq.moe_group_gemm_dt", MoeGroupGemmDt);
}

}  // namespace gq
}  // namespace llm
}  // namespace mlc
