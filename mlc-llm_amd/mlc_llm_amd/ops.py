"""Destination-passing operators over torch ROCm tensors.

Each function plays the role the Relax VM plays around `call_dps_packed`: it
checks shapes and dtypes, allocates the output tensor(s) and hands raw pointers
plus the current HIP stream to the C ABI.  uint32 storage is held in int32
torch tensors (same bits; torch's uint32 support on device is partial).
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _chk(t: torch.Tensor, dtype, name: str) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name}: expected a torch.Tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise ValueError(f"{name}: must live on the GPU (got {t.device})")
    dtypes = dtype if isinstance(dtype, tuple) else (dtype,)
    if t.dtype not in dtypes:
        raise TypeError(f"{name}: dtype {t.dtype}, expected {dtypes}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: must be contiguous")
    return t


_STORAGE = (torch.int32, torch.uint32)
# model dtypes of the reference's group-quant registry -> the C ABI's dtype codes
_MODEL_DTYPES = {torch.float16: _lib.F16, torch.float32: _lib.F32, torch.bfloat16: _lib.BF16}
_FLOATS = tuple(_MODEL_DTYPES)


def num_group(k: int, group_size: int) -> int:
    return -(-k // group_size)


def num_storage(k: int, bits: int, group_size: int) -> int:
    return (group_size // (32 // bits)) * num_group(k, group_size)


def quantize(w: torch.Tensor, bits: int, group_size: int, round_mode: int = _lib.ROUND_HALF_AWAY
             ) -> Tuple[torch.Tensor, torch.Tensor]:
    """w [..., K] in the model dtype (float16, or float32 / bfloat16 for the q4f32 / q4bf16 schemes)
    -> (q_weight int32-as-uint32 [..., nw], q_scale [..., ng] in the same dtype)."""
    _chk(w, _FLOATS, "w")
    k = w.shape[-1]
    rows = w.numel() // k if k else 0
    lead = tuple(w.shape[:-1])
    qw = torch.empty((*lead, num_storage(k, bits, group_size)), dtype=torch.int32, device=w.device)
    qs = torch.empty((*lead, num_group(k, group_size)), dtype=w.dtype, device=w.device)
    if w.dtype == torch.float16:
        _lib.call("mi355gq_quantize", w.data_ptr(), rows, k, bits, group_size, round_mode,
                  qw.data_ptr(), qs.data_ptr(), _stream())
    else:
        _lib.call("mi355gq_quantize_dt", w.data_ptr(), rows, k, bits, group_size, round_mode,
                  _MODEL_DTYPES[w.dtype], qw.data_ptr(), qs.data_ptr(), _stream())
    return qw, qs


def dequantize(q_weight: torch.Tensor, q_scale: torch.Tensor, k: int, bits: int, group_size: int
               ) -> torch.Tensor:
    """(q_weight, q_scale) -> [..., K] in the dtype of q_scale (the scheme's model dtype)."""
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, _FLOATS, "q_scale")
    lead = tuple(q_weight.shape[:-1])
    _check_qshapes(q_weight, q_scale, lead, k, bits, group_size)
    rows = 1
    for d in lead:
        rows *= d
    out = torch.empty((*lead, k), dtype=q_scale.dtype, device=q_weight.device)
    if q_scale.dtype == torch.float16:
        _lib.call("mi355gq_dequantize", q_weight.data_ptr(), q_scale.data_ptr(), rows, k, bits,
                  group_size, out.data_ptr(), _stream())
    else:
        _lib.call("mi355gq_dequantize_dt", q_weight.data_ptr(), q_scale.data_ptr(), rows, k, bits,
                  group_size, _MODEL_DTYPES[q_scale.dtype], out.data_ptr(), _stream())
    return out


def _check_qshapes(q_weight, q_scale, lead, k, bits, group_size):
    nw, ng = num_storage(k, bits, group_size), num_group(k, group_size)
    if tuple(q_weight.shape) != (*lead, nw):
        raise ValueError(f"q_weight shape {tuple(q_weight.shape)}, expected {(*lead, nw)}")
    if tuple(q_scale.shape) != (*lead, ng):
        raise ValueError(f"q_scale shape {tuple(q_scale.shape)}, expected {(*lead, ng)}")


def embedding_take(ids: torch.Tensor, q_weight: torch.Tensor, q_scale: torch.Tensor, k: int,
                   bits: int, group_size: int) -> torch.Tensor:
    _chk(ids, torch.int32, "ids")
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, _FLOATS, "q_scale")
    num = q_weight.shape[0]
    _check_qshapes(q_weight, q_scale, (num,), k, bits, group_size)
    t = ids.numel()
    out = torch.empty((*ids.shape, k), dtype=q_scale.dtype, device=q_weight.device)
    if q_scale.dtype == torch.float16:
        _lib.call("mi355gq_embedding_take", ids.data_ptr(), t, q_weight.data_ptr(), q_scale.data_ptr(),
                  num, k, bits, group_size, out.data_ptr(), _stream())
    else:
        _lib.call("mi355gq_embedding_take_dt", ids.data_ptr(), t, q_weight.data_ptr(), q_scale.data_ptr(),
                  num, k, bits, group_size, _MODEL_DTYPES[q_scale.dtype], out.data_ptr(), _stream())
    return out


def linear(x: torch.Tensor, q_weight: torch.Tensor, q_scale: torch.Tensor, bits: int,
           group_size: int, bias: Optional[torch.Tensor] = None, out_dtype=torch.float16,
           out: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y[..., N] = x[..., K] . dequantize(q_weight, q_scale)^T (+ bias) (+ residual[..., N]).

    `residual` (fp16, the shape of y) is added inside the kernel; passing the same tensor as `out`
    updates it in place."""
    _chk(x, _FLOATS, "x")
    if x.dtype != torch.float16:
        return _linear_other_dtype(x, q_weight, q_scale, bits, group_size, bias, out_dtype, out, residual)
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, torch.float16, "q_scale")
    k = x.shape[-1]
    n = q_weight.shape[0]
    _check_qshapes(q_weight, q_scale, (n,), k, bits, group_size)
    m = 1
    for d in x.shape[:-1]:
        m *= d
    if bias is not None:
        _chk(bias, torch.float16, "bias")
        if tuple(bias.shape) != (n,):
            raise ValueError(f"bias shape {tuple(bias.shape)}, expected {(n,)}")
    if out_dtype not in (torch.float16, torch.float32):
        raise TypeError(f"out_dtype {out_dtype}")
    if out is None:
        out = torch.empty((*x.shape[:-1], n), dtype=out_dtype, device=x.device)
    else:
        _chk(out, out_dtype, "out")
    if residual is not None:
        _chk(residual, torch.float16, "residual")
        if tuple(residual.shape) != tuple(out.shape) or not residual.is_contiguous():
            raise ValueError(f"residual shape {tuple(residual.shape)}, expected contiguous {tuple(out.shape)}")
    ws_bytes = _lib.lib().mi355gq_linear_workspace_bytes(m, n, k, bits, group_size)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    tail = (m, n, k, bits, group_size, _lib.F32 if out_dtype == torch.float32 else _lib.F16, out.data_ptr(),
            ws.data_ptr() if ws is not None else None, ws_bytes, _stream())
    head = (x.data_ptr(), q_weight.data_ptr(), q_scale.data_ptr(), bias.data_ptr() if bias is not None else None)
    if residual is None:
        _lib.call("mi355gq_linear", *head, *tail)
    else:
        _lib.call("mi355gq_linear_residual", *head, residual.data_ptr(), *tail)
    return out


def _check_kn_shapes(q_weight, q_scale, k, bits, group_size):
    ng = -(-k // group_size)
    nw = (group_size // (32 // bits)) * ng
    if q_weight.dim() != 2 or q_scale.dim() != 2 or q_weight.shape[0] != nw or q_scale.shape[0] != ng or \
            q_weight.shape[1] != q_scale.shape[1]:
        raise ValueError(f"KN layout: q_weight {tuple(q_weight.shape)} / q_scale {tuple(q_scale.shape)}, expected "
                         f"({nw}, N) / ({ng}, N) for K={k}")
    if not (q_weight.is_contiguous() and q_scale.is_contiguous()):
        raise ValueError("KN layout: q_weight and q_scale must be contiguous")
    return q_weight.shape[1]


def linear_kn(x: torch.Tensor, q_weight: torch.Tensor, q_scale: torch.Tensor, bits: int, group_size: int,
              bias: Optional[torch.Tensor] = None, out_dtype=torch.float16) -> torch.Tensor:
    """linear() on KN-layout tensors as a q4f16_0 / q3f16_0 model stores them: q_weight [nw, N], q_scale [ng, N]
    (float16 models).  Up to 8 rows stream them in place; more rows run on an NK copy made in a workspace."""
    _chk(x, torch.float16, "x")
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, torch.float16, "q_scale")
    k = x.shape[-1]
    n = _check_kn_shapes(q_weight, q_scale, k, bits, group_size)
    m = 1
    for d in x.shape[:-1]:
        m *= d
    if bias is not None:
        _chk(bias, torch.float16, "bias")
        if tuple(bias.shape) != (n,):
            raise ValueError(f"bias shape {tuple(bias.shape)}, expected {(n,)}")
    if out_dtype not in (torch.float16, torch.float32):
        raise TypeError(f"out_dtype {out_dtype}")
    out = torch.empty((*x.shape[:-1], n), dtype=out_dtype, device=x.device)
    ws_bytes = _lib.lib().mi355gq_linear_kn_workspace_bytes(m, n, k, bits, group_size)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    _lib.call("mi355gq_linear_kn", x.data_ptr(), q_weight.data_ptr(), q_scale.data_ptr(),
              bias.data_ptr() if bias is not None else None, m, n, k, bits, group_size,
              _lib.F32 if out_dtype == torch.float32 else _lib.F16, out.data_ptr(),
              ws.data_ptr() if ws is not None else None, ws_bytes, _stream())
    return out


def kn_to_nk(q_weight: torch.Tensor, q_scale: torch.Tensor, k: int, bits: int, group_size: int):
    """KN-layout tensors (q_weight [nw, N], q_scale [ng, N]) -> the NK tensors every other entry point takes."""
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, torch.float16, "q_scale")
    n = _check_kn_shapes(q_weight, q_scale, k, bits, group_size)
    qw = torch.empty((n, q_weight.shape[0]), dtype=torch.int32, device=q_weight.device)
    qs = torch.empty((n, q_scale.shape[0]), dtype=torch.float16, device=q_weight.device)
    _lib.call("mi355gq_kn_to_nk", q_weight.data_ptr(), q_scale.data_ptr(), n, k, bits, group_size, qw.data_ptr(),
              qs.data_ptr(), _stream())
    return qw, qs


def nk_to_kn(q_weight: torch.Tensor, q_scale: torch.Tensor, k: int, bits: int, group_size: int):
    """NK tensors (q_weight [N, nw], q_scale [N, ng]) -> the KN layout of the `_0` schemes."""
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, torch.float16, "q_scale")
    n = q_weight.shape[0]
    _check_qshapes(q_weight, q_scale, (n,), k, bits, group_size)
    qw = torch.empty((q_weight.shape[1], n), dtype=torch.int32, device=q_weight.device)
    qs = torch.empty((q_scale.shape[1], n), dtype=torch.float16, device=q_weight.device)
    _lib.call("mi355gq_nk_to_kn", q_weight.data_ptr(), q_scale.data_ptr(), n, k, bits, group_size, qw.data_ptr(),
              qs.data_ptr(), _stream())
    return qw, qs


def dequantize_kn(q_weight: torch.Tensor, q_scale: torch.Tensor, k: int, bits: int, group_size: int) -> torch.Tensor:
    """GroupQuantize._dequantize along axis 0: KN tensors -> float16 [K, N]."""
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, torch.float16, "q_scale")
    n = _check_kn_shapes(q_weight, q_scale, k, bits, group_size)
    out = torch.empty((k, n), dtype=torch.float16, device=q_weight.device)
    _lib.call("mi355gq_dequantize_kn", q_weight.data_ptr(), q_scale.data_ptr(), n, k, bits, group_size, out.data_ptr(),
              _stream())
    return out


def _linear_other_dtype(x, q_weight, q_scale, bits, group_size, bias, out_dtype, out, residual):
    """linear() for float32 / bfloat16 models: x, q_scale and bias share the model dtype; the output is
    that dtype (the default here, whatever `out_dtype` defaults to for float16) or float32."""
    dt = x.dtype
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, dt, "q_scale")
    k = x.shape[-1]
    n = q_weight.shape[0]
    _check_qshapes(q_weight, q_scale, (n,), k, bits, group_size)
    m = 1
    for d in x.shape[:-1]:
        m *= d
    if bias is not None:
        _chk(bias, dt, "bias")
        if tuple(bias.shape) != (n,):
            raise ValueError(f"bias shape {tuple(bias.shape)}, expected {(n,)}")
    if out_dtype == torch.float16:  # the float16 default of the signature
        out_dtype = dt
    if out_dtype not in (dt, torch.float32):
        raise TypeError(f"out_dtype {out_dtype} for a {dt} model")
    if out is None:
        out = torch.empty((*x.shape[:-1], n), dtype=out_dtype, device=x.device)
    else:
        _chk(out, out_dtype, "out")
    if residual is not None:
        _chk(residual, dt, "residual")
        if tuple(residual.shape) != tuple(out.shape) or not residual.is_contiguous():
            raise ValueError(f"residual shape {tuple(residual.shape)}, expected contiguous {tuple(out.shape)}")
    ws_bytes = _lib.lib().mi355gq_linear_dt_workspace_bytes(m, n, k, bits, group_size, _MODEL_DTYPES[dt])
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    head = (x.data_ptr(), q_weight.data_ptr(), q_scale.data_ptr(), bias.data_ptr() if bias is not None else None)
    tail = (m, n, k, bits, group_size, _MODEL_DTYPES[dt], _MODEL_DTYPES[out_dtype], out.data_ptr(),
            ws.data_ptr() if ws is not None else None, ws_bytes, _stream())
    if residual is None:
        _lib.call("mi355gq_linear_dt", *head, *tail)
    else:
        _lib.call("mi355gq_linear_residual_dt", *head, residual.data_ptr(), *tail)
    return out


def _unsupported(err: _lib.Mi355gqError) -> bool:
    return err.code == _lib.ERR_UNSUPPORTED


def linear_silu_mul(x: torch.Tensor, q_weight: torch.Tensor, q_scale: torch.Tensor, bits: int,
                    group_size: int) -> torch.Tensor:
    """silu(x1) * x2 with x1, x2 = split(linear(x), 2, axis=-1): the gate_up projection of an MLP
    with its activation folded into the matmul kernel.  Bit-identical to linear then silu_mul;
    shapes without a fused kernel run exactly those two calls."""
    _chk(x, _FLOATS, "x")
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, x.dtype, "q_scale")
    k = x.shape[-1]
    n = q_weight.shape[0]
    _check_qshapes(q_weight, q_scale, (n,), k, bits, group_size)
    if n % 2:
        raise ValueError(f"linear_silu_mul: {n} rows cannot be split into gate and up halves")
    m = 1
    for d in x.shape[:-1]:
        m *= d
    out = torch.empty((*x.shape[:-1], n // 2), dtype=x.dtype, device=x.device)
    dt = _MODEL_DTYPES[x.dtype]
    ws_bytes = _lib.lib().mi355gq_linear_silu_mul_dt_workspace_bytes(m, n, k, bits, group_size, dt)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    try:
        _lib.call("mi355gq_linear_silu_mul_dt", x.data_ptr(), q_weight.data_ptr(), q_scale.data_ptr(), m, n, k,
                  bits, group_size, dt, out.data_ptr(), ws.data_ptr() if ws is not None else None, ws_bytes,
                  _stream())
    except _lib.Mi355gqError as err:
        if not _unsupported(err):
            raise
        return silu_mul(linear(x.reshape(m, k), q_weight, q_scale, bits, group_size)).reshape(out.shape)
    return out


def moe_gemv_routed_silu_mul(x: torch.Tensor, gate_logits: torch.Tensor, top_k: int, q_weight: torch.Tensor,
                             q_scale: torch.Tensor, bits: int, group_size: int):
    """One token: gating_softmax_topk and the e1_e3 expert matmul with silu(x1) * x3 folded in, in one launch.
    x [1, K], gate_logits [1, num_experts] (model dtype), q_weight [E, N, nw], q_scale [E, N, ng].  Returns
    (out [top_k, N / 2], expert_weights [1, top_k], expert_ids int32 [1, top_k]); raises Mi355gqError with
    ERR_UNSUPPORTED where the fused kernel does not apply (float32 models, top_k > 2, more than 64 experts)."""
    _chk(x, _FLOATS, "x")
    _chk(gate_logits, x.dtype, "gate_logits")
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, x.dtype, "q_scale")
    if x.dim() != 2 or x.shape[0] != 1 or gate_logits.dim() != 2 or gate_logits.shape[0] != 1:
        raise ValueError("moe_gemv_routed_silu_mul: x must be [1, K] and gate_logits [1, num_experts]")
    ne, n, _ = q_weight.shape
    k = x.shape[1]
    if gate_logits.shape[1] != ne:
        raise ValueError(f"moe_gemv_routed_silu_mul: {gate_logits.shape[1]} logits for {ne} experts")
    if n % 2:
        raise ValueError(f"moe_gemv_routed_silu_mul: {n} rows cannot be split into gate and up halves")
    _check_qshapes(q_weight, q_scale, (ne, n), k, bits, group_size)
    out = torch.empty((top_k, n // 2), dtype=x.dtype, device=x.device)
    weights = torch.empty((1, top_k), dtype=x.dtype, device=x.device)
    ids = torch.empty((1, top_k), dtype=torch.int32, device=x.device)
    _lib.call("mi355gq_moe_gemv_routed_silu_mul", x.data_ptr(), gate_logits.data_ptr(), ne, top_k, q_weight.data_ptr(),
              q_scale.data_ptr(), n, k, bits, group_size, _MODEL_DTYPES[x.dtype], weights.data_ptr(), ids.data_ptr(),
              out.data_ptr(), _stream())
    return out, weights, ids


def moe_gemv_combine(x: torch.Tensor, q_weight: torch.Tensor, q_scale: torch.Tensor, expert_ids: torch.Tensor,
                     expert_weights: torch.Tensor, bits: int, group_size: int) -> torch.Tensor:
    """One token: the e2 expert matmul on its top_k rows and the weighted sum over them, in one launch.
    x [top_k, K], expert_ids int32 [1, top_k], expert_weights [1, top_k] (model dtype), q_weight [E, N, nw],
    q_scale [E, N, ng].  Returns out [1, N]; raises Mi355gqError with ERR_UNSUPPORTED where the fused kernel does not
    apply (float32 models, top_k other than 2, short or very long K)."""
    _chk(x, _FLOATS, "x")
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, x.dtype, "q_scale")
    _chk(expert_ids, torch.int32, "expert_ids")
    _chk(expert_weights, x.dtype, "expert_weights")
    if x.dim() != 2 or expert_ids.dim() != 2 or expert_ids.shape[0] != 1 or tuple(expert_weights.shape) != tuple(expert_ids.shape):
        raise ValueError("moe_gemv_combine: x must be [top_k, K], expert_ids and expert_weights [1, top_k]")
    top_k = expert_ids.shape[1]
    if x.shape[0] != top_k:
        raise ValueError(f"moe_gemv_combine: {x.shape[0]} rows of x for {top_k} experts")
    ne, n, _ = q_weight.shape
    k = x.shape[1]
    _check_qshapes(q_weight, q_scale, (ne, n), k, bits, group_size)
    out = torch.empty((1, n), dtype=x.dtype, device=x.device)
    _lib.call("mi355gq_moe_gemv_combine", x.data_ptr(), q_weight.data_ptr(), q_scale.data_ptr(), n, k, bits, group_size,
              _MODEL_DTYPES[x.dtype], ne, expert_ids.data_ptr(), expert_weights.data_ptr(), top_k, out.data_ptr(),
              _stream())
    return out


def moe_gemv(x: torch.Tensor, q_weight: torch.Tensor, q_scale: torch.Tensor,
             expert_ids: torch.Tensor, bits: int, group_size: int, silu_mul_halves: bool = False
             ) -> torch.Tensor:
    """silu_mul_halves: the experts' rows are [gate; up] and the result is silu(gate) * up, [k, N / 2].
    x, q_scale and the result share the model dtype (float16, float32 or bfloat16)."""
    _chk(x, _FLOATS, "x")
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, x.dtype, "q_scale")
    _chk(expert_ids, torch.int32, "expert_ids")
    if x.dim() != 2 or expert_ids.dim() != 2 or expert_ids.shape[0] != 1:
        raise ValueError("moe_gemv: x must be [1|k, K] and expert_ids [1, k]")
    ne, n, _ = q_weight.shape
    k = x.shape[1]
    _check_qshapes(q_weight, q_scale, (ne, n), k, bits, group_size)
    top_k = expert_ids.shape[1]
    if x.dtype != torch.float16:
        dt_args = (x.data_ptr(), x.shape[0], q_weight.data_ptr(), q_scale.data_ptr(), expert_ids.data_ptr(), top_k, ne,
                   n, k, bits, group_size, _MODEL_DTYPES[x.dtype])
        if silu_mul_halves:
            if n % 2:
                raise ValueError(f"moe_gemv: {n} rows cannot be split into gate and up halves")
            out = torch.empty((top_k, n // 2), dtype=x.dtype, device=x.device)
            try:
                _lib.call("mi355gq_moe_gemv_silu_mul_dt", *dt_args, out.data_ptr(), _stream())
                return out
            except _lib.Mi355gqError as err:
                if not _unsupported(err):
                    raise
                return silu_mul(moe_gemv(x, q_weight, q_scale, expert_ids, bits, group_size))
        out = torch.empty((top_k, n), dtype=x.dtype, device=x.device)
        _lib.call("mi355gq_moe_gemv_dt", *dt_args, out.data_ptr(), _stream())
        return out
    args = (x.data_ptr(), x.shape[0], q_weight.data_ptr(), q_scale.data_ptr(), expert_ids.data_ptr(), top_k, ne,
            n, k, bits, group_size)
    if silu_mul_halves:
        if n % 2:
            raise ValueError(f"moe_gemv: {n} rows cannot be split into gate and up halves")
        out = torch.empty((top_k, n // 2), dtype=torch.float16, device=x.device)
        try:
            _lib.call("mi355gq_moe_gemv_silu_mul", *args, out.data_ptr(), _stream())
            return out
        except _lib.Mi355gqError as err:
            if not _unsupported(err):
                raise
            return silu_mul(moe_gemv(x, q_weight, q_scale, expert_ids, bits, group_size))
    out = torch.empty((top_k, n), dtype=torch.float16, device=x.device)
    _lib.call("mi355gq_moe_gemv", *args, out.data_ptr(), _stream())
    return out


def moe_group_gemm(x: torch.Tensor, q_weight: torch.Tensor, q_scale: torch.Tensor,
                   indptr: torch.Tensor, bits: int, group_size: int, silu_mul_halves: bool = False
                   ) -> torch.Tensor:
    """x, q_scale and the result share the model dtype (float16, float32 or bfloat16)."""
    _chk(x, _FLOATS, "x")
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, x.dtype, "q_scale")
    _chk(indptr, (torch.int32, torch.int64), "indptr")
    ne, n, _ = q_weight.shape
    rows, k = x.shape
    _check_qshapes(q_weight, q_scale, (ne, n), k, bits, group_size)
    if tuple(indptr.shape) != (ne + 1,):
        raise ValueError(f"indptr shape {tuple(indptr.shape)}, expected {(ne + 1,)}")
    if x.dtype != torch.float16:
        dt_args = (x.data_ptr(), rows, q_weight.data_ptr(), q_scale.data_ptr(), indptr.data_ptr(),
                   _lib.I64 if indptr.dtype == torch.int64 else _lib.I32, ne, n, k, bits, group_size,
                   _MODEL_DTYPES[x.dtype])
        if silu_mul_halves:
            if n % 2:
                raise ValueError(f"moe_group_gemm: {n} rows cannot be split into gate and up halves")
            out = torch.zeros((rows, n // 2), dtype=x.dtype, device=x.device)
            try:
                _lib.call("mi355gq_moe_group_gemm_silu_mul_dt", *dt_args, out.data_ptr(), _stream())
                return out
            except _lib.Mi355gqError as err:
                if not _unsupported(err):
                    raise
                return silu_mul(moe_group_gemm(x, q_weight, q_scale, indptr, bits, group_size))
        out = torch.zeros((rows, n), dtype=x.dtype, device=x.device)
        _lib.call("mi355gq_moe_group_gemm_dt", *dt_args, out.data_ptr(), _stream())
        return out
    args = (x.data_ptr(), rows, q_weight.data_ptr(), q_scale.data_ptr(), indptr.data_ptr(),
            _lib.I64 if indptr.dtype == torch.int64 else _lib.I32, ne, n, k, bits, group_size)
    if silu_mul_halves:
        if n % 2:
            raise ValueError(f"moe_group_gemm: {n} rows cannot be split into gate and up halves")
        out = torch.zeros((rows, n // 2), dtype=torch.float16, device=x.device)
        try:
            _lib.call("mi355gq_moe_group_gemm_silu_mul", *args, out.data_ptr(), _stream())
            return out
        except _lib.Mi355gqError as err:
            if not _unsupported(err):
                raise
            return silu_mul(moe_group_gemm(x, q_weight, q_scale, indptr, bits, group_size))
    out = torch.zeros((rows, n), dtype=torch.float16, device=x.device)
    _lib.call("mi355gq_moe_group_gemm", *args, out.data_ptr(), _stream())
    return out


def moe_experts(x: torch.Tensor, x_row_index: Optional[torch.Tensor], q_weight: torch.Tensor,
                q_scale: torch.Tensor, indptr: torch.Tensor, bits: int, group_size: int,
                silu_mul_halves: bool = False) -> torch.Tensor:
    """moe_group_gemm on x[x_row_index] (the layer's gather folded into the matmul's row addressing);
    x_row_index None: x is already in expert order.  Float16 and bfloat16 models; anything without such a
    kernel (float32 models, odd shapes) runs take_rows and moe_group_gemm."""
    _chk(x, _FLOATS, "x")
    _chk(q_weight, _STORAGE, "q_weight")
    _chk(q_scale, x.dtype, "q_scale")
    _chk(indptr, (torch.int32, torch.int64), "indptr")
    ne, n, _ = q_weight.shape
    x_rows, k = x.shape
    _check_qshapes(q_weight, q_scale, (ne, n), k, bits, group_size)
    if tuple(indptr.shape) != (ne + 1,):
        raise ValueError(f"indptr shape {tuple(indptr.shape)}, expected {(ne + 1,)}")
    rows = x_rows
    if x_row_index is not None:
        _chk(x_row_index, torch.int32, "x_row_index")
        rows = x_row_index.numel()
    if silu_mul_halves and n % 2:
        raise ValueError(f"moe_experts: {n} rows cannot be split into gate and up halves")
    out = torch.zeros((rows, n // 2 if silu_mul_halves else n), dtype=x.dtype, device=x.device)
    try:
        _lib.call("mi355gq_moe_experts_dt", x.data_ptr(), x_rows,
                  x_row_index.data_ptr() if x_row_index is not None else None, rows, q_weight.data_ptr(),
                  q_scale.data_ptr(), indptr.data_ptr(), _lib.I64 if indptr.dtype == torch.int64 else _lib.I32,
                  ne, n, k, bits, group_size, _lib.EPILOGUE_SILU_MUL if silu_mul_halves else _lib.EPILOGUE_NONE,
                  _MODEL_DTYPES[x.dtype], out.data_ptr(), _stream())
    except _lib.Mi355gqError as err:
        if not _unsupported(err):
            raise
        gathered = take_rows(x, x_row_index) if x_row_index is not None else x
        return moe_group_gemm(gathered, q_weight, q_scale, indptr, bits, group_size, silu_mul_halves)
    return out


def moe_route(logits: torch.Tensor, top_k: int, indptr_dtype=torch.int32):
    """The routing of a MoE layer in one launch.  Returns (weights [T, k] fp16, ids [T, k] int32,
    token_indices [T * k], reverse_indices [T * k], slot_positions [T * k], indptr [experts + 1]).
    Raises Mi355gqError with code ERR_UNSUPPORTED for batches past the single-workgroup form."""
    _chk(logits, _FLOATS, "logits")
    t, ne = logits.shape
    dev = logits.device
    w = torch.empty((t, top_k), dtype=logits.dtype, device=dev)
    ids = torch.empty((t, top_k), dtype=torch.int32, device=dev)
    tok, rev, pos = (torch.empty((t * top_k,), dtype=torch.int32, device=dev) for _ in range(3))
    indptr = torch.empty((ne + 1,), dtype=indptr_dtype, device=dev)
    _lib.call("mi355gq_moe_route_dt", logits.data_ptr(), t, ne, top_k, w.data_ptr(), ids.data_ptr(), tok.data_ptr(),
              rev.data_ptr(), pos.data_ptr(), indptr.data_ptr(),
              _lib.I64 if indptr_dtype == torch.int64 else _lib.I32, _MODEL_DTYPES[logits.dtype], _stream())
    return w, ids, tok, rev, pos, indptr


def moe_combine_sorted(y: torch.Tensor, slot_positions: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
    """y fp16 [T * k, H] in expert-sorted order, slot_positions int32 [T * k], weights fp16 [T, k] -> [T, H]."""
    _chk(y, _FLOATS, "y")
    _chk(slot_positions, torch.int32, "slot_positions")
    _chk(weights, y.dtype, "weights")
    t, k = weights.shape
    if y.shape[0] != t * k or slot_positions.numel() != t * k:
        raise ValueError("moe_combine_sorted: y and slot_positions must have T * k rows")
    h = y.shape[1]
    out = torch.empty((t, h), dtype=y.dtype, device=y.device)
    _lib.call("mi355gq_moe_combine_dt", y.data_ptr(), slot_positions.data_ptr(), weights.data_ptr(), t, k, h,
              out.data_ptr(), _MODEL_DTYPES[y.dtype], _stream())
    return out


def gating_softmax_topk(logits: torch.Tensor, top_k: int, norm_topk_prob: bool = True
                        ) -> Tuple[torch.Tensor, torch.Tensor]:
    _chk(logits, _FLOATS, "logits")
    t, ne = logits.shape
    w = torch.empty((t, top_k), dtype=logits.dtype, device=logits.device)
    ids = torch.empty((t, top_k), dtype=torch.int32, device=logits.device)
    _lib.call("mi355gq_gating_softmax_topk_ex", logits.data_ptr(), t, ne, top_k, 1 if norm_topk_prob else 0,
              _MODEL_DTYPES[logits.dtype], w.data_ptr(), ids.data_ptr(), _stream())
    return w, ids


def gating_topk(scores: torch.Tensor, top_k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    _chk(scores, _FLOATS, "scores")
    t, ne = scores.shape
    w = torch.empty((t, top_k), dtype=scores.dtype, device=scores.device)
    ids = torch.empty((t, top_k), dtype=torch.int32, device=scores.device)
    _lib.call("mi355gq_gating_topk", scores.data_ptr(), t, ne, top_k, w.data_ptr(), ids.data_ptr(),
              _MODEL_DTYPES[scores.dtype], _stream())
    return w, ids


def moe_cumsum(expert_indices: torch.Tensor, num_local_experts: int) -> torch.Tensor:
    _chk(expert_indices, torch.int32, "expert_indices")
    t, k = expert_indices.shape
    out = torch.empty((num_local_experts * t,), dtype=torch.int32, device=expert_indices.device)
    _lib.call("mi355gq_moe_cumsum", expert_indices.data_ptr(), t, k, num_local_experts,
              out.data_ptr(), _stream())
    return out


def get_indices(cumsum: torch.Tensor, expert_indices: torch.Tensor
                ) -> Tuple[torch.Tensor, torch.Tensor]:
    _chk(cumsum, torch.int32, "cumsum")
    _chk(expert_indices, torch.int32, "expert_indices")
    t, k = expert_indices.shape
    ne = cumsum.numel() // t if t else 1
    rev = torch.zeros((t * k,), dtype=torch.int32, device=cumsum.device)
    tok = torch.zeros((t * k,), dtype=torch.int32, device=cumsum.device)
    _lib.call("mi355gq_moe_get_indices", cumsum.data_ptr(), expert_indices.data_ptr(), t, k, ne,
              rev.data_ptr(), tok.data_ptr(), _stream())
    return rev, tok


def get_indptr(cumsum: torch.Tensor, num_local_experts: int, batch_size: int, inclusive: bool,
               out_dtype=torch.int32) -> torch.Tensor:
    _chk(cumsum, torch.int32, "cumsum")
    n = num_local_experts if inclusive else num_local_experts + 1
    out = torch.empty((n,), dtype=out_dtype, device=cumsum.device)
    _lib.call("mi355gq_moe_get_indptr", cumsum.data_ptr(), num_local_experts, batch_size,
              int(inclusive), _lib.I64 if out_dtype == torch.int64 else _lib.I32, out.data_ptr(),
              _stream())
    return out


def take_rows(x: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    _chk(x, _FLOATS, "x")
    _chk(indices, torch.int32, "indices")
    r, h = indices.numel(), x.shape[1]
    out = torch.zeros((r, h), dtype=x.dtype, device=x.device)
    _lib.call("mi355gq_take_rows_dt", x.data_ptr(), indices.data_ptr(), r, h, x.shape[0],
              out.data_ptr(), _MODEL_DTYPES[x.dtype], _stream())
    return out


def scatter_output(x: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    _chk(x, _FLOATS, "x")
    _chk(indices, torch.int32, "indices")
    r, h = x.shape
    out = torch.zeros_like(x)
    _lib.call("mi355gq_moe_scatter_output_dt", x.data_ptr(), indices.data_ptr(), r, h,
              out.data_ptr(), _MODEL_DTYPES[x.dtype], _stream())
    return out


def silu_mul(x: torch.Tensor) -> torch.Tensor:
    _chk(x, _FLOATS, "x")
    r, two_i = x.shape
    out = torch.empty((r, two_i // 2), dtype=x.dtype, device=x.device)
    _lib.call("mi355gq_silu_mul_dt", x.data_ptr(), r, two_i // 2, out.data_ptr(), _MODEL_DTYPES[x.dtype], _stream())
    return out


def moe_combine(y: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
    """y [T, k, H], weights [T, k] -> [T, H], all in the model dtype."""
    _chk(y, _FLOATS, "y")
    _chk(weights, y.dtype, "weights")
    t, k, h = y.shape
    out = torch.empty((t, h), dtype=y.dtype, device=y.device)
    _lib.call("mi355gq_moe_combine_dt", y.data_ptr(), None, weights.data_ptr(), t, k, h, out.data_ptr(),
              _MODEL_DTYPES[y.dtype], _stream())
    return out
