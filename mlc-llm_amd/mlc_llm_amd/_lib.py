"""ctypes binding of libmi355gq.so (the C ABI declared in include/mi355gq.h).

There is no fallback: if the shared library is missing or a call fails, an
exception is raised.  Tensors are torch tensors on the ROCm device; only their
`data_ptr()` and the current HIP stream cross the boundary.
"""

from __future__ import annotations

import ctypes
import os
import re
from ctypes import c_char_p, c_int, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libmi355gq.so")
HEADER_PATH = os.path.join(os.path.dirname(os.path.dirname(_HERE)), "include", "mi355gq.h")

OK = 0
ERR_ARG, ERR_HIP, ERR_UNSUPPORTED, ERR_WORKSPACE = -1, -2, -3, -4
F16, F32, BF16 = 0, 1, 2
ROUND_HALF_AWAY, ROUND_HALF_EVEN = 0, 1
I32, I64 = 0, 1
EPILOGUE_NONE, EPILOGUE_SILU_MUL = 0, 1

_P, _I, _L = c_void_p, c_int, c_int64

# name -> (restype, argtypes); mirrors include/mi355gq.h one to one
SIGNATURES = {
    "mi355gq_version": (_I, []),
    "mi355gq_last_error": (c_char_p, []),
    "mi355gq_check_device": (_I, []),
    "mi355gq_quantize": (_I, [_P, _L, _L, _I, _I, _I, _P, _P, _P]),
    "mi355gq_dequantize": (_I, [_P, _P, _L, _L, _I, _I, _P, _P]),
    "mi355gq_quantize_dt": (_I, [_P, _L, _L, _I, _I, _I, _I, _P, _P, _P]),
    "mi355gq_dequantize_dt": (_I, [_P, _P, _L, _L, _I, _I, _I, _P, _P]),
    "mi355gq_embedding_take_dt": (_I, [_P, _L, _P, _P, _L, _L, _I, _I, _I, _P, _P]),
    "mi355gq_linear_residual_dt": (_I, [_P, _P, _P, _P, _P, _L, _L, _L, _I, _I, _I, _I, _P, _P, _L, _P]),
    "mi355gq_linear_dt_workspace_bytes": (_L, [_L, _L, _L, _I, _I, _I]),
    "mi355gq_linear_dt": (_I, [_P, _P, _P, _P, _L, _L, _L, _I, _I, _I, _I, _P, _P, _L, _P]),
    "mi355gq_embedding_take": (_I, [_P, _L, _P, _P, _L, _L, _I, _I, _P, _P]),
    "mi355gq_linear_workspace_bytes": (_L, [_L, _L, _L, _I, _I]),
    "mi355gq_linear": (_I, [_P, _P, _P, _P, _L, _L, _L, _I, _I, _I, _P, _P, _L, _P]),
    "mi355gq_linear_static_scratch_max_bytes": (_L, []),
    "mi355gq_linear_static_scratch_init": (_I, []),
    "mi355gq_linear_static_scratch": (_I, [_P, _P, _P, _P, _L, _L, _L, _I, _I, _I, _P, _P]),
    "mi355gq_kn_to_nk": (_I, [_P, _P, _L, _L, _I, _I, _P, _P, _P]),
    "mi355gq_nk_to_kn": (_I, [_P, _P, _L, _L, _I, _I, _P, _P, _P]),
    "mi355gq_dequantize_kn": (_I, [_P, _P, _L, _L, _I, _I, _P, _P]),
    "mi355gq_linear_kn_workspace_bytes": (_L, [_L, _L, _L, _I, _I]),
    "mi355gq_linear_kn": (_I, [_P, _P, _P, _P, _L, _L, _L, _I, _I, _I, _P, _P, _L, _P]),
    "mi355gq_linear_residual": (_I, [_P, _P, _P, _P, _P, _L, _L, _L, _I, _I, _I, _P, _P, _L, _P]),
    "mi355gq_linear_silu_mul_workspace_bytes": (_L, [_L, _L, _L, _I, _I]),
    "mi355gq_linear_silu_mul": (_I, [_P, _P, _P, _L, _L, _L, _I, _I, _P, _P, _L, _P]),
    "mi355gq_moe_gemv_silu_mul": (_I, [_P, _L, _P, _P, _P, _L, _L, _L, _L, _I, _I, _P, _P]),
    "mi355gq_moe_gemv_routed_silu_mul": (_I, [_P, _P, _L, _L, _P, _P, _L, _L, _I, _I, _I, _P, _P, _P, _P]),
    "mi355gq_moe_gemv_combine": (_I, [_P, _P, _P, _L, _L, _I, _I, _I, _L, _P, _P, _L, _P, _P]),
    "mi355gq_moe_group_gemm_silu_mul": (_I, [_P, _L, _P, _P, _P, _I, _L, _L, _L, _I, _I, _P, _P]),
    "mi355gq_linear_silu_mul_dt_workspace_bytes": (_L, [_L, _L, _L, _I, _I, _I]),
    "mi355gq_linear_silu_mul_dt": (_I, [_P, _P, _P, _L, _L, _L, _I, _I, _I, _P, _P, _L, _P]),
    "mi355gq_moe_gemv_silu_mul_dt": (_I, [_P, _L, _P, _P, _P, _L, _L, _L, _L, _I, _I, _I, _P, _P]),
    "mi355gq_moe_group_gemm_silu_mul_dt": (_I, [_P, _L, _P, _P, _P, _I, _L, _L, _L, _I, _I, _I, _P, _P]),
    "mi355gq_moe_experts_dt": (_I, [_P, _L, _P, _L, _P, _P, _P, _I, _L, _L, _L, _I, _I, _I, _I, _P, _P]),
    "mi355gq_gating_softmax_topk_dt": (_I, [_P, _L, _L, _L, _P, _P, _I, _P]),
    "mi355gq_moe_route_dt": (_I, [_P, _L, _L, _L, _P, _P, _P, _P, _P, _P, _I, _I, _P]),
    "mi355gq_take_rows_dt": (_I, [_P, _P, _L, _L, _L, _P, _I, _P]),
    "mi355gq_moe_scatter_output_dt": (_I, [_P, _P, _L, _L, _P, _I, _P]),
    "mi355gq_silu_mul_dt": (_I, [_P, _L, _L, _P, _I, _P]),
    "mi355gq_moe_combine_dt": (_I, [_P, _P, _P, _L, _L, _L, _P, _I, _P]),
    "mi355gq_moe_gemv_dt": (_I, [_P, _L, _P, _P, _P, _L, _L, _L, _L, _I, _I, _I, _P, _P]),
    "mi355gq_moe_group_gemm_dt": (_I, [_P, _L, _P, _P, _P, _I, _L, _L, _L, _I, _I, _I, _P, _P]),
    "mi355gq_moe_gemv": (_I, [_P, _L, _P, _P, _P, _L, _L, _L, _L, _I, _I, _P, _P]),
    "mi355gq_moe_group_gemm": (_I, [_P, _L, _P, _P, _P, _I, _L, _L, _L, _I, _I, _P, _P]),
    "mi355gq_moe_experts": (_I, [_P, _L, _P, _L, _P, _P, _P, _I, _L, _L, _L, _I, _I, _I, _P, _P]),
    "mi355gq_moe_route": (_I, [_P, _L, _L, _L, _P, _P, _P, _P, _P, _P, _I, _P]),
    "mi355gq_moe_combine_sorted": (_I, [_P, _P, _P, _L, _L, _L, _P, _P]),
    "mi355gq_gating_softmax_topk": (_I, [_P, _L, _L, _L, _P, _P, _P]),
    "mi355gq_gating_topk": (_I, [_P, _L, _L, _L, _P, _P, _I, _P]),
    "mi355gq_gating_softmax_topk_ex": (_I, [_P, _L, _L, _L, _I, _I, _P, _P, _P]),
    "mi355gq_moe_cumsum": (_I, [_P, _L, _L, _L, _P, _P]),
    "mi355gq_moe_get_indices": (_I, [_P, _P, _L, _L, _L, _P, _P, _P]),
    "mi355gq_moe_get_indptr": (_I, [_P, _L, _L, _I, _I, _P, _P]),
    "mi355gq_take_rows": (_I, [_P, _P, _L, _L, _L, _P, _P]),
    "mi355gq_moe_scatter_output": (_I, [_P, _P, _L, _L, _P, _P]),
    "mi355gq_silu_mul": (_I, [_P, _L, _L, _P, _P]),
    "mi355gq_moe_combine": (_I, [_P, _P, _L, _L, _L, _P, _P]),
}


# exported for tests and tuning sweeps only (csrc/gq_testing.h); not declared in the public header
TEST_HOOKS = {
    "mi355gq_testing_set_option": (_I, [c_char_p, _I]),
    "mi355gq_testing_last_kernel": (c_char_p, []),
    "mi355gq_testing_stream_read": (_I, [_P, _L, _P, _L, _P, _P]),
}


class Mi355gqError(RuntimeError):
    """A C-ABI call returned a non-zero code."""

    def __init__(self, func: str, code: int, message: str):
        super().__init__(f"{func} failed ({code}): {message}")
        self.code = code
        self.message = message


_LIB = None


def declared_symbols() -> list[str]:
    """Names of the entry points declared in include/mi355gq.h."""
    with open(HEADER_PATH, encoding="utf-8") as f:
        text = f.read()
    return sorted(set(re.findall(r"MI355GQ_API\s+[\w\s\*]+?\b(mi355gq_\w+)\s*\(", text)))


def lib() -> ctypes.CDLL:
    """Load the shared library (once).  Raises if it has not been built."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python mlc-llm_amd/build.py` "
                "(there is no non-HIP fallback)"
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in {**SIGNATURES, **TEST_HOOKS}.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _LIB = handle
    return _LIB


def call(name: str, *args) -> None:
    """Invoke an int-returning entry point; raise Mi355gqError on failure."""
    handle = lib()
    rc = getattr(handle, name)(*args)
    if rc != OK:
        raise Mi355gqError(name, rc, handle.mi355gq_last_error().decode("utf-8", "replace"))


def last_kernel() -> str:
    """Test / measurement hook: the kernel instantiation this thread's last matmul call launched."""
    return lib().mi355gq_testing_last_kernel().decode()


def set_option(name: str, value: int) -> None:
    """Test / tuning hook (csrc/gq_testing.h): force a kernel family or launch shape for later calls of THIS
    thread; a negative value restores the heuristic."""
    call("mi355gq_testing_set_option", name.encode(), int(value))
