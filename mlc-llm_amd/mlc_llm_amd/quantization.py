"""Host-side mirror of the reference's group-quantization interface, over torch tensors.

Same names, argument meaning and error behaviour as
python/mlc_llm/quantization/group_quantization.py and quantization.py of the
reference; the arithmetic runs in the HIP library through `ops`.

* GroupQuantize            <- group_quantization.py:27-63  (+ quantize_weight :188-233,
                              quantize_model :65-153)
* QUANTIZATION             <- quantization.py:47-90 (the group-quant float16 entries)
* GroupQuantizeLinear      <- group_quantization.py:309-449
* GroupQuantizeEmbedding   <- group_quantization.py:452-556
* GroupQuantizeMixtralExperts <- group_quantization.py:559-660
* MixtralExperts           <- nn/expert.py:9-33 (parameter holder that quantize_model replaces)
* QuantizeMapping          <- loader/mapping.py (param_map / map_func)
"""

from __future__ import annotations

import dataclasses
from functools import partial
from typing import Callable, Dict, List, Literal, Optional

import torch
from torch import nn

from . import _lib, ops

_DTYPE_BITS = {"int3": 3, "int4": 4, "int8": 8, "uint32": 32}
_TORCH_DTYPE = {"float16": torch.float16, "float32": torch.float32, "bfloat16": torch.bfloat16}
MATMUL_MODEL_DTYPES = ("float16", "float32", "bfloat16")  # model dtypes with a linear kernel
MOE_MODEL_DTYPES = ("float16", "float32", "bfloat16")  # ... and with the expert matmuls


@dataclasses.dataclass
class QuantizeMapping:
    """param_map: fp name -> quantized names; map_func: fp name -> quantize function."""

    param_map: Dict[str, List[str]]
    map_func: Dict[str, Callable]


def is_final_fc(name: str) -> bool:
    """quantization/utils.py:51-54 of the reference."""
    return name in ["head", "lm_head", "lm_head.linear", "embed_out"]


def is_moe_gate(name: str, node: nn.Linear) -> bool:
    """quantization/utils.py:57-59 of the reference."""
    return name.endswith("gate") and isinstance(node.out_features, int) and node.out_features <= 256


@dataclasses.dataclass
class GroupQuantize:
    """Configuration for group quantization (same fields as the reference dataclass)."""

    name: str
    kind: str
    group_size: int
    quantize_dtype: Literal["int3", "int4", "int8"]
    storage_dtype: Literal["uint32"]
    model_dtype: Literal["float16", "float32", "bfloat16"]
    linear_weight_layout: Literal["KN", "NK"]
    quantize_embedding: bool = True
    quantize_final_fc: bool = True

    num_elem_per_storage: int = 0
    num_storage_per_group: int = 0
    max_int_value: int = 0
    tensor_parallel_shards: int = 0
    # tie rule of round() in quantize_weight: "half_away" is what TVM's llvm/rocm targets emit
    round_mode: Literal["half_away", "half_even"] = "half_away"

    def __post_init__(self):
        assert self.kind == "group-quant"
        assert self.quantize_dtype in ("int3", "int4", "int8")
        assert self.storage_dtype.startswith("uint")
        assert self.model_dtype in _TORCH_DTYPE
        qbits = _DTYPE_BITS[self.quantize_dtype]
        sbits = _DTYPE_BITS[self.storage_dtype]
        if sbits < qbits:
            raise ValueError("Storage unit should be greater or equal to quantized element")
        self.num_elem_per_storage = sbits // qbits
        if self.group_size % self.num_elem_per_storage != 0:
            raise ValueError("Group size should be divisible by numbers of elements per storage")
        self.num_storage_per_group = self.group_size // self.num_elem_per_storage
        self.max_int_value = (2 ** (qbits - 1)) - 1
        self.linear_quant_axis = 0 if self.linear_weight_layout == "KN" else 1

    @property
    def bits(self) -> int:
        return _DTYPE_BITS[self.quantize_dtype]

    def _require_built(self, matmul: bool = True):
        """Packing (quantize / dequantize / embedding take) exists for every model dtype of the
        registry; the dequantize-fused matmuls for those in MATMUL_MODEL_DTYPES."""
        if matmul and self.model_dtype not in MATMUL_MODEL_DTYPES:
            raise NotImplementedError(
                f"{self.name}: no gfx950 matmul kernel for model dtype {self.model_dtype} "
                f"(built: {', '.join(MATMUL_MODEL_DTYPES)}); quantize / dequantize / embedding are available"
            )

    def quantize_weight(self, weight: torch.Tensor, axis: int = -1, output_transpose: bool = False
                        ) -> List[torch.Tensor]:
        """Quantize `weight` along `axis` (must be the last axis): [q_weight, q_scale]."""
        self._require_built(matmul=False)
        weight = weight.to(_TORCH_DTYPE[self.model_dtype])
        axis = axis if axis >= 0 else weight.dim() + axis
        if axis != weight.dim() - 1:
            raise NotImplementedError("quantize_weight: only the last axis is supported (NK layout)")
        mode = _lib.ROUND_HALF_AWAY if self.round_mode == "half_away" else _lib.ROUND_HALF_EVEN
        qw, qs = ops.quantize(weight.contiguous(), self.bits, self.group_size, mode)
        if output_transpose:
            # the KN layouts store the same words and scales transposed (group_quantization.py:299-305)
            if qw.dim() != 2 or qs.dim() != 2:
                raise ValueError("Does not support transpose output quantized weight with ndim != 2")
            qw, qs = qw.t().contiguous(), qs.t().contiguous()
        return [qw, qs]

    def dequantize_weight(self, q_weight: torch.Tensor, q_scale: torch.Tensor, in_features: int
                          ) -> torch.Tensor:
        """GroupQuantize._dequantize over the last axis, out_shape [..., in_features]."""
        self._require_built(matmul=False)
        return ops.dequantize(q_weight, q_scale, in_features, self.bits, self.group_size)

    def quantize_model(self, model: nn.Module, quant_map: QuantizeMapping, name_prefix: str
                       ) -> nn.Module:
        """Replace Linear / Embedding / MixtralExperts by their quantized twins, record names."""
        config = self

        def visit(prefix: str, module: nn.Module) -> nn.Module:
            for child_name, child in list(module.named_children()):
                name = f"{prefix}.{child_name}" if prefix else child_name
                new = replace(name, child)
                if new is not child:
                    setattr(module, child_name, new)
            return module

        def replace(name: str, node: nn.Module) -> nn.Module:
            if getattr(node, "no_quantization", False):
                return node
            if (
                isinstance(node, nn.Linear)
                and (not is_final_fc(name) or config.quantize_final_fc)
                and not is_moe_gate(name, node)
            ):
                weight_name = f"{name}.weight"
                quant_map.param_map[weight_name] = [f"{name}.q_weight", f"{name}.q_scale"]
                quant_map.map_func[weight_name] = partial(
                    config.quantize_weight, output_transpose=config.linear_weight_layout == "KN"
                )
                return GroupQuantizeLinear.from_linear(node, config)
            if isinstance(node, nn.Embedding) and config.quantize_embedding:
                weight_name = f"{name}.weight"
                quant_map.param_map[weight_name] = [f"{name}.q_weight", f"{name}.q_scale"]
                quant_map.map_func[weight_name] = config.quantize_weight
                return GroupQuantizeEmbedding.from_embedding(node, config)
            if isinstance(node, MixtralExperts):
                weight_name = f"{name}.weight"
                quant_map.param_map[weight_name] = [f"{name}.q_weight", f"{name}.q_scale"]
                quant_map.map_func[weight_name] = config.quantize_weight
                return GroupQuantizeMixtralExperts.from_mixtral_experts(node, config)
            return visit(name, node)

        return visit(name_prefix, model)


def _ceildiv(a: int, b: int) -> int:
    return -(-a // b)


def _storage_param(shape, device) -> nn.Parameter:
    return nn.Parameter(torch.zeros(shape, dtype=torch.int32, device=device), requires_grad=False)


def _float_param(shape, dtype, device) -> nn.Parameter:
    return nn.Parameter(torch.zeros(shape, dtype=dtype, device=device), requires_grad=False)


class GroupQuantizeLinear(nn.Module):
    """An nn.Linear with group-quantized weight: q_weight [N, nw], q_scale [N, ng] (NK)."""

    def __init__(self, in_features: int, out_features: int, config: GroupQuantize,
                 bias: bool = True, out_dtype: Optional[str] = None, device=None) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.out_dtype = out_dtype
        self.config = config
        num_group = _ceildiv(in_features, config.group_size)
        num_shards = config.tensor_parallel_shards
        if num_shards > 1 and (in_features * num_shards // config.group_size) % num_shards != 0:
            raise ValueError(
                f"The linear dimension {in_features * num_shards} has "
                f"{in_features * num_shards // config.group_size} groups under group size "
                f"{config.group_size}. The groups cannot be evenly distributed on "
                f"{num_shards} GPUs.\n"
                "Possible solutions: reduce number of GPUs, or use quantization with smaller "
                "group size."
            )
        model_dtype = _TORCH_DTYPE[config.model_dtype]
        if config.linear_weight_layout == "KN":
            self.q_weight = _storage_param(
                (config.num_storage_per_group * num_group, out_features), device)
            self.q_scale = _float_param((num_group, out_features), model_dtype, device)
        else:
            self.q_weight = _storage_param(
                (out_features, config.num_storage_per_group * num_group), device)
            self.q_scale = _float_param((out_features, num_group), model_dtype, device)
        if bias:
            bias_dtype = model_dtype if out_dtype is None else _TORCH_DTYPE[out_dtype]
            self.bias = _float_param((out_features,), bias_dtype, device)
        else:
            self.bias = None

    @staticmethod
    def from_linear(src: nn.Linear, config: GroupQuantize) -> "GroupQuantizeLinear":
        out_features, in_features = src.weight.shape
        return GroupQuantizeLinear(
            in_features=in_features,
            out_features=out_features,
            config=config,
            bias=getattr(src, "bias", None) is not None,
            out_dtype=getattr(src, "out_dtype", None),
            device=src.weight.device,
        )

    def _nk_tensors(self):
        """(q_weight, q_scale) in the [N, ...] layout the kernels stream.  A KN-layout module
        (q4f16_0 / q3f16_0: the same words and scales, transposed) keeps a transposed copy, made
        on the device the first time it is needed and again after load_state_dict or when the
        parameter tensors are replaced; writing into them in place (`.data.copy_`) needs
        `invalidate_layout_cache()`."""
        if self.config.linear_weight_layout == "NK":
            return self.q_weight, self.q_scale
        key = (self.q_weight.data_ptr(), self.q_scale.data_ptr())
        if getattr(self, "_nk_key", None) != key:
            if self.q_scale.dtype == torch.float16 and self.q_weight.is_cuda:
                self._nk = ops.kn_to_nk(self.q_weight.detach(), self.q_scale.detach(), self.in_features,
                                        self.config.bits, self.config.group_size)
            else:
                self._nk = (self.q_weight.detach().t().contiguous(), self.q_scale.detach().t().contiguous())
            self._nk_key = key
        return self._nk

    def invalidate_layout_cache(self) -> None:
        self._nk_key = None
        self._nk = None

    def _load_from_state_dict(self, *args, **kwargs):
        super()._load_from_state_dict(*args, **kwargs)
        self.invalidate_layout_cache()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        self.config._require_built()
        model_dtype = _TORCH_DTYPE[self.config.model_dtype]
        out_dtype = model_dtype if self.out_dtype is None else _TORCH_DTYPE[self.out_dtype]
        bias = self.bias
        rows = x.numel() // max(x.shape[-1], 1)
        if (self.config.linear_weight_layout == "KN" and model_dtype == torch.float16 and rows <= 8
                and self.out_features % 4 == 0 and (bias is None or bias.dtype == model_dtype)):
            # decode batches of a KN-layout model: the stored tensors are streamed as they are
            return ops.linear_kn(x, self.q_weight, self.q_scale, self.config.bits, self.config.group_size, bias, out_dtype)
        q_weight, q_scale = self._nk_tensors()
        if bias is not None and bias.dtype != model_dtype:
            # fp32 bias with fp32 output: added after the kernel, as the reference's `x + bias`
            y = ops.linear(x, q_weight, q_scale, self.config.bits, self.config.group_size, None, out_dtype)
            return y + bias
        return ops.linear(x, q_weight, q_scale, self.config.bits, self.config.group_size, bias, out_dtype)

    def forward_silu_mul(self, x: torch.Tensor) -> torch.Tensor:
        """For a gate_up projection: `x1, x2 = split(self(x), 2, axis=-1); silu(x1) * x2` of the MLP
        (model/llama/llama_model.py:122-125) in one kernel; same bits as the two steps."""
        self.config._require_built()
        if self.bias is not None or self.out_dtype not in (None, self.config.model_dtype):
            return ops.silu_mul(self.forward(x).reshape(-1, self.out_features)).reshape(*x.shape[:-1], -1)
        q_weight, q_scale = self._nk_tensors()
        return ops.linear_silu_mul(x, q_weight, q_scale, self.config.bits, self.config.group_size)


class GroupQuantizeEmbedding(nn.Module):
    """An nn.Embedding with group-quantized table, usable as tied lm_head."""

    def __init__(self, num: int, dim: int, config: GroupQuantize, device=None):
        super().__init__()
        self.num = num
        self.dim = dim
        self.config = config
        num_group = _ceildiv(dim, config.group_size)
        self.q_weight = _storage_param((num, config.num_storage_per_group * num_group), device)
        self.q_scale = _float_param((num, num_group), _TORCH_DTYPE[config.model_dtype], device)

    @staticmethod
    def from_embedding(embedding: nn.Embedding, config: GroupQuantize) -> "GroupQuantizeEmbedding":
        num, dim = embedding.weight.shape
        return GroupQuantizeEmbedding(num, dim, config, device=embedding.weight.device)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        self.config._require_built(matmul=False)
        ids = x.reshape(-1).to(torch.int32).contiguous()
        out = ops.embedding_take(ids, self.q_weight, self.q_scale, self.dim, self.config.bits,
                                 self.config.group_size)
        return out.reshape(*x.shape, self.dim)

    def lm_head_forward(self, x: torch.Tensor) -> torch.Tensor:
        """Dequantize the table and multiply: logits in float32."""
        self.config._require_built()
        return ops.linear(x, self.q_weight, self.q_scale, self.config.bits, self.config.group_size,
                          None, torch.float32)


class MixtralExperts(nn.Module):
    """Unquantized expert stack [num_local_experts, out_features, in_features] (holder only)."""

    def __init__(self, num_local_experts, in_features, out_features, tensor_parallel_shards=1,
                 device=None):
        super().__init__()
        self.num_local_experts = num_local_experts
        self.in_features = in_features
        self.out_features = out_features
        self.tensor_parallel_shards = tensor_parallel_shards
        self.weight = nn.Parameter(
            torch.zeros((num_local_experts, out_features, in_features), dtype=torch.float16,
                        device=device), requires_grad=False)


class GroupQuantizeMixtralExperts(nn.Module):
    """MixtralExperts with group-quantized weights [Ne, N, nw] / [Ne, N, ng]."""

    def __init__(self, num_local_experts, in_features, out_features, config: GroupQuantize,
                 device=None):
        super().__init__()
        self.num_local_experts = num_local_experts
        self.in_features = in_features
        self.out_features = out_features
        self.config = config
        num_group = _ceildiv(in_features, config.group_size)
        self.q_weight = _storage_param(
            (num_local_experts, out_features, config.num_storage_per_group * num_group), device)
        self.q_scale = _float_param((num_local_experts, out_features, num_group),
                                    _TORCH_DTYPE[config.model_dtype], device)
        self.quantize_dtype = config.quantize_dtype
        self.group_size = config.group_size
        self.dtype = config.model_dtype
        if config.linear_weight_layout == "KN":
            raise NotImplementedError("GroupQuantizeMixtralExperts does not support KN layout now.")

    @staticmethod
    def from_mixtral_experts(src: MixtralExperts, config: GroupQuantize
                             ) -> "GroupQuantizeMixtralExperts":
        return GroupQuantizeMixtralExperts(
            num_local_experts=src.num_local_experts,
            in_features=src.in_features,
            out_features=src.out_features,
            config=config,
            device=src.weight.device,
        )

    def forward(self, x: torch.Tensor, indptr: torch.Tensor, silu_mul_halves: bool = False) -> torch.Tensor:
        """2-D `indptr` [1, k] holds the selected expert ids (single token); 1-D is a true indptr.
        silu_mul_halves: return silu(x1) * x3 of the two halves of the output (the e1_e3 stack of
        mixtral_model.py:64-68) from the same kernel."""
        assert x.dim() == 2
        if self.config.model_dtype not in MOE_MODEL_DTYPES:
            raise NotImplementedError(f"{self.config.name}: the expert matmuls are built for {MOE_MODEL_DTYPES} models")
        if indptr.dim() == 2:
            assert indptr.shape[0] == 1
            return ops.moe_gemv(x, self.q_weight, self.q_scale, indptr, self.config.bits,
                                self.group_size, silu_mul_halves)
        assert indptr.dim() == 1
        return ops.moe_group_gemm(x, self.q_weight, self.q_scale, indptr, self.config.bits,
                                  self.group_size, silu_mul_halves)


def _group(name: str, group_size: int, qdtype: str, layout: str, model_dtype: str = "float16",
           embedding_and_final_fc: bool = True):
    return GroupQuantize(
        name=name,
        kind="group-quant",
        group_size=group_size,
        quantize_dtype=qdtype,
        storage_dtype="uint32",
        model_dtype=model_dtype,
        linear_weight_layout=layout,
        quantize_embedding=embedding_and_final_fc,
        quantize_final_fc=embedding_and_final_fc,
    )


# The group-quant entries of the reference registry (quantization.py:47-90).  The KN-layout
# entries hold the NK tensors transposed; their linears run the NK kernels on a transposed copy.
QUANTIZATION: Dict[str, GroupQuantize] = {
    "q3f16_0": _group("q3f16_0", 40, "int3", "KN"),
    "q3f16_1": _group("q3f16_1", 40, "int3", "NK"),
    "q4f16_0": _group("q4f16_0", 32, "int4", "KN"),
    "q4f16_1": _group("q4f16_1", 32, "int4", "NK"),
    # q4f16_1 that leaves the embedding and the final fc unquantized (quantization.py:124-134)
    "q4f16_2": _group("q4f16_2", 32, "int4", "NK", embedding_and_final_fc=False),
    # other model dtypes (quantization.py:91-123): packing built, matmuls per MATMUL_MODEL_DTYPES
    "q4bf16_0": _group("q4bf16_0", 32, "int4", "KN", "bfloat16"),
    "q4bf16_1": _group("q4bf16_1", 32, "int4", "NK", "bfloat16"),
    "q4f32_1": _group("q4f32_1", 32, "int4", "NK", "float32"),
}
