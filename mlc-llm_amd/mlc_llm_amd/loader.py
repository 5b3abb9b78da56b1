"""HuggingFace checkpoint -> MLC parameters for the Llama / Mistral, Mixtral, Qwen2 / Qwen3, Gemma / Gemma2 and
Phi-3 families, quantised on the GPU while loading, written as an MLC weight directory.

Mirrors the reference's conversion path for exactly the parameters this package's kernels
consume:

* parameter correspondence: ``ExternMapping`` (python/mlc_llm/loader/mapping.py), the standard
  HF mapping of Llama (q/k/v and gate/up concatenated along the output dimension,
  python/mlc_llm/loader/standard_loader.py:89-134) and Mixtral's expert stacking
  (python/mlc_llm/model/mixtral/mixtral_loader.py:44-104: ``e1_e3[e] = concat(w1_e, w3_e)``,
  ``e2[e] = w2_e``, the router ``gate`` passes through);
* which parameters are quantised: every Linear except the MoE router, the embedding, the final
  projection, and the stacked experts (python/mlc_llm/quantization/group_quantization.py:113-150),
  each becoming ``<name>.q_weight`` / ``<name>.q_scale``;
* load -> map -> quantise -> yield, one MLC parameter at a time
  (python/mlc_llm/loader/huggingface_loader.py:102-185), then ``dump_tensor_cache`` with the
  reference's metadata block (python/mlc_llm/interface/convert_weight.py:175-196).

The model definitions themselves are not part of this package, so the MLC parameter lists are
written out here from the reference's module trees (python/mlc_llm/model/llama/llama_model.py:106-253,
python/mlc_llm/model/mixtral/mixtral_model.py:32-62).
"""

from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, Callable, Dict, Iterator, List, Optional, Set, Tuple

import numpy as np
import torch

from .quantization import QUANTIZATION, GroupQuantize
from .tensor_cache import dump_tensor_cache


@dataclasses.dataclass
class ExternMapping:
    """MLC parameter name -> the source names it is built from and the function that builds it."""

    param_map: Dict[str, List[str]] = dataclasses.field(default_factory=dict)
    map_func: Dict[str, Callable[..., np.ndarray]] = dataclasses.field(default_factory=dict)
    unused_params: Set[str] = dataclasses.field(default_factory=set)

    def add_mapping(self, map_from: str, map_to: List[str], func: Callable[..., np.ndarray]) -> None:
        self.param_map[map_from] = map_to
        self.map_func[map_from] = func

    def add_unused(self, name: str) -> None:
        self.unused_params.add(name)


def _concat0(*parts: np.ndarray) -> np.ndarray:
    return np.concatenate(parts, axis=0)


def _identity(x: np.ndarray) -> np.ndarray:
    return x


def _cfg(config: Dict[str, Any], key: str, default=None):
    if key in config:
        return config[key]
    if default is None:
        raise KeyError(f"model config lacks {key!r}")
    return default


def _attention_and_norms(mapping: ExternMapping, quantized: List[str], i: int) -> None:
    attn = f"model.layers.{i}.self_attn"
    mapping.add_mapping(f"{attn}.qkv_proj.weight",
                        [f"{attn}.q_proj.weight", f"{attn}.k_proj.weight", f"{attn}.v_proj.weight"],
                        _concat0)
    mapping.add_mapping(f"{attn}.o_proj.weight", [f"{attn}.o_proj.weight"], _identity)
    quantized += [f"{attn}.qkv_proj.weight", f"{attn}.o_proj.weight"]
    mapping.add_unused(f"{attn}.rotary_emb.inv_freq")
    for norm in ("input_layernorm", "post_attention_layernorm"):
        name = f"model.layers.{i}.{norm}.weight"
        mapping.add_mapping(name, [name], _identity)


def llama_huggingface(config: Dict[str, Any]) -> Tuple[ExternMapping, List[str]]:
    """(mapping, names of the MLC parameters that group quantisation replaces) for
    ``LlamaForCausalLM``; parameter order is the module tree's."""
    mapping, quantized = ExternMapping(), []
    mapping.add_mapping("model.embed_tokens.weight", ["model.embed_tokens.weight"], _identity)
    quantized.append("model.embed_tokens.weight")
    for i in range(_cfg(config, "num_hidden_layers")):
        _attention_and_norms(mapping, quantized, i)
        mlp = f"model.layers.{i}.mlp"
        mapping.add_mapping(f"{mlp}.gate_up_proj.weight",
                            [f"{mlp}.gate_proj.weight", f"{mlp}.up_proj.weight"], _concat0)
        mapping.add_mapping(f"{mlp}.down_proj.weight", [f"{mlp}.down_proj.weight"], _identity)
        quantized += [f"{mlp}.gate_up_proj.weight", f"{mlp}.down_proj.weight"]
    mapping.add_mapping("model.norm.weight", ["model.norm.weight"], _identity)
    if not config.get("tie_word_embeddings", False):
        mapping.add_mapping("lm_head.weight", ["lm_head.weight"], _identity)
        quantized.append("lm_head.weight")
    else:
        mapping.add_unused("lm_head.weight")
    return mapping, quantized


def mixtral_huggingface(config: Dict[str, Any]) -> Tuple[ExternMapping, List[str]]:
    """Same for ``MixtralForCausalLM``: experts stacked, router left in floating point."""
    mapping, quantized = ExternMapping(), []
    ne = _cfg(config, "num_local_experts")
    mapping.add_mapping("model.embed_tokens.weight", ["model.embed_tokens.weight"], _identity)
    quantized.append("model.embed_tokens.weight")

    def gate_up_stack(*parts: np.ndarray) -> np.ndarray:
        return np.stack([np.concatenate([parts[2 * e], parts[2 * e + 1]], axis=0)
                         for e in range(len(parts) // 2)], axis=0)

    def stack(*parts: np.ndarray) -> np.ndarray:
        return np.stack(parts, axis=0)

    for i in range(_cfg(config, "num_hidden_layers")):
        _attention_and_norms(mapping, quantized, i)
        hf, mlc = f"model.layers.{i}.block_sparse_moe", f"model.layers.{i}.moe"
        mapping.add_mapping(f"{mlc}.gate.weight", [f"{hf}.gate.weight"], _identity)  # never quantised
        src: List[str] = []
        for e in range(ne):
            src += [f"{hf}.experts.{e}.w1.weight", f"{hf}.experts.{e}.w3.weight"]
        mapping.add_mapping(f"{mlc}.e1_e3.weight", src, gate_up_stack)
        mapping.add_mapping(f"{mlc}.e2.weight", [f"{hf}.experts.{e}.w2.weight" for e in range(ne)], stack)
        quantized += [f"{mlc}.e1_e3.weight", f"{mlc}.e2.weight"]
    mapping.add_mapping("model.norm.weight", ["model.norm.weight"], _identity)
    if not config.get("tie_word_embeddings", False):
        mapping.add_mapping("lm_head.weight", ["lm_head.weight"], _identity)
        quantized.append("lm_head.weight")
    else:
        mapping.add_unused("lm_head.weight")
    return mapping, quantized


def _plus_one(x: np.ndarray) -> np.ndarray:
    return (x.astype(np.float32) + 1.0).astype(x.dtype)


def _standard_decoder(config: Dict[str, Any], *, qkv_target: str = "qkv_proj", qkv_bias: bool = False,
                      qk_norm: bool = False, norm_plus_one: bool = False, always_tied: bool = False,
                      layer_norms: Tuple[str, ...] = ("input_layernorm", "post_attention_layernorm"),
                      ) -> Tuple[ExternMapping, List[str]]:
    """The reference's standard HF mapping (python/mlc_llm/loader/standard_loader.py:22-167) over a decoder
    whose layers hold ``self_attn.<qkv_target>`` (+ bias), ``self_attn.o_proj``, optional per-head
    ``q_norm`` / ``k_norm``, ``mlp.gate_up_proj`` / ``mlp.down_proj`` and the given RMSNorm weights;
    parameter order follows the module trees (attention, MLP, norms)."""
    mapping, quantized = ExternMapping(), []
    norm_func = _plus_one if norm_plus_one else _identity
    mapping.add_mapping("model.embed_tokens.weight", ["model.embed_tokens.weight"], _identity)
    quantized.append("model.embed_tokens.weight")
    for i in range(_cfg(config, "num_hidden_layers")):
        attn, mlp = f"model.layers.{i}.self_attn", f"model.layers.{i}.mlp"
        mapping.add_mapping(f"{attn}.{qkv_target}.weight",
                            [f"{attn}.q_proj.weight", f"{attn}.k_proj.weight", f"{attn}.v_proj.weight"], _concat0)
        quantized.append(f"{attn}.{qkv_target}.weight")
        if qkv_bias:
            mapping.add_mapping(f"{attn}.{qkv_target}.bias",
                                [f"{attn}.q_proj.bias", f"{attn}.k_proj.bias", f"{attn}.v_proj.bias"], _concat0)
        mapping.add_mapping(f"{attn}.o_proj.weight", [f"{attn}.o_proj.weight"], _identity)
        quantized.append(f"{attn}.o_proj.weight")
        if qk_norm:
            for name in (f"{attn}.q_norm.weight", f"{attn}.k_norm.weight"):
                mapping.add_mapping(name, [name], norm_func)
        mapping.add_unused(f"{attn}.rotary_emb.inv_freq")
        mapping.add_mapping(f"{mlp}.gate_up_proj.weight", [f"{mlp}.gate_proj.weight", f"{mlp}.up_proj.weight"],
                            _concat0)
        mapping.add_mapping(f"{mlp}.down_proj.weight", [f"{mlp}.down_proj.weight"], _identity)
        quantized += [f"{mlp}.gate_up_proj.weight", f"{mlp}.down_proj.weight"]
        for norm in layer_norms:
            name = f"model.layers.{i}.{norm}.weight"
            mapping.add_mapping(name, [name], norm_func)
    mapping.add_mapping("model.norm.weight", ["model.norm.weight"], norm_func)
    if always_tied or config.get("tie_word_embeddings", False):
        mapping.add_unused("lm_head.weight")
    else:
        mapping.add_mapping("lm_head.weight", ["lm_head.weight"], _identity)
        quantized.append("lm_head.weight")
    return mapping, quantized


def qwen2_huggingface(config: Dict[str, Any]) -> Tuple[ExternMapping, List[str]]:
    """``Qwen2ForCausalLM`` (python/mlc_llm/model/qwen2/qwen2_loader.py:10-15, qwen2_model.py:96-232): the fused
    projection is ``c_attn`` and carries a bias, which stays in the model dtype."""
    return _standard_decoder(config, qkv_target="c_attn", qkv_bias=True)


def qwen3_huggingface(config: Dict[str, Any]) -> Tuple[ExternMapping, List[str]]:
    """``Qwen3ForCausalLM`` (python/mlc_llm/model/qwen3/qwen3_loader.py:94-150, qwen3_model.py:119-130): ``c_attn``
    (a bias only with ``attention_bias``) and the per-head q / k RMSNorm weights."""
    return _standard_decoder(config, qkv_target="c_attn", qkv_bias=bool(config.get("attention_bias", False)),
                             qk_norm=True)


def gemma_huggingface(config: Dict[str, Any]) -> Tuple[ExternMapping, List[str]]:
    """``GemmaForCausalLM`` (python/mlc_llm/model/gemma/gemma_loader.py:15-48): RMSNorm weights are stored minus one
    in the checkpoint, the output projection is the embedding (gemma_model.py:228-260)."""
    return _standard_decoder(config, norm_plus_one=True, always_tied=True)


def gemma2_huggingface(config: Dict[str, Any]) -> Tuple[ExternMapping, List[str]]:
    """``Gemma2ForCausalLM`` (python/mlc_llm/model/gemma2/gemma2_loader.py): Gemma plus the two feed-forward norms."""
    return _standard_decoder(config, norm_plus_one=True, always_tied=True,
                             layer_norms=("input_layernorm", "post_attention_layernorm",
                                          "pre_feedforward_layernorm", "post_feedforward_layernorm"))


def phi3_huggingface(config: Dict[str, Any]) -> Tuple[ExternMapping, List[str]]:
    """``Phi3ForCausalLM`` (python/mlc_llm/model/phi3/phi3_loader.py:40-78): the checkpoint already holds fused
    ``qkv_proj`` / ``gate_up_proj``; only the names differ (``transformer.h.<i>.mixer`` ...)."""
    mapping, quantized = ExternMapping(), []
    if not config.get("tie_word_embeddings", False):
        mapping.add_mapping("lm_head.weight", ["lm_head.weight"], _identity)
        quantized.append("lm_head.weight")
    else:
        mapping.add_unused("lm_head.weight")
    mapping.add_mapping("transformer.norm.weight", ["model.norm.weight"], _identity)
    mapping.add_mapping("transformer.embd.weight", ["model.embed_tokens.weight"], _identity)
    quantized.append("transformer.embd.weight")
    for i in range(_cfg(config, "num_hidden_layers")):
        mlc, hf = f"transformer.h.{i}", f"model.layers.{i}"
        mapping.add_mapping(f"{mlc}.ln.weight", [f"{hf}.input_layernorm.weight"], _identity)
        for mlc_name, hf_name in ((f"{mlc}.mlp.down_proj.weight", f"{hf}.mlp.down_proj.weight"),
                                  (f"{mlc}.mlp.gate_up_proj.weight", f"{hf}.mlp.gate_up_proj.weight")):
            mapping.add_mapping(mlc_name, [hf_name], _identity)
            quantized.append(mlc_name)
        mapping.add_mapping(f"{mlc}.post_attention_layernorm.weight", [f"{hf}.post_attention_layernorm.weight"],
                            _identity)
        for mlc_name, hf_name in ((f"{mlc}.mixer.out_proj.weight", f"{hf}.self_attn.o_proj.weight"),
                                  (f"{mlc}.mixer.qkv_proj.weight", f"{hf}.self_attn.qkv_proj.weight")):
            mapping.add_mapping(mlc_name, [hf_name], _identity)
            quantized.append(mlc_name)
        mapping.add_unused(f"{hf}.self_attn.rotary_emb.inv_freq")
    return mapping, quantized


MODEL_MAPPINGS: Dict[str, Callable[[Dict[str, Any]], Tuple[ExternMapping, List[str]]]] = {
    "llama": llama_huggingface,
    "mistral": llama_huggingface,  # same module tree and HF names
    "mixtral": mixtral_huggingface,
    "qwen2": qwen2_huggingface,
    "qwen3": qwen3_huggingface,
    "gemma": gemma_huggingface,
    "gemma2": gemma2_huggingface,
    "phi3": phi3_huggingface,
}


def check_parameter_usage(mapping: ExternMapping, extern_names: Set[str]) -> Set[str]:
    """Every source name the mapping needs must exist (else ValueError); returns the source names
    that are neither used nor listed as unused, which the reference only warns about
    (python/mlc_llm/loader/utils.py:20-36)."""
    used: Set[str] = set()
    for names in mapping.param_map.values():
        used.update(names)
    leftover = extern_names - used - mapping.unused_params
    if leftover:
        import warnings

        warnings.warn("unused parameters in the weight files: " + ", ".join(sorted(leftover)))
    missing = used - extern_names
    if missing:
        raise ValueError("the following parameters do not exist in the weight files:\n  "
                         + "\n  ".join(sorted(missing)))
    return leftover


def param_kind(mlc_name: str) -> str:
    """Which module of GroupQuantize.quantize_model a quantised parameter belongs to, from its MLC name
    (python/mlc_llm/quantization/group_quantization.py:105-147): "embedding" (nn.Embedding), "final_fc" (a Linear
    that is_final_fc names: quantization/utils.py:51-54), "experts" (MixtralExperts) or "linear"."""
    base = mlc_name[: -len(".weight")] if mlc_name.endswith(".weight") else mlc_name
    leaf = base.rsplit(".", 1)[-1]
    if leaf in ("embed_tokens", "embd", "wte"):
        return "embedding"
    if base in ("head", "lm_head", "lm_head.linear", "embed_out"):
        return "final_fc"
    if leaf in ("e1_e3", "e2"):
        return "experts"
    return "linear"


class HuggingFaceLoader:
    """Yields (MLC name, tensor) for a safetensors checkpoint directory (or single file),
    quantising on ``device`` the parameters group quantisation replaces."""

    def __init__(self, path: str, mapping: ExternMapping, quantized: List[str],
                 quantization: Optional[GroupQuantize], model_dtype: torch.dtype = torch.float16):
        from safetensors import safe_open  # local import: only the converter needs it

        self._safe_open = safe_open
        self.mapping, self.quantization, self.model_dtype = mapping, quantization, model_dtype
        self.quantized = set(quantized) if quantization is not None else set()
        self.name_to_file: Dict[str, str] = {}
        if os.path.isdir(path):
            index = os.path.join(path, "model.safetensors.index.json")
            if os.path.isfile(index):
                with open(index, encoding="utf-8") as f:
                    for name, rel in json.load(f)["weight_map"].items():
                        self.name_to_file[name] = os.path.join(path, rel)
            else:
                files = sorted(f for f in os.listdir(path) if f.endswith(".safetensors"))
                if not files:
                    raise FileNotFoundError(f"no .safetensors file under {path}")
                for fn in files:
                    self._index_file(os.path.join(path, fn))
        elif path.endswith(".safetensors"):
            self._index_file(path)
        else:
            raise FileNotFoundError(f"unknown checkpoint: {path}")
        check_parameter_usage(mapping, set(self.name_to_file))
        self._open: Dict[str, Any] = {}
        self.total_param_num = 0

    def _index_file(self, file: str) -> None:
        with self._safe_open(file, framework="pt") as f:
            for name in f.keys():
                self.name_to_file[name] = file

    def _tensor(self, name: str) -> torch.Tensor:
        file = self.name_to_file[name]
        if file not in self._open:
            if len(self._open) >= 2:  # keep at most two shard files mapped, like the reference's cache
                old = next(iter(self._open))
                self._open.pop(old).__exit__(None, None, None)
            self._open[file] = self._safe_open(file, framework="pt").__enter__()
        return self._open[file].get_tensor(name)

    def close(self) -> None:
        for f in self._open.values():
            f.__exit__(None, None, None)
        self._open.clear()

    def load(self, device) -> Iterator[Tuple[str, torch.Tensor]]:
        # parameters that live in the same file are visited together (fewer re-opens), otherwise
        # in the mapping's order
        order = {n: i for i, n in enumerate(self.mapping.param_map)}
        names = sorted(self.mapping.param_map,
                       key=lambda n: (self.name_to_file[self.mapping.param_map[n][0]], order[n]))
        try:
            for mlc_name in names:
                parts = [self._tensor(n) for n in self.mapping.param_map[mlc_name]]
                # the map functions are written over numpy like the reference's; bf16 checkpoints
                # go through float32, which represents every bf16 value exactly
                np_parts = [(p.float() if p.dtype == torch.bfloat16 else p).numpy() for p in parts]
                value = torch.from_numpy(np.ascontiguousarray(self.mapping.map_func[mlc_name](*np_parts)))
                value = value.to(self.model_dtype)
                self.total_param_num += value.numel()
                q = self.quantization
                kind = param_kind(mlc_name)
                # what quantize_model leaves alone (group_quantization.py:117-139): the embedding under
                # quantize_embedding=False, the final fc under quantize_final_fc=False (q4f16_2)
                skip = mlc_name not in self.quantized or (kind == "embedding" and not q.quantize_embedding) or \
                    (kind == "final_fc" and not q.quantize_final_fc)
                if skip:
                    yield mlc_name, value.to(device)
                    continue
                if kind == "experts" and q.linear_weight_layout == "KN":
                    raise NotImplementedError("GroupQuantizeMixtralExperts does not support the KN layout "
                                              "(group_quantization.py:584-585)")
                base = mlc_name[: -len(".weight")]
                # KN schemes store a Linear's words and scales transposed (:125-130, 299-305); embeddings and
                # experts always quantise along their last axis and keep that layout
                transpose = q.linear_weight_layout == "KN" and kind in ("linear", "final_fc")
                qw, qs = q.quantize_weight(value.to(device), output_transpose=transpose)
                yield f"{base}.q_weight", qw
                yield f"{base}.q_scale", qs
        finally:
            self.close()


def convert_weight(source: str, output: str, quantization: str = "q4f16_1",
                   model_type: Optional[str] = None, device="cuda:0",
                   config: Optional[Dict[str, Any]] = None) -> Dict[str, Any]:
    """Checkpoint directory -> ``output/tensor-cache.json`` + shards (+ a minimal
    ``mlc-chat-config.json`` naming the scheme, the field the runtime reads it from:
    python/mlc_llm/protocol/mlc_chat_config.py:32).  Returns the metadata block."""
    if config is None:
        with open(os.path.join(source, "config.json"), encoding="utf-8") as f:
            config = json.load(f)
    model_type = model_type or config.get("model_type")
    if model_type not in MODEL_MAPPINGS:
        raise ValueError(f"no parameter mapping for model type {model_type!r}; known: {sorted(MODEL_MAPPINGS)}")
    quant = None
    if not quantization.startswith("q0"):
        quant = QUANTIZATION[quantization]
    elif quantization != "q0f16":
        raise ValueError("unquantised conversion is float16 only")
    mapping, quantized = MODEL_MAPPINGS[model_type](config)
    from .quantization import _TORCH_DTYPE

    # every tensor is cast to the scheme's model dtype, not to float16 (q4bf16_*, q4f32_1)
    loader = HuggingFaceLoader(source, mapping, quantized, quant,
                               _TORCH_DTYPE[quant.model_dtype] if quant is not None else torch.float16)
    total_bytes = 0
    count = 0

    def generate() -> Iterator[Tuple[str, Any]]:
        nonlocal total_bytes, count
        for name, t in loader.load(device):
            host = t.detach().cpu()
            total_bytes += host.numel() * host.element_size()
            count += 1
            # packed storage is uint32 in the file; torch carries the same bits as int32
            yield name, (host.numpy().view(np.uint32) if name.endswith(".q_weight") else host)

    def metadata() -> Dict[str, Any]:
        return {"ParamSize": count, "ParamBytes": float(total_bytes),
                "BitsPerParam": total_bytes * 8.0 / max(loader.total_param_num, 1)}

    doc = dump_tensor_cache(generate(), output, encode_format="f32-to-bf16", meta_data=metadata)
    with open(os.path.join(output, "mlc-chat-config.json"), "w", encoding="utf-8") as f:
        json.dump({"model_type": model_type, "quantization": quantization, "model_config": config}, f, indent=2)
    return doc["metadata"]
