"""CPU-only checks of the host side: the C-ABI library loads and exports what the header
declares, argument validation fails cleanly (no kernel is launched), and the mirrored
configuration / module-rewriting logic behaves like the reference's
(tests/python/quantization/test_group_quantization.py:149-182,
tests/python/model/test_llama_quantization.py:11-50)."""

import ctypes
import os

import pytest
import torch
from torch import nn

import mlc_llm_amd as gq
from mlc_llm_amd import _lib
from mlc_llm_amd.quantization import is_final_fc, is_moe_gate


def test_library_exports_every_declared_symbol():
    declared = _lib.declared_symbols()
    assert declared == sorted(_lib.SIGNATURES), "header and ctypes signature table disagree"
    assert len(declared) >= 19
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), f"{name} is declared in include/mi355gq.h but not exported"
    assert _lib.lib().mi355gq_version() == 100


def test_only_c_abi_symbols_are_exported():
    import subprocess

    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True).stdout
    funcs = [l.split()[-1] for l in out.splitlines() if " T " in l]
    assert funcs and all(f.startswith("mi355gq_") for f in funcs), funcs


def _err():
    return _lib.lib().mi355gq_last_error().decode()


def test_argument_validation_never_launches():
    lib = _lib.lib()
    # scheme errors come before anything touches the device
    assert lib.mi355gq_linear(None, None, None, None, 1, 8, 32, 5, 32, 0, None, None, 0, None) == -3
    assert "bits=5" in _err()
    assert lib.mi355gq_linear(None, None, None, None, 1, 8, 32, 4, 30, 0, None, None, 0, None) == -1
    assert lib.mi355gq_linear(None, None, None, None, 1, 8, 128, 4, 128, 0, None, None, 0, None) == -3
    assert "4 storage words" in _err()
    # null pointers, negative sizes, bad enums
    assert lib.mi355gq_linear(None, None, None, None, 1, 8, 32, 4, 32, 0, None, None, 0, None) == -1
    assert "null" in _err()
    assert lib.mi355gq_linear(None, None, None, None, -1, 8, 32, 4, 32, 0, None, None, 0, None) == -1
    assert lib.mi355gq_linear(None, None, None, None, 1, 8, 32, 4, 32, 7, None, None, 0, None) == -1
    assert lib.mi355gq_quantize(None, 4, 32, 4, 32, 9, None, None, None) == -1
    assert lib.mi355gq_quantize(None, 4, 32, 4, 32, 0, None, None, None) == -1
    assert lib.mi355gq_moe_gemv(None, 3, None, None, None, 2, 8, 16, 32, 4, 32, None, None) == -1
    assert "expected 1 or top_k" in _err()
    assert lib.mi355gq_gating_softmax_topk(None, 4, 8, 9, None, None, None) == -1
    assert lib.mi355gq_moe_cumsum(None, 4, 2, 300, None, None) == -1
    assert lib.mi355gq_testing_set_option(b"no_such_option", 1) == -1
    # misaligned pointers are rejected, not dereferenced
    assert lib.mi355gq_dequantize(ctypes.c_void_p(0x1004), ctypes.c_void_p(0x2000), 1, 32, 4, 32,
                                  ctypes.c_void_p(0x3000), None) == -1
    assert "aligned" in _err()
    # empty problems are a no-op success
    assert lib.mi355gq_linear(None, None, None, None, 0, 8, 32, 4, 32, 0, None, None, 0, None) == 0
    assert lib.mi355gq_quantize(None, 0, 32, 4, 32, 0, None, None, None) == 0
    assert lib.mi355gq_embedding_take(None, 0, None, None, 10, 32, 4, 32, None, None) == 0
    with pytest.raises(_lib.Mi355gqError) as ei:
        _lib.call("mi355gq_testing_set_option", b"bogus", 0)
    assert ei.value.code == -1 and "bogus" in str(ei.value)


def test_argument_validation_of_the_later_entry_points():
    lib = _lib.lib()
    P = ctypes.c_void_p
    # folded activation: odd N is an argument error; empty problems succeed
    assert lib.mi355gq_linear_silu_mul(P(0x1000), P(0x2000), P(0x3000), 2, 63, 64, 4, 32, P(0x4000), None, 0, None) == -1
    assert "even" in _err()
    assert lib.mi355gq_linear_silu_mul(None, None, None, 0, 64, 64, 4, 32, None, None, 0, None) == 0
    assert lib.mi355gq_linear_silu_mul_workspace_bytes(4, 28672, 4096, 4, 32) == 0
    assert lib.mi355gq_moe_gemv_silu_mul(P(0x1000), 1, P(0x2000), P(0x3000), P(0x4000), 2, 8, 15, 64, 4, 32, P(0x5000), None) == -1
    # routing: limits of the single-workgroup form are a missing kernel, bad sizes an argument error
    assert lib.mi355gq_moe_route(P(0x1000), 9000, 8, 2, P(0x2000), P(0x3000), P(0x4000), P(0x5000), P(0x6000),
                                 P(0x7000), 0, None) == -3
    assert "four" in _err() or "gating_softmax_topk" in _err()
    assert lib.mi355gq_moe_route(P(0x1000), 5000, 128, 2, P(0x2000), P(0x3000), P(0x4000), P(0x5000), P(0x6000),
                                 P(0x7000), 0, None) == -3
    assert lib.mi355gq_moe_route(P(0x1000), 16, 8, 9, P(0x2000), P(0x3000), P(0x4000), P(0x5000), P(0x6000),
                                 P(0x7000), 0, None) == -1
    assert lib.mi355gq_moe_route(P(0x1000), 16, 8, 2, P(0x2000), P(0x3000), P(0x4000), P(0x5000), P(0x6000),
                                 None, 0, None) == -1
    assert lib.mi355gq_moe_experts(P(0x1000), 4, None, 5, P(0x2000), P(0x3000), P(0x4000), 0, 8, 16, 64, 4, 32, 0,
                                   P(0x5000), None) == -1  # x rows must equal rows without an index
    assert lib.mi355gq_moe_experts(P(0x1000), 4, None, 4, P(0x2000), P(0x3000), P(0x4000), 0, 8, 16, 64, 4, 32, 7,
                                   P(0x5000), None) == -1  # unknown epilogue
    assert lib.mi355gq_moe_combine_sorted(P(0x1000), None, P(0x2000), 4, 2, 64, P(0x3000), None) == -1
    # model dtypes: unknown code, out dtype that is neither the model's nor float32, K = 0
    assert lib.mi355gq_quantize_dt(P(0x1000), 4, 32, 4, 32, 0, 5, P(0x2000), P(0x3000), None) == -1
    assert "model_dtype" in _err()
    assert lib.mi355gq_dequantize_dt(P(0x1000), P(0x2000), 4, 32, 4, 32, 3, P(0x3000), None) == -1
    assert lib.mi355gq_linear_dt(P(0x1000), P(0x2000), P(0x3000), None, 2, 8, 64, 4, 32, 2, 0, P(0x4000), None, 0, None) == -1
    assert "out_dtype" in _err()
    assert lib.mi355gq_linear_dt(P(0x1000), P(0x2000), P(0x3000), None, 2, 8, 0, 4, 32, 1, 1, P(0x4000), None, 0, None) == -1
    assert lib.mi355gq_linear_dt(P(0x1002), P(0x2000), P(0x3000), None, 2, 8, 64, 4, 32, 1, 1, P(0x4000), None, 0, None) == -1
    # the expert matmuls in the other model dtypes
    assert lib.mi355gq_moe_gemv_dt(P(0x1000), 3, P(0x2000), P(0x3000), P(0x4000), 2, 8, 16, 32, 4, 32, 1, P(0x5000), None) == -1
    assert "expected 1 or top_k" in _err()
    assert lib.mi355gq_moe_gemv_dt(P(0x1000), 1, P(0x2000), P(0x3000), P(0x4000), 2, 8, 16, 32, 4, 32, 7, P(0x5000), None) == -1
    assert "model_dtype" in _err()
    assert lib.mi355gq_moe_gemv_dt(P(0x1000), 1, P(0x2000), P(0x3000), P(0x4000), 2, 8, 16, 0, 4, 32, 2, P(0x5000), None) == -1
    assert lib.mi355gq_moe_gemv_dt(P(0x1001), 1, P(0x2000), P(0x3000), P(0x4000), 2, 8, 16, 32, 4, 32, 2, P(0x5000), None) == -1
    assert "aligned" in _err()
    assert lib.mi355gq_moe_group_gemm_dt(P(0x1000), 4, P(0x2000), P(0x3000), P(0x4000), 9, 8, 16, 32, 4, 32, 1, P(0x5000), None) == -1
    assert "indptr_dtype" in _err()
    assert lib.mi355gq_moe_group_gemm_dt(P(0x1000), 4, P(0x2000), P(0x3000), None, 0, 8, 16, 32, 4, 32, 1, P(0x5000), None) == -1
    assert "null" in _err()
    assert lib.mi355gq_moe_group_gemm_dt(None, 0, None, None, None, 0, 8, 16, 32, 4, 32, 2, None, None) == 0
    assert lib.mi355gq_moe_gemv_dt(None, 1, None, None, None, 0, 8, 16, 32, 4, 32, 1, None, None) == 0
    # folded activation in the other model dtypes: float32 has no fused kernel, odd N is an error
    assert lib.mi355gq_linear_silu_mul_dt(P(0x1000), P(0x2000), P(0x3000), 2, 8, 64, 4, 32, 1, P(0x4000), None, 0,
                                          None) == _lib.ERR_UNSUPPORTED
    assert lib.mi355gq_linear_silu_mul_dt(P(0x1000), P(0x2000), P(0x3000), 2, 7, 64, 4, 32, 2, P(0x4000), None, 0,
                                          None) == -1
    assert lib.mi355gq_moe_gemv_silu_mul_dt(P(0x1000), 1, P(0x2000), P(0x3000), P(0x4000), 2, 8, 16, 32, 4, 32, 1,
                                            P(0x5000), None) == _lib.ERR_UNSUPPORTED
    assert lib.mi355gq_linear_silu_mul_dt_workspace_bytes(40, 100, 4096, 4, 32, 2) == 0  # N % 64 != 0
    assert lib.mi355gq_linear_silu_mul_dt_workspace_bytes(40, 128, 4096, 4, 32, 2) > 0
    # routing glue in the other model dtypes
    assert lib.mi355gq_gating_softmax_topk_dt(P(0x1000), 4, 8, 9, P(0x2000), P(0x3000), 2, None) == -1
    assert "top_k" in _err()
    assert lib.mi355gq_gating_softmax_topk_dt(P(0x1000), 4, 8, 2, P(0x2000), P(0x3000), 9, None) == -1
    assert "model_dtype" in _err()
    assert lib.mi355gq_silu_mul_dt(None, 4, 8, None, 1, None) == -1
    assert lib.mi355gq_silu_mul_dt(None, 0, 8, None, 2, None) == 0
    assert lib.mi355gq_take_rows_dt(P(0x1002), P(0x2000), 4, 8, 4, P(0x3000), 1, None) == -1
    assert "misaligned" in _err()
    assert lib.mi355gq_moe_scatter_output_dt(None, None, 0, 8, None, 2, None) == 0
    assert lib.mi355gq_moe_combine_dt(None, None, None, 4, 0, 8, None, 1, None) == -1
    assert lib.mi355gq_moe_route_dt(P(0x1000), 9000, 8, 2, P(0x2000), P(0x3000), P(0x4000), P(0x5000), P(0x6000),
                                    P(0x7000), 0, 2, None) == _lib.ERR_UNSUPPORTED
    assert lib.mi355gq_quantize_dt(None, 0, 32, 4, 32, 0, 2, None, None, None) == 0
    assert lib.mi355gq_embedding_take_dt(None, 0, None, None, 10, 32, 4, 32, 1, None, None) == 0


def test_ops_refuse_cpu_tensors():
    x = torch.zeros(1, 32, dtype=torch.float16)
    qw = torch.zeros(8, 4, dtype=torch.int32)
    qs = torch.zeros(8, 1, dtype=torch.float16)
    with pytest.raises(ValueError, match="GPU"):
        gq.ops.linear(x, qw, qs, 4, 32)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_LIB", None)
    monkeypatch.setattr(_lib, "LIB_PATH", os.path.join(os.path.dirname(_lib.LIB_PATH), "nope.so"))
    with pytest.raises(RuntimeError, match="no non-HIP fallback"):
        _lib.lib()


def test_registry_and_derived_fields():
    q4, q3 = gq.QUANTIZATION["q4f16_1"], gq.QUANTIZATION["q3f16_1"]
    assert (q4.group_size, q4.num_elem_per_storage, q4.num_storage_per_group, q4.max_int_value) == (32, 8, 4, 7)
    assert (q3.group_size, q3.num_elem_per_storage, q3.num_storage_per_group, q3.max_int_value) == (40, 10, 4, 3)
    assert q4.linear_quant_axis == 1 and gq.QUANTIZATION["q4f16_0"].linear_quant_axis == 0
    with pytest.raises(ValueError, match="divisible"):
        gq.GroupQuantize("bad", "group-quant", 36, "int3", "uint32", "float16", "NK")
    # the KN entries describe the same tensors transposed: [nw, N] words, [ng, N] scales
    kn = gq.GroupQuantizeLinear(64, 24, gq.QUANTIZATION["q4f16_0"], bias=False)
    assert tuple(kn.q_weight.shape) == (8, 24) and tuple(kn.q_scale.shape) == (2, 24)
    kn3 = gq.GroupQuantizeLinear(80, 24, gq.QUANTIZATION["q3f16_0"], bias=False)
    assert tuple(kn3.q_weight.shape) == (8, 24) and tuple(kn3.q_scale.shape) == (2, 24)


def test_name_predicates():
    assert is_final_fc("lm_head") and not is_final_fc("model.lm_head")
    gate = nn.Linear(16, 8, bias=False)
    assert is_moe_gate("model.layers.0.moe.gate", gate)
    assert not is_moe_gate("model.layers.0.mlp.gate_up_proj", gate)
    assert not is_moe_gate("x.gate", nn.Linear(16, 512, bias=False))


@pytest.mark.parametrize("quant_name", ["q3f16_1", "q4f16_1"])
def test_quantize_model(quant_name):
    # same structure as the reference's test_quantize_model (shape [16, 128])
    class Test(nn.Module):
        def __init__(self):
            super().__init__()
            self.linear = nn.Linear(16, 128, dtype=torch.float16)
            self.embedding = nn.Embedding(16, 128, dtype=torch.float16)

    config = gq.QUANTIZATION[quant_name]
    quant_map = gq.QuantizeMapping({}, {})
    mod = config.quantize_model(Test(), quant_map, "model")
    assert quant_map.param_map["model.linear.weight"] == ["model.linear.q_weight", "model.linear.q_scale"]
    assert quant_map.map_func["model.linear.weight"].func == config.quantize_weight
    assert isinstance(mod.linear, gq.GroupQuantizeLinear)
    assert quant_map.param_map["model.embedding.weight"] == ["model.embedding.q_weight", "model.embedding.q_scale"]
    assert quant_map.map_func["model.embedding.weight"] == config.quantize_weight
    assert isinstance(mod.embedding, gq.GroupQuantizeEmbedding)
    ng = -(-16 // config.group_size)
    assert tuple(mod.linear.q_weight.shape) == (128, 4 * ng) and tuple(mod.linear.q_scale.shape) == (128, ng)
    assert mod.linear.bias is not None and tuple(mod.linear.bias.shape) == (128,)
    ngd = -(-128 // config.group_size)
    assert tuple(mod.embedding.q_weight.shape) == (16, 4 * ngd)


def test_quantize_model_llama_like_structure():
    # every projection and lm_head become GroupQuantizeLinear, embed_tokens GroupQuantizeEmbedding,
    # MoE router gates and no_quantization modules are left alone, experts are replaced
    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.qkv_proj = nn.Linear(64, 96, bias=False)
            self.o_proj = nn.Linear(64, 64, bias=False)
            self.gate = nn.Linear(64, 8, bias=False)
            self.e1_e3 = gq.MixtralExperts(8, 64, 256)
            self.norm = nn.LayerNorm(64)
            self.keep = nn.Linear(64, 64)
            self.keep.no_quantization = True

    class Model(nn.Module):
        def __init__(self):
            super().__init__()
            self.embed_tokens = nn.Embedding(100, 64)
            self.layers = nn.ModuleList([Block(), Block()])

    class LM(nn.Module):
        def __init__(self):
            super().__init__()
            self.model = Model()
            self.lm_head = nn.Linear(64, 100, bias=False)

    config = gq.QUANTIZATION["q4f16_1"]
    qm = gq.QuantizeMapping({}, {})
    lm = config.quantize_model(LM(), qm, "")
    for layer in lm.model.layers:
        assert isinstance(layer.qkv_proj, gq.GroupQuantizeLinear) and layer.qkv_proj.bias is None
        assert isinstance(layer.o_proj, gq.GroupQuantizeLinear)
        assert isinstance(layer.gate, nn.Linear) and isinstance(layer.keep, nn.Linear)
        assert isinstance(layer.e1_e3, gq.GroupQuantizeMixtralExperts)
        assert tuple(layer.e1_e3.q_weight.shape) == (8, 256, 8) and tuple(layer.e1_e3.q_scale.shape) == (8, 256, 2)
    assert isinstance(lm.model.embed_tokens, gq.GroupQuantizeEmbedding)
    assert isinstance(lm.lm_head, gq.GroupQuantizeLinear)
    assert "lm_head.weight" in qm.param_map and "model.layers.1.e1_e3.weight" in qm.param_map
    assert "model.layers.0.gate.weight" not in qm.param_map
    no_fc = gq.GroupQuantize("q4_nofc", "group-quant", 32, "int4", "uint32", "float16", "NK",
                             quantize_final_fc=False)
    lm2 = no_fc.quantize_model(LM(), gq.QuantizeMapping({}, {}), "")
    assert isinstance(lm2.lm_head, nn.Linear)


def test_tensor_parallel_group_check():
    cfg = gq.GroupQuantize("q4tp", "group-quant", 32, "int4", "uint32", "float16", "NK",
                           tensor_parallel_shards=2)
    with pytest.raises(ValueError, match="cannot be evenly distributed"):
        gq.GroupQuantizeLinear(48, 8, cfg)  # 96 input features = 3 groups over 2 shards
    gq.GroupQuantizeLinear(64, 8, cfg)  # 4 groups over 2 shards


def test_registry_holds_every_group_quant_entry_of_the_reference():
    # quantization/quantization.py:47-134 of the reference
    want = {"q3f16_0": (40, "int3", "KN", "float16", True), "q3f16_1": (40, "int3", "NK", "float16", True),
            "q4f16_0": (32, "int4", "KN", "float16", True), "q4f16_1": (32, "int4", "NK", "float16", True),
            "q4bf16_0": (32, "int4", "KN", "bfloat16", True), "q4bf16_1": (32, "int4", "NK", "bfloat16", True),
            "q4f32_1": (32, "int4", "NK", "float32", True), "q4f16_2": (32, "int4", "NK", "float16", False)}
    assert set(gq.QUANTIZATION) == set(want)
    for name, (g, qd, layout, md, emb) in want.items():
        c = gq.QUANTIZATION[name]
        assert (c.group_size, c.quantize_dtype, c.linear_weight_layout, c.model_dtype) == (g, qd, layout, md)
        assert c.quantize_embedding == emb and c.quantize_final_fc == emb


def test_q4f16_2_leaves_embedding_and_final_fc_alone():
    import torch
    from torch import nn

    class Tiny(nn.Module):
        def __init__(self):
            super().__init__()
            self.embed_tokens = nn.Embedding(16, 64)
            self.proj = nn.Linear(64, 64, bias=False)
            self.lm_head = nn.Linear(64, 16, bias=False)

    qmap = gq.QuantizeMapping({}, {})
    m = gq.QUANTIZATION["q4f16_2"].quantize_model(Tiny(), qmap, "")
    assert isinstance(m.embed_tokens, nn.Embedding) and isinstance(m.lm_head, nn.Linear)
    assert isinstance(m.proj, gq.GroupQuantizeLinear)
    assert set(qmap.param_map) == {"proj.weight"}


def test_other_model_dtypes_carry_their_dtype_in_the_parameters():
    import torch
    for name, dt in (("q4bf16_1", torch.bfloat16), ("q4f32_1", torch.float32)):
        lin = gq.GroupQuantizeLinear(64, 24, gq.QUANTIZATION[name], bias=True)
        assert lin.q_scale.dtype == dt and lin.bias.dtype == dt and lin.q_weight.shape == (24, 8)
        emb = gq.GroupQuantizeEmbedding(10, 64, gq.QUANTIZATION[name])
        assert emb.q_scale.dtype == dt
