"""Weight directory format and HuggingFace -> MLC parameter mapping.

No weight directory and no checkpoint ship with the reference, so these tests build tiny synthetic
checkpoints with the HuggingFace parameter names and check (a) the file format by round trip and
against its published field list, (b) the mapping against what the reference's loaders do
(python/mlc_llm/loader/standard_loader.py:89-134, python/mlc_llm/model/mixtral/mixtral_loader.py:44-104),
(c) on the GPU, that the converted ``q_weight`` / ``q_scale`` equal the oracle's quantisation of the
concatenated / stacked matrices bit for bit."""

import json
import os
import zlib

import numpy as np
import pytest
import torch

from mlc_llm_amd import loader, tensor_cache
from oracle import gq_oracle as o

LLAMA = {"model_type": "llama", "hidden_size": 64, "intermediate_size": 160, "num_hidden_layers": 2,
         "num_attention_heads": 4, "num_key_value_heads": 2, "vocab_size": 96, "tie_word_embeddings": False}
QWEN2 = dict(LLAMA, model_type="qwen2", tie_word_embeddings=True)
MIXTRAL = {"model_type": "mixtral", "hidden_size": 64, "intermediate_size": 96, "num_hidden_layers": 1,
           "num_attention_heads": 4, "num_key_value_heads": 2, "vocab_size": 80, "num_local_experts": 3,
           "num_experts_per_tok": 2}


def _hf_tensors(cfg, seed=0):
    rng = np.random.default_rng(seed)
    h, inter, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    kv = h // cfg["num_attention_heads"] * cfg["num_key_value_heads"]

    def w(*shape):
        return torch.from_numpy((rng.standard_normal(shape) * 0.05).astype(np.float16))

    t = {"model.embed_tokens.weight": w(v, h), "model.norm.weight": w(h), "lm_head.weight": w(v, h)}
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        t[f"{p}.self_attn.q_proj.weight"] = w(h, h)
        t[f"{p}.self_attn.k_proj.weight"] = w(kv, h)
        t[f"{p}.self_attn.v_proj.weight"] = w(kv, h)
        t[f"{p}.self_attn.o_proj.weight"] = w(h, h)
        t[f"{p}.input_layernorm.weight"] = w(h)
        t[f"{p}.post_attention_layernorm.weight"] = w(h)
        t[f"{p}.self_attn.rotary_emb.inv_freq"] = w(8)
        if cfg["model_type"] == "qwen2":
            t[f"{p}.self_attn.q_proj.bias"], t[f"{p}.self_attn.k_proj.bias"] = w(h), w(kv)
            t[f"{p}.self_attn.v_proj.bias"] = w(kv)
        if cfg["model_type"] == "mixtral":
            t[f"{p}.block_sparse_moe.gate.weight"] = w(cfg["num_local_experts"], h)
            for e in range(cfg["num_local_experts"]):
                t[f"{p}.block_sparse_moe.experts.{e}.w1.weight"] = w(inter, h)
                t[f"{p}.block_sparse_moe.experts.{e}.w2.weight"] = w(h, inter)
                t[f"{p}.block_sparse_moe.experts.{e}.w3.weight"] = w(inter, h)
        else:
            t[f"{p}.mlp.gate_proj.weight"] = w(inter, h)
            t[f"{p}.mlp.up_proj.weight"] = w(inter, h)
            t[f"{p}.mlp.down_proj.weight"] = w(h, inter)
    return t


def _write_checkpoint(path, cfg, tensors, shards=2):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    names = list(tensors)
    weight_map = {}
    for s in range(shards):
        part = {n: tensors[n] for n in names[s::shards]}
        fn = f"model-{s + 1:05d}-of-{shards:05d}.safetensors"
        save_file(part, os.path.join(path, fn))
        weight_map.update({n: fn for n in part})
    with open(os.path.join(path, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": weight_map}, f)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)


# ------------------------------------------------------------------------------ file format

def test_bf16_encoding_known_values():
    # 1.0 -> 0x3F80; ties go to even: 0x3F808000 -> 0x3F80, 0x3F818000 -> 0x3F82; above half rounds up
    bits = np.array([0x3F800000, 0x3F808000, 0x3F818000, 0x3F808001, 0xBF808001, 0x00000000], np.uint32)
    enc = tensor_cache.f32_to_bf16(bits.view(np.float32))
    assert enc.tolist() == [0x3F80, 0x3F80, 0x3F82, 0x3F81, 0xBF81, 0x0000]
    # the largest float32 must clip to the largest bf16, not round up to infinity
    big = np.array([np.finfo(np.float32).max, -np.finfo(np.float32).max], np.float32)
    assert tensor_cache.f32_to_bf16(big).tolist() == [0x7F7F, 0xFF7F]
    # decode is the exact left shift
    assert tensor_cache.bf16_to_f32(np.array([0x3F80, 0xC000], np.uint16)).tolist() == [1.0, -2.0]
    # every bf16-representable float survives a round trip
    rep = (np.arange(0, 0x7F80, 7, dtype=np.uint32) << 16).view(np.float32)
    assert np.array_equal(tensor_cache.bf16_to_f32(tensor_cache.f32_to_bf16(rep)), rep)


def test_tensor_cache_round_trip_and_schema(tmp_path):
    rng = np.random.default_rng(3)
    params = {
        "a.q_weight": rng.integers(0, 2**32, (40, 16), dtype=np.uint32),
        "a.q_scale": rng.standard_normal((40, 4)).astype(np.float16),
        "norm.weight": torch.from_numpy(rng.standard_normal(64).astype(np.float16)),
        "f32": (np.arange(24, dtype=np.float32) * 0.5).reshape(2, 3, 4),  # exactly representable in bf16
        "big": rng.integers(0, 2**32, (300, 1024), dtype=np.uint32),      # 1.2 MB > 1 MiB cap: own shard
        "tail": rng.standard_normal(10).astype(np.float16),
        "empty": np.zeros((0, 8), np.float16),
    }
    doc = tensor_cache.dump_tensor_cache(params, str(tmp_path), meta_data=lambda: {"ParamSize": len(params)},
                                         shard_cap_mb=1)
    on_disk = json.load(open(tmp_path / "tensor-cache.json"))
    assert on_disk == doc and on_disk["metadata"] == {"ParamSize": 7}
    shards = on_disk["records"]
    assert [s["dataPath"] for s in shards] == [f"params_shard_{i}.bin" for i in range(len(shards))]
    for s in shards:
        assert set(s) == {"dataPath", "format", "nbytes", "records", "md5sum"} and s["format"] == "raw-shard"
        assert os.path.getsize(tmp_path / s["dataPath"]) == s["nbytes"] <= max(1 << 20, s["records"][0]["nbytes"])
        end = 0
        for r in s["records"]:
            assert set(r) == {"name", "shape", "dtype", "format", "nbytes", "byteOffset"}
            assert r["byteOffset"] == end  # packed back to back
            end += r["nbytes"]
        assert end == s["nbytes"]
    big = [s for s in shards if s["records"][0]["name"] == "big"][0]
    assert len(big["records"]) == 1
    recs = {r["name"]: r for s in shards for r in s["records"]}
    # a tensor with a shard of its own is written at once, the rest keeps iteration order
    assert [n for n in recs if n != "big"] == [n for n in params if n != "big"] and "big" in recs
    assert recs["f32"]["format"] == "f32-to-bf16" and recs["f32"]["nbytes"] == 48 and recs["f32"]["dtype"] == "float32"
    assert recs["a.q_weight"]["dtype"] == "uint32" and recs["a.q_weight"]["format"] == "raw"

    loaded, meta = tensor_cache.load_tensor_cache(str(tmp_path), verify_md5=True)
    assert meta == {"ParamSize": 7} and set(loaded) == set(params)
    assert loaded["a.q_weight"].dtype == torch.int32
    assert np.array_equal(loaded["a.q_weight"].numpy().view(np.uint32), params["a.q_weight"])
    assert np.array_equal(loaded["big"].numpy().view(np.uint32), params["big"])
    assert torch.equal(loaded["norm.weight"], params["norm.weight"])
    assert np.array_equal(loaded["f32"].numpy(), params["f32"]) and loaded["f32"].dtype == torch.float32
    assert tuple(loaded["empty"].shape) == (0, 8)
    only = dict(tensor_cache.iter_tensor_cache(str(tmp_path), names=["tail"]))
    assert list(only) == ["tail"] and np.array_equal(only["tail"].numpy(), params["tail"])


def test_tensor_cache_detects_corruption(tmp_path):
    tensor_cache.dump_tensor_cache({"x": np.arange(64, dtype=np.int32)}, str(tmp_path))
    shard = tmp_path / "params_shard_0.bin"
    data = bytearray(shard.read_bytes())
    data[5] ^= 0xFF
    shard.write_bytes(bytes(data))
    with pytest.raises(ValueError, match="md5"):
        tensor_cache.load_tensor_cache(str(tmp_path), verify_md5=True)
    shard.write_bytes(bytes(data[:-4]))
    with pytest.raises(ValueError, match="bytes on disk"):
        tensor_cache.load_tensor_cache(str(tmp_path))
    with pytest.raises(ValueError, match="duplicate"):
        tensor_cache.dump_tensor_cache([("x", np.zeros(1, np.int32)), ("x", np.zeros(1, np.int32))], str(tmp_path))


# ------------------------------------------------------------------------------ mapping

def test_llama_mapping_names_and_concatenation():
    mapping, quantized = loader.llama_huggingface(LLAMA)
    t = {k: v.numpy() for k, v in _hf_tensors(LLAMA).items()}
    assert list(mapping.param_map)[:3] == ["model.embed_tokens.weight", "model.layers.0.self_attn.qkv_proj.weight",
                                          "model.layers.0.self_attn.o_proj.weight"]
    qkv = mapping.map_func["model.layers.1.self_attn.qkv_proj.weight"](
        *[t[n] for n in mapping.param_map["model.layers.1.self_attn.qkv_proj.weight"]])
    assert qkv.shape == (64 + 32 + 32, 64)
    assert np.array_equal(qkv[:64], t["model.layers.1.self_attn.q_proj.weight"])
    assert np.array_equal(qkv[64:96], t["model.layers.1.self_attn.k_proj.weight"])
    assert np.array_equal(qkv[96:], t["model.layers.1.self_attn.v_proj.weight"])
    gu = mapping.map_func["model.layers.0.mlp.gate_up_proj.weight"](
        *[t[n] for n in mapping.param_map["model.layers.0.mlp.gate_up_proj.weight"]])
    assert np.array_equal(gu[:160], t["model.layers.0.mlp.gate_proj.weight"])
    assert np.array_equal(gu[160:], t["model.layers.0.mlp.up_proj.weight"])
    # norms are never quantised; embedding, every projection and the final fc are
    assert not any("norm" in q for q in quantized)
    assert {"model.embed_tokens.weight", "lm_head.weight", "model.layers.0.mlp.down_proj.weight"} <= set(quantized)
    assert len(quantized) == 2 + 4 * LLAMA["num_hidden_layers"]
    assert loader.check_parameter_usage(mapping, set(t)) == set()  # inv_freq is declared unused
    tied = dict(LLAMA, tie_word_embeddings=True)
    m2, q2 = loader.llama_huggingface(tied)
    assert "lm_head.weight" not in m2.param_map and "lm_head.weight" not in q2
    with pytest.raises(ValueError, match="do not exist"):
        loader.check_parameter_usage(mapping, set(t) - {"model.layers.0.mlp.up_proj.weight"})


def test_mixtral_mapping_stacks_experts():
    mapping, quantized = loader.mixtral_huggingface(MIXTRAL)
    t = {k: v.numpy() for k, v in _hf_tensors(MIXTRAL).items()}
    e13 = mapping.map_func["model.layers.0.moe.e1_e3.weight"](
        *[t[n] for n in mapping.param_map["model.layers.0.moe.e1_e3.weight"]])
    e2 = mapping.map_func["model.layers.0.moe.e2.weight"](
        *[t[n] for n in mapping.param_map["model.layers.0.moe.e2.weight"]])
    assert e13.shape == (3, 192, 64) and e2.shape == (3, 64, 96)
    for e in range(3):
        assert np.array_equal(e13[e, :96], t[f"model.layers.0.block_sparse_moe.experts.{e}.w1.weight"])
        assert np.array_equal(e13[e, 96:], t[f"model.layers.0.block_sparse_moe.experts.{e}.w3.weight"])
        assert np.array_equal(e2[e], t[f"model.layers.0.block_sparse_moe.experts.{e}.w2.weight"])
    assert mapping.param_map["model.layers.0.moe.gate.weight"] == ["model.layers.0.block_sparse_moe.gate.weight"]
    assert "model.layers.0.moe.gate.weight" not in quantized  # the router stays in floating point
    assert {"model.layers.0.moe.e1_e3.weight", "model.layers.0.moe.e2.weight"} <= set(quantized)


def test_other_family_mappings():
    """Qwen2 / Qwen3 (c_attn, bias, q / k norms), Gemma / Gemma2 (norm + 1, tied output projection) and Phi-3
    (already fused in the checkpoint, renamed): names, transforms and which parameters are quantised."""
    base = dict(LLAMA)
    t = {k: v.numpy() for k, v in _hf_tensors(LLAMA).items()}
    rng = np.random.default_rng(3)
    for i in range(LLAMA["num_hidden_layers"]):
        attn = f"model.layers.{i}.self_attn"
        for n, rows in (("q_proj", 64), ("k_proj", 32), ("v_proj", 32)):
            t[f"{attn}.{n}.bias"] = rng.standard_normal(rows).astype(np.float16)
        t[f"{attn}.q_norm.weight"] = rng.standard_normal(16).astype(np.float16)
        t[f"{attn}.k_norm.weight"] = rng.standard_normal(16).astype(np.float16)
        for n in ("pre_feedforward_layernorm", "post_feedforward_layernorm"):
            t[f"model.layers.{i}.{n}.weight"] = rng.standard_normal(64).astype(np.float16)

    def build(mapping, name):
        return mapping.map_func[name](*[t[n] for n in mapping.param_map[name]])

    # Qwen2: fused projection named c_attn, with a concatenated bias that is not quantised
    m, q = loader.MODEL_MAPPINGS["qwen2"](dict(base, model_type="qwen2"))
    w = build(m, "model.layers.1.self_attn.c_attn.weight")
    b = build(m, "model.layers.1.self_attn.c_attn.bias")
    assert w.shape == (128, 64) and b.shape == (128,)
    assert np.array_equal(b[64:96], t["model.layers.1.self_attn.k_proj.bias"])
    assert "model.layers.1.self_attn.c_attn.weight" in q and "model.layers.1.self_attn.c_attn.bias" not in q
    assert "model.layers.0.self_attn.qkv_proj.weight" not in m.param_map
    unused = loader.check_parameter_usage(m, set(t))
    assert all("q_norm" in n or "k_norm" in n or "feedforward" in n for n in unused)
    # Qwen3: the per-head norms pass through unquantised; a bias only when the config says so
    m, q = loader.MODEL_MAPPINGS["qwen3"](dict(base, model_type="qwen3"))
    assert np.array_equal(build(m, "model.layers.0.self_attn.q_norm.weight"), t["model.layers.0.self_attn.q_norm.weight"])
    assert "model.layers.0.self_attn.c_attn.bias" not in m.param_map and not any("norm" in n for n in q)
    m, _ = loader.MODEL_MAPPINGS["qwen3"](dict(base, model_type="qwen3", attention_bias=True))
    assert "model.layers.0.self_attn.c_attn.bias" in m.param_map
    # Gemma: norm weights + 1, no lm_head parameter whatever the config says; Gemma2 adds two norms per layer
    m, q = loader.MODEL_MAPPINGS["gemma"](dict(base, model_type="gemma"))
    n0 = "model.layers.0.input_layernorm.weight"
    want = (t[n0].astype(np.float32) + 1.0).astype(np.float16)
    assert np.array_equal(build(m, n0), want) and build(m, n0).dtype == np.float16
    assert np.array_equal(build(m, "model.norm.weight"), (t["model.norm.weight"].astype(np.float32) + 1).astype(np.float16))
    assert "lm_head.weight" not in m.param_map and "lm_head.weight" not in q
    assert np.array_equal(build(m, "model.layers.0.self_attn.qkv_proj.weight")[:64], t["model.layers.0.self_attn.q_proj.weight"])
    m2, _ = loader.MODEL_MAPPINGS["gemma2"](dict(base, model_type="gemma2"))
    extra = set(m2.param_map) - set(m.param_map)
    assert extra == {f"model.layers.{i}.{n}.weight" for i in range(2)
                     for n in ("pre_feedforward_layernorm", "post_feedforward_layernorm")}
    # Phi-3: fused tensors pass through under the transformer.h.<i>.mixer / mlp names
    p3 = {"model.embed_tokens.weight": t["model.embed_tokens.weight"], "model.norm.weight": t["model.norm.weight"],
          "lm_head.weight": t["lm_head.weight"]}
    for i in range(2):
        hf = f"model.layers.{i}"
        p3[f"{hf}.self_attn.qkv_proj.weight"] = rng.standard_normal((128, 64)).astype(np.float16)
        p3[f"{hf}.self_attn.o_proj.weight"] = t[f"{hf}.self_attn.o_proj.weight"]
        p3[f"{hf}.mlp.gate_up_proj.weight"] = rng.standard_normal((320, 64)).astype(np.float16)
        p3[f"{hf}.mlp.down_proj.weight"] = t[f"{hf}.mlp.down_proj.weight"]
        p3[f"{hf}.input_layernorm.weight"] = t[f"{hf}.input_layernorm.weight"]
        p3[f"{hf}.post_attention_layernorm.weight"] = t[f"{hf}.post_attention_layernorm.weight"]
    m, q = loader.MODEL_MAPPINGS["phi3"](dict(base, model_type="phi3"))
    assert m.param_map["transformer.h.1.mixer.qkv_proj.weight"] == ["model.layers.1.self_attn.qkv_proj.weight"]
    assert m.param_map["transformer.h.0.ln.weight"] == ["model.layers.0.input_layernorm.weight"]
    assert m.param_map["transformer.embd.weight"] == ["model.embed_tokens.weight"]
    assert set(q) == {"lm_head.weight", "transformer.embd.weight"} | {
        f"transformer.h.{i}.{n}.weight" for i in range(2)
        for n in ("mixer.qkv_proj", "mixer.out_proj", "mlp.gate_up_proj", "mlp.down_proj")}
    assert loader.check_parameter_usage(m, set(p3)) == set()


def test_convert_weight_unquantised_on_cpu(tmp_path):
    src, dst = str(tmp_path / "hf"), str(tmp_path / "mlc")
    tensors = _hf_tensors(LLAMA, seed=5)
    _write_checkpoint(src, LLAMA, tensors)
    meta = loader.convert_weight(src, dst, quantization="q0f16", device="cpu")
    params, meta2 = tensor_cache.load_tensor_cache(dst, verify_md5=True)
    assert meta == meta2 and meta["ParamSize"] == len(params) == 3 + 6 * 2
    assert meta["BitsPerParam"] == 16.0
    assert torch.equal(params["model.layers.0.self_attn.qkv_proj.weight"],
                       torch.cat([tensors[f"model.layers.0.self_attn.{p}_proj.weight"] for p in "qkv"]))
    assert json.load(open(os.path.join(dst, "mlc-chat-config.json")))["quantization"] == "q0f16"


def test_param_kind_and_scheme_flags_on_cpu(tmp_path, monkeypatch):
    """Names, shapes and dtypes of a converted directory for the schemes that differ from q4f16_1 in layout or in
    what they leave alone: q4f16_0 (KN: a Linear's words and scales transposed), q4f16_2 (embedding and final fc
    stay in floating point), q4bf16_1 (everything in bfloat16).  The packing itself is the GPU kernel's job (checked
    bit for bit in the gpu tests below); here the oracle stands in for it so that the host logic runs without one."""
    from mlc_llm_amd import ops

    assert loader.param_kind("model.embed_tokens.weight") == "embedding"
    assert loader.param_kind("transformer.embd.weight") == "embedding"
    assert loader.param_kind("lm_head.weight") == "final_fc"
    assert loader.param_kind("model.layers.3.moe.e1_e3.weight") == "experts"
    assert loader.param_kind("model.layers.3.moe.e2.weight") == "experts"
    assert loader.param_kind("model.layers.3.mlp.down_proj.weight") == "linear"
    assert loader.param_kind("model.layers.0.self_attn.c_attn.weight") == "linear"

    def fake_quantize(w, bits, group_size, round_mode=0):
        md = {torch.float16: "float16", torch.float32: "float32", torch.bfloat16: "bfloat16"}[w.dtype]
        qw, qs = o.quantize_dt(w.float().numpy(), o.SCHEMES["q4f16_1" if bits == 4 else "q3f16_1"], md)
        return torch.from_numpy(qw.view(np.int32)), torch.from_numpy(qs).to(w.dtype)

    monkeypatch.setattr(ops, "quantize", fake_quantize)
    src = str(tmp_path / "hf")
    tensors = _hf_tensors(LLAMA, seed=9)
    _write_checkpoint(src, LLAMA, tensors)
    h, inter, v = LLAMA["hidden_size"], LLAMA["intermediate_size"], LLAMA["vocab_size"]

    # q4f16_0: KN layout for every Linear (final fc included), embedding stays [vocab, words]
    dst = str(tmp_path / "kn")
    loader.convert_weight(src, dst, quantization="q4f16_0", device="cpu")
    p, _ = tensor_cache.load_tensor_cache(dst)
    assert tuple(p["model.layers.0.mlp.down_proj.q_weight"].shape) == (inter // 8, h)
    assert tuple(p["model.layers.0.mlp.down_proj.q_scale"].shape) == (inter // 32, h)
    assert tuple(p["model.layers.0.self_attn.qkv_proj.q_weight"].shape) == (h // 8, 2 * h)
    assert tuple(p["lm_head.q_weight"].shape) == (h // 8, v) and tuple(p["lm_head.q_scale"].shape) == (h // 32, v)
    assert tuple(p["model.embed_tokens.q_weight"].shape) == (v, h // 8)
    nk, _ = o.quantize(tensors["model.layers.0.mlp.down_proj.weight"].numpy(), o.SCHEMES["q4f16_1"])
    assert np.array_equal(p["model.layers.0.mlp.down_proj.q_weight"].numpy().view(np.uint32), nk.T)

    # q4f16_2: embedding and final fc are left in float16 under their .weight names
    dst = str(tmp_path / "f2")
    loader.convert_weight(src, dst, quantization="q4f16_2", device="cpu")
    p, _ = tensor_cache.load_tensor_cache(dst)
    assert "model.embed_tokens.q_weight" not in p and "lm_head.q_weight" not in p
    assert p["model.embed_tokens.weight"].dtype == torch.float16 and tuple(p["lm_head.weight"].shape) == (v, h)
    assert torch.equal(p["lm_head.weight"], tensors["lm_head.weight"])
    assert tuple(p["model.layers.1.mlp.gate_up_proj.q_weight"].shape) == (2 * inter, h // 8)

    # q4bf16_1: norms and scales in bfloat16; values come straight from the checkpoint, not through float16
    big = dict(tensors)
    big["model.norm.weight"] = torch.full((h,), 1.0e5, dtype=torch.float32).bfloat16()  # overflows float16
    src2 = str(tmp_path / "hf_bf16")
    _write_checkpoint(src2, LLAMA, {k: (t if k == "model.norm.weight" else t.bfloat16()) for k, t in big.items()})
    dst = str(tmp_path / "bf")
    loader.convert_weight(src2, dst, quantization="q4bf16_1", device="cpu")
    p, _ = tensor_cache.load_tensor_cache(dst)
    assert p["model.norm.weight"].dtype == torch.bfloat16 and torch.isfinite(p["model.norm.weight"].float()).all()
    assert float(p["model.norm.weight"][0]) == float(torch.tensor(1.0e5).bfloat16())
    assert p["model.layers.0.mlp.down_proj.q_scale"].dtype == torch.bfloat16
    qw, qs = o.quantize_dt(tensors["model.layers.0.mlp.down_proj.weight"].bfloat16().float().numpy(),
                           o.SCHEMES["q4f16_1"], "bfloat16")
    assert np.array_equal(p["model.layers.0.mlp.down_proj.q_weight"].numpy().view(np.uint32), qw)
    assert np.array_equal(p["model.layers.0.mlp.down_proj.q_scale"].float().numpy(), qs)

    # experts have no KN form (group_quantization.py:584-585)
    srcm = str(tmp_path / "hf_mixtral")
    _write_checkpoint(srcm, MIXTRAL, _hf_tensors(MIXTRAL, seed=2))
    with pytest.raises(NotImplementedError, match="KN"):
        loader.convert_weight(srcm, str(tmp_path / "mkn"), quantization="q4f16_0", device="cpu")


# ------------------------------------------------------------------------------ on the GPU

@pytest.mark.gpu
@pytest.mark.parametrize("scheme", ["q4bf16_1", "q4f32_1", "q4f16_0", "q4f16_2"])
def test_convert_weight_other_schemes_match_oracle(tmp_path, scheme):
    """The schemes beyond q4f16_1 / q3f16_1 through the real GPU quantizer: packed words and scales of every
    quantised parameter equal the oracle's for the scheme's model dtype and layout, bit for bit."""
    from mlc_llm_amd.quantization import QUANTIZATION

    quant = QUANTIZATION[scheme]
    md = quant.model_dtype
    tdt = {"float16": torch.float16, "float32": torch.float32, "bfloat16": torch.bfloat16}[md]
    src, dst = str(tmp_path / "hf"), str(tmp_path / "mlc")
    tensors = {k: t.float().mul(1.37).to(tdt) for k, t in _hf_tensors(LLAMA, seed=21).items()}
    _write_checkpoint(src, LLAMA, tensors, shards=2)
    loader.convert_weight(src, dst, quantization=scheme, device="cuda:0")
    params, _ = tensor_cache.load_tensor_cache(dst, device="cpu", verify_md5=True)
    mapping, quantized = loader.llama_huggingface(LLAMA)
    np_t = {k: v.float().numpy() for k, v in tensors.items()}
    s = o.SCHEMES["q4f16_1"]
    # float32 tensors are stored as their upper 16 bits ("f32-to-bf16", interface/convert_weight.py:182-196 of the
    # reference): what comes back from the directory is that encoding of the exact value
    on_disk = (lambda a: tensor_cache.bf16_to_f32(tensor_cache.f32_to_bf16(a))) if md == "float32" else (lambda a: a)
    for name in mapping.param_map:
        full = mapping.map_func[name](*[np_t[n] for n in mapping.param_map[name]])
        kind = loader.param_kind(name)
        kept = name not in quantized or (kind == "embedding" and not quant.quantize_embedding) or \
            (kind == "final_fc" and not quant.quantize_final_fc)
        if kept:
            assert params[name].dtype == tdt and np.array_equal(params[name].float().numpy(), on_disk(full)), name
            continue
        base = name[: -len(".weight")]
        qw, qs = o.quantize_dt(full, s, md)
        if quant.linear_weight_layout == "KN" and kind in ("linear", "final_fc"):
            qw, qs = qw.T, qs.T
        assert np.array_equal(params[f"{base}.q_weight"].numpy().view(np.uint32), qw), name
        assert params[f"{base}.q_scale"].dtype == tdt
        assert np.array_equal(params[f"{base}.q_scale"].float().numpy(), on_disk(qs)), name



@pytest.mark.gpu
@pytest.mark.parametrize("scheme", ["q4f16_1", "q3f16_1"])
@pytest.mark.parametrize("cfg", [LLAMA, MIXTRAL, QWEN2], ids=["llama", "mixtral", "qwen2"])
def test_convert_weight_quantised_matches_oracle(tmp_path, cfg, scheme):
    import mlc_llm_amd as gq
    from mlc_llm_amd import ops

    src, dst = str(tmp_path / "hf"), str(tmp_path / "mlc")
    tensors = _hf_tensors(cfg, seed=zlib.crc32(scheme.encode()) & 0xFFFF)
    _write_checkpoint(src, cfg, tensors, shards=3)
    meta = loader.convert_weight(src, dst, quantization=scheme, device="cuda:0")
    params, _ = tensor_cache.load_tensor_cache(dst, device="cpu", verify_md5=True)
    s = o.SCHEMES[scheme]
    mapping, quantized = loader.MODEL_MAPPINGS[cfg["model_type"]](cfg)
    assert meta["ParamSize"] == len(params) == len(mapping.param_map) + len(quantized)
    np_t = {k: v.numpy() for k, v in tensors.items()}
    for name in mapping.param_map:
        full = mapping.map_func[name](*[np_t[n] for n in mapping.param_map[name]])
        if name in quantized:
            base = name[: -len(".weight")]
            qw, qs = o.quantize(full, s)
            assert np.array_equal(params[f"{base}.q_weight"].numpy().view(np.uint32), qw), name
            assert np.array_equal(params[f"{base}.q_scale"].numpy().view(np.uint16), qs.view(np.uint16)), name
            assert name not in params
        else:
            assert np.array_equal(params[name].numpy(), full), name
    # the converted directory feeds the kernels: one projection against the oracle
    name = "model.layers.0.self_attn." + ("c_attn" if cfg["model_type"] == "qwen2" else "qkv_proj")
    dev = torch.device("cuda:0")
    x = np.random.default_rng(1).standard_normal((3, cfg["hidden_size"])).astype(np.float16)
    bias = params.get(f"{name}.bias")  # Qwen2: the concatenated q / k / v bias, kept in float16
    assert (bias is not None) == (cfg["model_type"] == "qwen2")
    y = ops.linear(torch.from_numpy(x).to(dev), params[f"{name}.q_weight"].to(dev), params[f"{name}.q_scale"].to(dev),
                   s.bits, s.group_size, bias.to(dev) if bias is not None else None)
    ref = o.linear_fp32(x, params[f"{name}.q_weight"].numpy().view(np.uint32), params[f"{name}.q_scale"].numpy(), s,
                        bias.numpy() if bias is not None else None)
    err, bound, rel = o.check_linear(y.float().cpu().numpy(), ref, x, cfg["hidden_size"])
    assert err <= bound and rel <= 2e-3  # the linear tolerance of the hot path


@pytest.mark.gpu
def test_converted_directory_loads_into_quantized_modules(tmp_path):
    """HF checkpoint -> convert_weight -> load_tensor_cache -> load_state_dict into a module tree
    rewritten by GroupQuantize.quantize_model -> one decoder MLP + residual on the GPU, against
    fp64 arithmetic over the dequantised weights."""
    from torch import nn

    from mlc_llm_amd import ops
    from mlc_llm_amd.quantization import QUANTIZATION, QuantizeMapping

    cfg = dict(LLAMA, hidden_size=256, intermediate_size=384, num_hidden_layers=1)
    src, dst = str(tmp_path / "hf"), str(tmp_path / "mlc")
    tensors = _hf_tensors(cfg, seed=11)
    _write_checkpoint(src, cfg, tensors, shards=1)
    loader.convert_weight(src, dst, quantization="q4f16_1", device="cuda:0")
    params, _ = tensor_cache.load_tensor_cache(dst, device="cuda:0")

    class MLP(nn.Module):
        def __init__(self):
            super().__init__()
            self.gate_up_proj = nn.Linear(256, 2 * 384, bias=False)
            self.down_proj = nn.Linear(384, 256, bias=False)

    class Layer(nn.Module):
        def __init__(self):
            super().__init__()
            self.mlp = MLP()

    class Model(nn.Module):
        def __init__(self):
            super().__init__()
            self.layers = nn.ModuleList([Layer()])

    class Top(nn.Module):
        def __init__(self):
            super().__init__()
            self.model = Model()

    top = Top().half().to("cuda:0")
    quant = QUANTIZATION["q4f16_1"]
    qmap = QuantizeMapping({}, {})
    top = quant.quantize_model(top, qmap, "")
    assert qmap.param_map["model.layers.0.mlp.down_proj.weight"] == [
        "model.layers.0.mlp.down_proj.q_weight", "model.layers.0.mlp.down_proj.q_scale"]
    wanted = {k: v for k, v in params.items() if ".mlp." in k}
    top.load_state_dict(wanted, strict=True)  # names and shapes of the directory are the modules'
    mlp = top.model.layers[0].mlp

    x = np.random.default_rng(4).standard_normal((5, 256)).astype(np.float16)
    xd = torch.from_numpy(x).to("cuda:0")
    h = ops.silu_mul(mlp.gate_up_proj(xd))
    y = ops.linear(h, mlp.down_proj.q_weight, mlp.down_proj.q_scale, 4, 32, residual=xd)  # x + down(act)

    s = o.SCHEMES["q4f16_1"]
    gu = np.concatenate([tensors["model.layers.0.mlp.gate_proj.weight"].numpy(),
                         tensors["model.layers.0.mlp.up_proj.weight"].numpy()], axis=0)
    qw1, qs1 = o.quantize(gu, s)
    qw2, qs2 = o.quantize(tensors["model.layers.0.mlp.down_proj.weight"].numpy(), s)
    g_ref = o.linear_fp32(x, qw1, qs1, s).astype(np.float16)   # the fp16 the first kernel hands on
    act = o.silu_mul_f16(g_ref)
    ref = o.linear_fp32(h.cpu().numpy(), qw2, qs2, s) + x.astype(np.float64)
    err, bound, rel = o.check_linear(y.float().cpu().numpy(), ref, h.cpu().numpy(), 384)
    assert err <= bound and rel <= 2e-3
    # and the whole block against the oracle end to end (two roundings to fp16 on the way)
    ref_all = o.linear_fp32(act, qw2, qs2, s) + x.astype(np.float64)
    assert np.abs(y.float().cpu().numpy() - ref_all).max() <= 2 * bound + 1e-2
