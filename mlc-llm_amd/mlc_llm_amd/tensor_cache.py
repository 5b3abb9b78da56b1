"""Reader and writer of the MLC weight directory: ``tensor-cache.json`` + ``params_shard_*.bin``.

The reference writes this format with ``tvmjs.dump_tensor_cache`` (call site
python/mlc_llm/interface/convert_weight.py:182-196: ``encode_format="f32-to-bf16"``, metadata
``ParamSize`` / ``ParamBytes`` / ``BitsPerParam``) and reads it with TVM's
``TensorCacheMetadata`` (cpp/multi_gpu/multi_gpu_loader.cc:162-190, cpp/serve/function_table.cc:155-204)
or ``tvmjs.load_tensor_cache`` (python/mlc_llm/serve/engine_utils.py:288).  Both live in Apache TVM
(``python/tvm/contrib/tvmjs.py``, ``src/runtime/vm/tensor_cache_support.cc``), which is not part
of the reference tree, so the layout below is restated from that published format:

``tensor-cache.json``::

    {"metadata": {...},
     "records": [{"dataPath": "params_shard_0.bin", "format": "raw-shard", "nbytes": N,
                  "records": [{"name": ..., "shape": [...], "dtype": "uint32", "format": "raw",
                               "nbytes": n, "byteOffset": o}, ...],
                  "md5sum": "..."}, ...]}

Tensors are little-endian raw bytes.  Only float32 tensors are re-encoded (``"f32-to-bf16"``:
round-to-nearest-even to the upper 16 bits, truncation outside the bf16 range); ``q_weight``
(uint32) and ``q_scale`` (float16) are stored raw.  A tensor of at least the shard size gets a
shard of its own, others are appended until the shard would overflow (32 MiB by default).

PARITY UNPINNED: no weight directory ships with the reference and TVM is absent, so the format is
checked here only by round trip and by the schema fields the reference's own readers touch
(``records[].dataPath``, ``md5sum``: python/mlc_llm/support/download_cache.py:183-191).
"""

from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Callable, Dict, Iterable, Iterator, List, Optional, Tuple, Union

import numpy as np
import torch

TENSOR_CACHE_JSON = "tensor-cache.json"
LEGACY_CACHE_JSON = "ndarray-cache.json"  # name used by older converted models
SHARD_PREFIX = "params_shard"

ArrayLike = Union[np.ndarray, torch.Tensor]

_NP_DTYPES = {
    "float16": np.float16, "float32": np.float32, "float64": np.float64,
    "uint32": np.uint32, "int32": np.int32, "uint16": np.uint16, "int16": np.int16,
    "uint8": np.uint8, "int8": np.int8, "int64": np.int64, "uint64": np.uint64, "bool": np.bool_,
}


def _to_numpy(t: ArrayLike) -> Tuple[np.ndarray, str]:
    """Host array + dtype string of the record.  Packed storage travels as int32 in torch (which
    has no full uint32 support) and is recorded as what it is, uint32, when flagged by the caller
    through a numpy uint32 array; a torch.int32 tensor stays int32."""
    if isinstance(t, torch.Tensor):
        if t.dtype == torch.bfloat16:
            a = t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)
            return a, "bfloat16"
        a = t.detach().cpu().contiguous().numpy()
    else:
        a = np.ascontiguousarray(t)
    name = a.dtype.name
    if name not in _NP_DTYPES:
        raise TypeError(f"tensor cache: unsupported dtype {a.dtype}")
    return a, name


def f32_to_bf16(value: np.ndarray) -> np.ndarray:
    """float32 -> the upper 16 bits, round to nearest even inside the bf16 range, truncation
    outside it (so that +-max float32 clip to +-max bf16 instead of overflowing to inf)."""
    value = np.ascontiguousarray(value, dtype=np.float32)
    bits = value.view(np.uint32)
    limit = np.array([0x7F7F0000], dtype=np.uint32).view(np.float32)[0]  # largest finite bf16
    inside = np.logical_and(value < limit, value > -limit)
    bias = np.where(inside, ((bits >> 16) & 1) + np.uint32(0x7FFF), np.uint32(0)).astype(np.uint32)
    return ((bits + bias) >> 16).astype(np.uint16)


def bf16_to_f32(value: np.ndarray) -> np.ndarray:
    return (value.astype(np.uint32) << 16).view(np.float32)


class _ShardWriter:
    def __init__(self, cache_dir: str, cap: int):
        self.cache_dir, self.cap = cache_dir, cap
        self.counter = 0
        self.buf = bytearray()
        self.pending: List[Dict[str, Any]] = []
        self.shards: List[Dict[str, Any]] = []

    def _write(self, data: bytes, records: List[Dict[str, Any]]) -> None:
        path = f"{SHARD_PREFIX}_{self.counter}.bin"
        self.counter += 1
        with open(os.path.join(self.cache_dir, path), "wb") as f:
            f.write(data)
        self.shards.append({"dataPath": path, "format": "raw-shard", "nbytes": len(data),
                            "records": records, "md5sum": hashlib.md5(data).hexdigest()})

    def add(self, data: bytes, rec: Dict[str, Any]) -> None:
        if len(data) >= self.cap:  # a shard of its own, written at once (order of shards = order of arrival)
            rec["byteOffset"] = 0
            self._write(data, [rec])
            return
        if len(self.buf) + len(data) > self.cap:
            self.commit()
        rec["byteOffset"] = len(self.buf)
        self.pending.append(rec)
        self.buf += data

    def commit(self) -> None:
        if self.pending:
            self._write(bytes(self.buf), self.pending)
            self.buf, self.pending = bytearray(), []


def dump_tensor_cache(params: Union[Dict[str, ArrayLike], Iterable[Tuple[str, ArrayLike]]],
                      cache_dir: str, encode_format: str = "f32-to-bf16",
                      meta_data: Union[None, Dict[str, Any], Callable[[], Dict[str, Any]]] = None,
                      shard_cap_mb: int = 32) -> Dict[str, Any]:
    """Write ``params`` (name -> tensor, in iteration order) under ``cache_dir``; returns the
    JSON document.  ``meta_data`` may be a callable evaluated after the last tensor, as in the
    reference's converter (its totals are only known then)."""
    if encode_format not in ("f32-to-bf16", "raw"):
        raise ValueError(f"unknown encode_format {encode_format!r}")
    os.makedirs(cache_dir, exist_ok=True)
    writer = _ShardWriter(cache_dir, shard_cap_mb * (1 << 20))
    items = params.items() if isinstance(params, dict) else params
    seen = set()
    for name, tensor in items:
        if name in seen:
            raise ValueError(f"tensor cache: duplicate parameter {name}")
        seen.add(name)
        a, dtype = _to_numpy(tensor)
        fmt = "raw"
        if encode_format == "f32-to-bf16" and dtype == "float32":
            data, fmt = f32_to_bf16(a).tobytes(), "f32-to-bf16"
        else:
            data = a.tobytes()
        writer.add(data, {"name": name, "shape": [int(d) for d in a.shape], "dtype": dtype,
                          "format": fmt, "nbytes": len(data)})
    writer.commit()
    meta = meta_data() if callable(meta_data) else dict(meta_data or {})
    doc = {"metadata": meta, "records": writer.shards}
    with open(os.path.join(cache_dir, TENSOR_CACHE_JSON), "w", encoding="utf-8") as f:
        json.dump(doc, f, indent=2)
    return doc


def load_metadata(cache_dir: str) -> Dict[str, Any]:
    for name in (TENSOR_CACHE_JSON, LEGACY_CACHE_JSON):
        path = os.path.join(cache_dir, name)
        if os.path.isfile(path):
            with open(path, encoding="utf-8") as f:
                return json.load(f)
    raise FileNotFoundError(f"no {TENSOR_CACHE_JSON} under {cache_dir}")


def _decode(rec: Dict[str, Any], raw: np.ndarray) -> Tuple[np.ndarray, str]:
    """raw: uint8 view of the record's bytes -> (array, dtype string)."""
    shape, dtype, fmt = tuple(rec["shape"]), rec["dtype"], rec.get("format", "raw")
    count = int(np.prod(shape, dtype=np.int64)) if shape else 1
    if fmt == "f32-to-bf16":
        if dtype != "float32" or raw.size != 2 * count:
            raise ValueError(f"{rec['name']}: f32-to-bf16 record with dtype {dtype}, {raw.size} bytes")
        return bf16_to_f32(raw.view(np.uint16)).reshape(shape), dtype
    if fmt != "raw":
        raise ValueError(f"{rec['name']}: unknown record format {fmt!r}")
    if dtype == "bfloat16":
        np_dtype = np.uint16
    elif dtype in _NP_DTYPES:
        np_dtype = _NP_DTYPES[dtype]
    else:
        raise TypeError(f"{rec['name']}: unsupported dtype {dtype}")
    if raw.size != count * np.dtype(np_dtype).itemsize:
        raise ValueError(f"{rec['name']}: {raw.size} bytes for shape {shape} of {dtype}")
    return raw.view(np_dtype).reshape(shape), dtype


def _to_torch(a: np.ndarray, dtype: str, device) -> torch.Tensor:
    if dtype == "uint32":  # packed storage: same bits, the dtype the ops of this package take
        t = torch.from_numpy(np.ascontiguousarray(a).view(np.int32))
    elif dtype == "bfloat16":
        t = torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)
    elif dtype in ("uint16", "uint64"):
        raise TypeError(f"dtype {dtype} has no torch counterpart")
    else:
        t = torch.from_numpy(np.ascontiguousarray(a))
    return t.to(device)


def iter_tensor_cache(cache_dir: str, device="cpu", verify_md5: bool = False,
                      names: Optional[Iterable[str]] = None) -> Iterator[Tuple[str, torch.Tensor]]:
    """Yield (name, tensor) in file order, one shard file mapped at a time."""
    want = set(names) if names is not None else None
    for shard in load_metadata(cache_dir)["records"]:
        if shard.get("format", "raw-shard") != "raw-shard":
            raise ValueError(f"{shard['dataPath']}: unknown shard format {shard.get('format')!r}")
        if want is not None and not any(r["name"] in want for r in shard["records"]):
            continue
        path = os.path.join(cache_dir, shard["dataPath"])
        size = os.path.getsize(path)
        if size != shard["nbytes"]:
            raise ValueError(f"{path}: {size} bytes on disk, {shard['nbytes']} recorded")
        data = np.memmap(path, dtype=np.uint8, mode="r") if size else np.zeros(0, np.uint8)
        if verify_md5 and "md5sum" in shard:
            if hashlib.md5(data.tobytes()).hexdigest() != shard["md5sum"]:
                raise ValueError(f"{path}: md5 mismatch")
        for rec in shard["records"]:
            if want is not None and rec["name"] not in want:
                continue
            lo = rec["byteOffset"]
            hi = lo + rec["nbytes"]
            if lo < 0 or hi > size:
                raise ValueError(f"{rec['name']}: bytes [{lo}, {hi}) outside {path}")
            a, dtype = _decode(rec, np.array(data[lo:hi]))  # a copy: the mapping goes away with the shard
            yield rec["name"], _to_torch(a, dtype, device)
        del data


def load_tensor_cache(cache_dir: str, device="cpu", verify_md5: bool = False
                      ) -> Tuple[Dict[str, torch.Tensor], Dict[str, Any]]:
    """All parameters and the metadata block (the pair ``tvmjs.load_tensor_cache`` returns)."""
    params = dict(iter_tensor_cache(cache_dir, device, verify_md5))
    return params, load_metadata(cache_dir).get("metadata", {})
