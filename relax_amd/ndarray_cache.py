"""Reader / writer of the NDArray-cache directory format that quantized Relax checkpoints are stored in
(`ndarray-cache.json` + `params_shard_<i>.bin`), so that packed weights and scales produced by the existing
quantization passes can be fed to this library without TVM.

Format (python/tvm/contrib/tvmjs.py:68-259):
  ndarray-cache.json = {"metadata": <any>, "records": [shard, ...]}
  shard  = {"dataPath": "params_shard_<i>.bin", "format": "raw-shard", "nbytes": n, "md5sum": hex,
            "records": [entry, ...]}
  entry  = {"name", "shape", "dtype", "format": "raw" | "f32-to-bf16", "nbytes", "byteOffset"}
Entries are laid back to back in their shard.  A shard is closed before an entry that would bring it to the
cap (32 MB by default); an entry of at least half the cap gets a shard of its own.  With "f32-to-bf16",
float32 tensors are stored as bfloat16 bits (round to nearest even inside the finite bf16 range, truncation
outside it) and widened again on load; a second index, ndarray-cache-b16.json, describes the same shards
with those entries typed "bfloat16"/"raw".
"""
from __future__ import annotations

import hashlib
import json
import math
import os
from typing import Any, Dict, Iterable, Mapping, Tuple, Union

import numpy as np

INDEX = "ndarray-cache.json"
INDEX_B16 = "ndarray-cache-b16.json"


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """float32 -> uint16 bfloat16 bit patterns, the writer's rule (tvmjs.py:36-52)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    bits = a.view(np.uint32)
    limit = np.array([np.finfo(np.float32).max], np.float32).view(np.uint32)
    limit = ((limit >> 16) << 16).view(np.float32)[0]  # largest finite bf16
    inside = (a < limit) & (a > -limit)
    bias = np.where(inside, ((bits >> 16) & 1) + 0x7FFF, 0).astype(np.uint32)
    return ((bits + bias) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def _md5(path: str) -> str:
    h = hashlib.md5()
    with open(path, "rb") as f:
        for chunk in iter(lambda: f.read(1 << 20), b""):
            h.update(chunk)
    return h.hexdigest()


class _ShardWriter:
    def __init__(self, cache_dir: str, cap: int):
        self.dir, self.cap = cache_dir, cap
        self.shards, self.pending, self.entries, self.count = [], bytearray(), [], 0

    def _write(self, data, entries):
        name = f"params_shard_{self.count}.bin"
        self.count += 1
        path = os.path.join(self.dir, name)
        with open(path, "wb") as f:
            f.write(data)
        self.shards.append({"dataPath": name, "format": "raw-shard", "nbytes": len(data), "records": entries,
                            "md5sum": _md5(path)})

    def flush(self):
        if self.pending:
            self._write(self.pending, self.entries)
            self.pending, self.entries = bytearray(), []

    def add(self, entry: dict, data: bytes):
        if len(self.pending) + len(data) >= self.cap:
            if 2 * len(data) >= self.cap:  # large entry: a shard of its own, pending shard stays open
                entry["byteOffset"] = 0
                self._write(data, [entry])
                return
            self.flush()
        entry["byteOffset"] = len(self.pending)
        self.entries.append(entry)
        self.pending += data


def dump(params: Union[Mapping[str, np.ndarray], Iterable[Tuple[str, np.ndarray]]], cache_dir: str,
         encode_format: str = "raw", meta_data: Any = None, shard_cap_mb: int = 32) -> dict:
    """Writes `params` (name -> array; device tensors are copied to the host) as an NDArray cache and
    returns the index that was written."""
    if encode_format not in ("raw", "f32-to-bf16"):
        raise ValueError(f"invalid encode_format {encode_format!r}")
    os.makedirs(cache_dir, exist_ok=True)
    w = _ShardWriter(cache_dir, shard_cap_mb << 20)
    any_bf16 = False
    items = params.items() if isinstance(params, Mapping) else params
    for name, v in items:
        if hasattr(v, "detach"):  # torch tensor
            v = v.detach().cpu().numpy()
        v = np.ascontiguousarray(v)
        dtype = str(v.dtype)
        if encode_format == "f32-to-bf16" and dtype == "float32":
            data = f32_to_bf16_bits(v).tobytes()
            any_bf16 = True
        else:
            data = v.tobytes()
        w.add({"name": name, "shape": [int(d) for d in v.shape], "dtype": dtype, "format": encode_format,
               "nbytes": len(data)}, data)
    w.flush()
    meta = {} if meta_data is None else (meta_data() if callable(meta_data) else meta_data)
    index = {"metadata": meta, "records": w.shards}
    with open(os.path.join(cache_dir, INDEX), "w") as f:
        json.dump(index, f, indent=4)
    if any_bf16:
        b16 = json.loads(json.dumps(index))
        for shard in b16["records"]:
            for e in shard["records"]:
                if e["dtype"] == "float32":
                    e["format"], e["dtype"] = "raw", "bfloat16"
        with open(os.path.join(cache_dir, INDEX_B16), "w") as f:
            json.dump(b16, f, indent=4)
    return index


def _entry_array(buf: np.ndarray, e: dict) -> np.ndarray:
    off, n = int(e["byteOffset"]), int(e["nbytes"])
    if off < 0 or off + n > buf.size:
        raise ValueError(f"entry {e['name']!r} lies outside its shard")
    raw = buf[off:off + n]
    shape, dtype = tuple(e["shape"]), e["dtype"]
    if e["format"] == "f32-to-bf16" and dtype == "float32":
        return bf16_bits_to_f32(raw.view(np.uint16)).reshape(shape)
    if dtype == "bfloat16":
        return raw.view(np.uint16).reshape(shape)  # bit patterns; the caller views them as bfloat16
    a = raw.view(np.dtype(dtype))
    if a.size != math.prod(shape):
        raise ValueError(f"entry {e['name']!r}: {n} bytes do not match shape {shape} of {dtype}")
    return a.reshape(shape)


def load(cachepath: str, device: str = "cpu", verify_md5: bool = False):
    """Reads a cache directory (or its .json index).  Returns ({name: array}, metadata); arrays are numpy
    for device "cpu" (views of memory-mapped shards, read-only), else torch tensors on `device` (uint32
    travels as int32, bfloat16 bit patterns become torch.bfloat16)."""
    if not cachepath.endswith(".json"):
        cachepath = os.path.join(cachepath, INDEX)
    root = os.path.dirname(cachepath)
    with open(cachepath) as f:
        index = json.load(f)
    out: Dict[str, Any] = {}
    for shard in index["records"]:
        if shard.get("format") != "raw-shard":
            raise ValueError(f"unknown shard format {shard.get('format')!r}")
        path = os.path.join(root, shard["dataPath"])
        if os.path.getsize(path) != int(shard["nbytes"]):
            raise ValueError(f"{path}: size differs from the index")
        if verify_md5 and "md5sum" in shard and _md5(path) != shard["md5sum"]:
            raise ValueError(f"{path}: md5 mismatch")
        buf = np.memmap(path, dtype=np.uint8, mode="r") if shard["nbytes"] else np.zeros(0, np.uint8)
        for e in shard["records"]:
            a = _entry_array(buf, e)
            if device == "cpu":
                out[e["name"]] = a
                continue
            import torch

            if a.dtype == np.uint32:
                t = torch.from_numpy(np.array(a).view(np.int32))
            elif e["dtype"] == "bfloat16":
                t = torch.from_numpy(np.array(a).view(np.int16)).view(torch.bfloat16)
            elif a.dtype == np.uint16:
                t = torch.from_numpy(np.array(a).view(np.int16))
            else:
                t = torch.from_numpy(np.array(a))
            out[e["name"]] = t.to(device)
    return out, index.get("metadata", {})
