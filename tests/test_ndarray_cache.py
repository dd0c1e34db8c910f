"""NDArray-cache directory format (python/tvm/contrib/tvmjs.py:68-259): a hand-written cache is read
correctly, the writer reproduces the sharding and bf16 rules, round trips are exact."""
import hashlib
import json
import os

import numpy as np
import pytest

from relax_amd import ndarray_cache as nc


def test_reads_a_hand_written_cache(tmp_path):
    # two shards written byte by byte as the format describes, including an f32-to-bf16 entry
    w = np.arange(24, dtype=np.uint32).reshape(3, 8) * 0x01010101
    s = np.array([[0.5, 0.25], [1.0, 2.0], [0.125, 4.0]], np.float16)
    f = np.array([1.0, -2.5, 3.0e38, 0.1], np.float32)
    shard0 = w.tobytes() + s.tobytes()
    shard1 = (f.view(np.uint32) >> 16).astype(np.uint16).tobytes()
    (tmp_path / "params_shard_0.bin").write_bytes(shard0)
    (tmp_path / "params_shard_1.bin").write_bytes(shard1)
    index = {"metadata": {"ParamSize": 3}, "records": [
        {"dataPath": "params_shard_0.bin", "format": "raw-shard", "nbytes": len(shard0), "md5sum": hashlib.md5(shard0).hexdigest(),
         "records": [{"name": "q_weight", "shape": [3, 8], "dtype": "uint32", "format": "raw", "nbytes": 96, "byteOffset": 0},
                     {"name": "q_scale", "shape": [3, 2], "dtype": "float16", "format": "raw", "nbytes": 12, "byteOffset": 96}]},
        {"dataPath": "params_shard_1.bin", "format": "raw-shard", "nbytes": len(shard1), "md5sum": hashlib.md5(shard1).hexdigest(),
         "records": [{"name": "norm", "shape": [4], "dtype": "float32", "format": "f32-to-bf16", "nbytes": 8, "byteOffset": 0}]}]}
    (tmp_path / "ndarray-cache.json").write_text(json.dumps(index))
    params, meta = nc.load(str(tmp_path), verify_md5=True)
    assert meta == {"ParamSize": 3}
    assert np.array_equal(params["q_weight"], w) and params["q_weight"].dtype == np.uint32
    assert np.array_equal(params["q_scale"], s)
    want = ((f.view(np.uint32) >> 16) << 16).view(np.float32)
    assert np.array_equal(params["norm"], want)
    # the .json path works as well as the directory
    p2, _ = nc.load(str(tmp_path / "ndarray-cache.json"))
    assert sorted(p2) == ["norm", "q_scale", "q_weight"]
    # corruption is detected
    (tmp_path / "params_shard_1.bin").write_bytes(shard1[:-1] + b"\x00")
    with pytest.raises(ValueError, match="md5"):
        nc.load(str(tmp_path), verify_md5=True)
    (tmp_path / "params_shard_1.bin").write_bytes(shard1[:-2])
    with pytest.raises(ValueError, match="size"):
        nc.load(str(tmp_path))


def test_bf16_rule():
    f = np.array([1.0, 1.00390625, 1.01171875, -1.00390625, 3.3895314e38, 3.4e38, -3.4e38, np.inf, 0.0, -0.0], np.float32)
    b = nc.f32_to_bf16_bits(f)
    # 1.00390625 = 0x3F808000 is a tie: rounds to the even mantissa 0x3F80; 1.01171875 = 0x3F818000 ties up to 0x3F82
    assert list(b[:4]) == [0x3F80, 0x3F80, 0x3F82, 0xBF80]
    # the largest finite bf16 and everything beyond it is truncated, not rounded (no overflow to inf)
    assert list(b[4:8]) == [0x7F7F, 0x7F7F, 0xFF7F, 0x7F80]
    assert list(b[8:]) == [0x0000, 0x8000]
    assert np.array_equal(nc.bf16_bits_to_f32(b[:1]), np.array([1.0], np.float32))
    # random values: nearest bf16 (error at most half a bf16 ulp)
    rng = np.random.default_rng(0)
    x = rng.standard_normal(10000).astype(np.float32) * 100
    back = nc.bf16_bits_to_f32(nc.f32_to_bf16_bits(x))
    assert np.all(np.abs(back - x) <= np.abs(x) * 2.0 ** -8)


def test_round_trip_and_sharding_rules(tmp_path):
    rng = np.random.default_rng(1)
    cap = 1 << 20  # 1 MB shards
    params = {
        "a": rng.integers(0, 2**32, size=(300, 512), dtype=np.uint64).astype(np.uint32),   # 600 KB >= cap/2 ...
        "b": rng.standard_normal((100, 16)).astype(np.float16),                            # 3.2 KB
        "c": rng.integers(-128, 128, size=(700, 1024)).astype(np.int8),                    # 700 KB: would pass the cap
        "d": rng.standard_normal((8,)).astype(np.float32),
        "e": np.zeros((0, 4), np.float16),
        "big": rng.integers(-128, 128, size=(3, 1 << 20)).astype(np.int8),                 # 3 MB: out of band
    }
    index = nc.dump(params, str(tmp_path), shard_cap_mb=1, meta_data=lambda: {"k": 1})
    on_disk = json.loads((tmp_path / "ndarray-cache.json").read_text())
    assert on_disk == index and index["metadata"] == {"k": 1}
    shards = index["records"]
    names = [[e["name"] for e in s["records"]] for s in shards]
    # "a" opens shard 0 and "b" joins it; "c" (>= cap/2, and a + b + c >= cap) and "big" get shards of their
    # own while the pending shard stays open and also takes "d" and "e"; it is written last
    assert names == [["c"], ["big"], ["a", "b", "d", "e"]]
    for s in shards:
        assert s["format"] == "raw-shard" and s["dataPath"].startswith("params_shard_")
        blob = (tmp_path / s["dataPath"]).read_bytes()
        assert len(blob) == s["nbytes"] and hashlib.md5(blob).hexdigest() == s["md5sum"]
        off = 0
        for e in s["records"]:
            assert e["byteOffset"] == off and e["format"] == "raw"
            off += e["nbytes"]
        assert off == s["nbytes"] and s["nbytes"] < cap or len(s["records"]) == 1
    loaded, meta = nc.load(str(tmp_path), verify_md5=True)
    assert meta == {"k": 1} and list(loaded) == ["c", "big", "a", "b", "d", "e"]
    for k, v in params.items():
        assert loaded[k].dtype == v.dtype and loaded[k].shape == v.shape and np.array_equal(loaded[k], v), k
    assert not os.path.exists(tmp_path / "ndarray-cache-b16.json")


def test_f32_to_bf16_cache(tmp_path):
    rng = np.random.default_rng(2)
    params = {"w": rng.standard_normal((64, 33)).astype(np.float32), "q": np.arange(12, dtype=np.uint32).reshape(3, 4)}
    nc.dump(params, str(tmp_path), encode_format="f32-to-bf16")
    loaded, _ = nc.load(str(tmp_path))
    assert np.array_equal(loaded["q"], params["q"])
    assert np.array_equal(loaded["w"], nc.bf16_bits_to_f32(nc.f32_to_bf16_bits(params["w"])))
    idx = json.loads((tmp_path / "ndarray-cache.json").read_text())["records"][0]["records"]
    assert {e["name"]: (e["dtype"], e["format"], e["nbytes"]) for e in idx} == {
        "w": ("float32", "f32-to-bf16", 64 * 33 * 2), "q": ("uint32", "f32-to-bf16", 48)}
    b16 = json.loads((tmp_path / "ndarray-cache-b16.json").read_text())["records"][0]["records"]
    assert {e["name"]: (e["dtype"], e["format"]) for e in b16} == {"w": ("bfloat16", "raw"), "q": ("uint32", "f32-to-bf16")}
    l16, _ = nc.load(str(tmp_path / "ndarray-cache-b16.json"))
    assert l16["w"].dtype == np.uint16 and np.array_equal(l16["w"], nc.f32_to_bf16_bits(params["w"]))
    with pytest.raises(ValueError):
        nc.dump(params, str(tmp_path), encode_format="zip")


@pytest.mark.gpu
def test_quantized_checkpoint_to_device_and_linear(tmp_path, oracle):
    """A q4f16_1 layer stored as a cache, loaded onto the GPU and multiplied."""
    import torch

    from relax_amd import ops
    from tests import gpu_util as u

    x, W, S = oracle.make_q4g32_inputs(4, 320, 512, seed=5)
    nc.dump({"layer.q_weight": W, "layer.q_scale": S}, str(tmp_path))
    p, _ = nc.load(str(tmp_path), device="cuda")
    assert p["layer.q_weight"].dtype == torch.int32 and p["layer.q_weight"].is_cuda
    got = u.host(ops.q4g32_linear(p["layer.q_weight"], p["layer.q_scale"], u.dev(x)))
    u.assert_close(got, oracle.q4g32_linear(W, S, x), "linear from a cache")
