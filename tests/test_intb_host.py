"""Host-side pieces of the format-B path that need no GPU: the reordering on host
memory (through the C ABI) against the golden vectors and the oracle."""
import os

import numpy as np
import pytest
import torch

GOLD = os.path.join(os.path.dirname(__file__), "golden", "ft_layout_vectors.npz")
CASES = ["int8_64x64", "int8_128x192", "int8_256x64", "int4_64x64", "int4_128x192", "int4_256x128"]


@pytest.fixture(scope="module")
def ops():
    from relax_amd import ops as _ops

    return _ops


@pytest.mark.parametrize("case", CASES)
def test_host_preprocess_matches_golden(ops, case):
    g = np.load(GOLD)
    a, want = g[case + "_in"], g[case + "_out"]
    got = ops.ft_preprocess_weight(torch.from_numpy(a), 80, case.startswith("int4")).numpy()
    assert got.dtype == np.int8 and got.shape == want.shape
    assert np.array_equal(got, want)


@pytest.mark.parametrize("is_int4", [False, True])
def test_host_preprocess_matches_oracle_and_experts(ops, oracle, is_int4):
    rng = np.random.default_rng(5)
    a = rng.integers(-128, 128, size=(3, 192, 128)).astype(np.int8)
    got = ops.ft_preprocess_weight(torch.from_numpy(a), 80, is_int4).numpy()
    assert np.array_equal(got, oracle.ft_preprocess(a, is_int4, 80))
    # the input is left untouched and a fresh tensor is returned
    assert got.ctypes.data != a.ctypes.data


def test_host_preprocess_errors(ops):
    from relax_amd._lib import WqError

    a = torch.zeros((64, 64), dtype=torch.int8)
    with pytest.raises(WqError, match="sm=90"):
        ops.ft_preprocess_weight(a, 90, False)
    with pytest.raises(WqError, match="multiples of 64"):
        ops.ft_preprocess_weight(torch.zeros((32, 64), dtype=torch.int8), 80, False)
    with pytest.raises(ValueError):
        ops.ft_preprocess_weight(a.to(torch.int32), 80, False)
    # empty tensors pass through
    assert ops.ft_preprocess_weight(torch.zeros((0, 64), dtype=torch.int8), 80, False).shape == (0, 64)


def test_gptq_host_side_checks(ops):
    """What the AutoGPTQ entry points decide on the host, before any kernel: workspace sizes, shape and
    pointer checks (null device pointers are never dereferenced: every call below fails its checks first)."""
    from relax_amd import _lib

    l = _lib.lib()
    assert ops.gptq_workspace_bytes(1, 4096, True) == 8192
    assert ops.gptq_workspace_bytes(300, 4096, True) == 300 * 4096 * 2
    assert ops.gptq_workspace_bytes(300, 4096, False) == 0 and ops.gptq_workspace_bytes(0, 4096, True) == 0
    # empty problems succeed without touching memory
    assert l.wq_gptq_linear(0, 0, 0, 0, 0, 0, 0, 0, 64, 256, 2, 0, 0, 0) == 0
    assert l.wq_gptq_dequantize(0, 0, 0, 0, 0, 0, 64, 2, 0) == 0
    # K not a multiple of the group count / group size not a multiple of 32 / null pointers
    assert l.wq_gptq_linear(0, 0, 0, 0, 0, 0, 0, 1, 64, 256, 3, 0, 0, 0) != 0 and b"groups" in l.wq_last_error()
    assert l.wq_gptq_linear(0, 0, 0, 0, 0, 0, 0, 1, 64, 192, 4, 0, 0, 0) != 0 and b"multiple of 32" in l.wq_last_error()
    assert l.wq_gptq_linear(0, 0, 0, 0, 0, 0, 0, 1, 64, 256, 2, 0, 0, 0) != 0 and b"null pointer" in l.wq_last_error()
    assert l.wq_gptq_dequantize(0, 0, 0, 0, 0, 12, 64, 1, 0) != 0 and b"multiples of 8" in l.wq_last_error()
    assert l.wq_gptq_prepare(0, 0, 0, 0, 0, 0, 0, 0, None, 256, 60, 2, 0) != 0 and b"multiple of 8" in l.wq_last_error()
