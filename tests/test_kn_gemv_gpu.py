"""The decode linear over a K-major q4f16_1 checkpoint used in place (wq_q4g32_kn_gemv), against the
K-major oracle (the decode of tests/python/dlight/test_gpu_reduction.py:102-120 followed by the fp32 matmul)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch

    assert torch.cuda.is_available()
    from relax_amd import ops as _ops

    return _ops


@pytest.fixture(scope="module")
def u():
    from tests import gpu_util

    return gpu_util


def _inputs(M, N, K, seed):
    rng = np.random.default_rng(seed)
    W_kn = rng.integers(0, 2**32, size=(K // 8, N), dtype=np.uint64).astype(np.uint32)
    S_kn = rng.uniform(0.005, 0.02, size=(K // 32, N)).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    return W_kn, S_kn, x


def _ref(oracle, W_kn, S_kn, x, bias=None, residual=None):
    """fp32-accumulated oracle over the bit-exact dequantized weight, epilogue as every linear of the library."""
    B = oracle.q4g32_kn_dequant(W_kn, S_kn)  # [K, N]
    return oracle.nt_matmul_f32acc(np.ascontiguousarray(B.T), x, bias, residual, nthreads=8)


# one slice (small K), many slices, ragged last slice and last column block; every row count of the passes (4, 2, 1)
_SMALL = [(4, 32), (72, 96), (260, 2048), (1000, 4096), (4096, 4096)]
_LLAMA = [(12288, 4096), (22016, 4096), (4096, 11008)]
_CASES = [(M, N, K) for N, K in _SMALL for M in (1, 2, 3, 4, 7, 16)] + [(M, N, K) for N, K in _LLAMA for M in (1, 2, 4, 16)]


@pytest.mark.parametrize("M,N,K", _CASES)
def test_kn_gemv_matches_oracle(ops, u, oracle, M, N, K):
    W_kn, S_kn, x = _inputs(M, N, K, seed=M + N + K)
    got = u.host(ops.q4g32_kn_gemv(u.dev(W_kn), u.dev(S_kn), u.dev(x)))
    u.assert_close(got, _ref(oracle, W_kn, S_kn, x), f"kn gemv {M}x{N}x{K}")


@pytest.mark.parametrize("N,K", [(72, 96), (4096, 4096)])
def test_kn_gemv_epilogue(ops, u, oracle, N, K):
    M = 5
    W_kn, S_kn, x = _inputs(M, N, K, seed=11)
    rng = np.random.default_rng(12)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    got = u.host(ops.q4g32_kn_gemv(u.dev(W_kn), u.dev(S_kn), u.dev(x), bias=u.dev(bias), residual=u.dev(res)))
    u.assert_close(got, _ref(oracle, W_kn, S_kn, x, bias, res), f"kn gemv bias + residual {N}x{K}")
    got = u.host(ops.q4g32_kn_gemv(u.dev(W_kn), u.dev(S_kn), u.dev(x), bias=u.dev(bias)))
    u.assert_close(got, _ref(oracle, W_kn, S_kn, x, bias), f"kn gemv bias {N}x{K}")


@pytest.mark.parametrize("N,K", [(264, 128), (4096, 4096)])
def test_kn_gemv_one_hot_rows_reproduce_the_dequantized_weight(ops, u, oracle, N, K):
    """x = e_k returns row k of the dequantized weight bit for bit: (code - 7) * scale with one rounding."""
    W_kn, S_kn, _ = _inputs(1, N, K, seed=5)
    B = oracle.q4g32_kn_dequant(W_kn, S_kn)
    ks = [0, 7, 8, 31, 33, K // 2 + 5, K - 1]
    x = np.zeros((len(ks), K), np.float16)
    for r, k in enumerate(ks):
        x[r, k] = 1.0
    got = u.host(ops.q4g32_kn_gemv(u.dev(W_kn), u.dev(S_kn), u.dev(x)))
    assert np.array_equal(got.view(np.uint16), B[ks].view(np.uint16))


def test_kn_gemv_agrees_with_the_transposed_path(ops, u, oracle):
    """The in-place kernel and kn_to_nk + the row-major linear see the same weights."""
    N, K, M = 4096, 4096, 2
    W_kn, S_kn, x = _inputs(M, N, K, seed=3)
    dW, dS, dx = u.dev(W_kn), u.dev(S_kn), u.dev(x)
    a = u.host(ops.q4g32_kn_gemv(dW, dS, dx)).astype(np.float64)
    W, S = ops.q4g32_kn_to_nk(dW, dS)
    b = u.host(ops.q4g32_linear(W, S, dx)).astype(np.float64)
    assert np.abs(a - b).max() <= 2e-3 * np.abs(b).max()


def test_kn_gemv_argument_errors(ops, u):
    import torch

    from relax_amd import _lib

    L = _lib.lib()
    W_kn, S_kn, x = _inputs(1, 8, 64, seed=1)
    dW, dS = u.dev(W_kn), u.dev(S_kn)
    with pytest.raises(ValueError):
        ops.q4g32_kn_gemv(dW, dS, torch.zeros((1, 32), dtype=torch.float16, device="cuda"))
    with pytest.raises(RuntimeError, match="convert the weights once"):
        ops.q4g32_kn_gemv(dW, dS, torch.zeros((17, 64), dtype=torch.float16, device="cuda"))
    # N not a multiple of 4
    W6 = torch.zeros((8, 6), dtype=torch.int32, device="cuda")
    S6 = torch.zeros((2, 6), dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="multiple of 4"):
        ops.q4g32_kn_gemv(W6, S6, torch.zeros((1, 64), dtype=torch.float16, device="cuda"))
    # a workspace that is too small
    N, K = 4096, 4096
    need = int(L.wq_q4g32_kn_gemv_workspace_bytes(1, N, K))
    assert need > 0
    Wb = torch.zeros((K // 8, N), dtype=torch.int32, device="cuda")
    Sb = torch.zeros((K // 32, N), dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="workspace"):
        ops.q4g32_kn_gemv(Wb, Sb, torch.zeros((1, K), dtype=torch.float16, device="cuda"),
                          workspace=torch.empty((need - 16,), dtype=torch.uint8, device="cuda"))
    # empty problems are accepted
    y = ops.q4g32_kn_gemv(dW, dS, torch.zeros((0, 64), dtype=torch.float16, device="cuda"))
    assert tuple(y.shape) == (0, 8)
