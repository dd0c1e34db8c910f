"""q4f16_1 weights packed along N (tests/python/dlight/test_gpu_matmul.py:352-401: W uint32 [K, N/8], S fp16
[K, N/32]): the load-time rearrangement and the GEMM against the CPU oracle, through the C ABI.

The oracle needs no new function: the decode block of that fixture (:366-377) is format A's decode with the two
dimensions exchanged, D[k, n] = q4g32_dequant(W, S)[k, n] for the same two arrays, and the matmul reads D[k, n]
where format A's reads D[n, k]."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch

    assert torch.cuda.is_available(), "these tests need a GPU"
    from relax_amd import ops
    from tests import gpu_util

    return ops, gpu_util, torch


def _inputs(oracle, M, N, K, seed):
    """x [M, K]; W [K, N/8], S [K, N/32] drawn like format A's operands of a [K, N] matrix."""
    _, W, S = oracle.make_q4g32_inputs(1, K, N, seed)  # (rows = K, row length = N)
    x = np.random.default_rng(seed + 1).standard_normal((M, K)).astype(np.float16)
    return x, W, S


def test_prepare_is_a_pure_rearrangement(env, oracle):
    ops, u, torch = env
    for N, K in [(32, 8), (96, 64), (4128, 320), (4096, 4096)]:
        _, W, S = _inputs(oracle, 1, N, K, seed=N + K)
        W_nk, ST = ops.q4n32_prepare(u.dev(W), u.dev(S))
        k, n = np.arange(K), np.arange(N)
        codes = ((W[:, n // 8] >> (4 * (n % 8)).astype(np.uint32)[None, :]) & 15).astype(np.uint32)  # [K, N]
        want = np.zeros((N, K // 8), np.uint32)
        for j in range(8):
            want |= codes[j::8, :].T << np.uint32(4 * j)
        assert np.array_equal(u.host(W_nk).view(np.uint32), want), (N, K)
        assert np.array_equal(u.host(ST).view(np.uint16), np.ascontiguousarray(S.T).view(np.uint16)), (N, K)
        # and the fp16 weight [K, N] is what the format-A decode returns for the unprepared operands
        D = u.host(ops.q4g32_dequantize(u.dev(W), u.dev(S)))
        ref = ((codes.astype(np.float16) - np.float16(7)) * S[:, n // 32]).astype(np.float16)
        assert np.array_equal(D.view(np.uint16), ref.view(np.uint16)), (N, K)
        assert np.array_equal(oracle.q4g32_dequant(W, S).view(np.uint16), ref.view(np.uint16)), (N, K)


# the fixture's shape (4096 x 4096, dynamic n) at several n; ragged tiles: N not a multiple of the tile width,
# M one row, one more than a tile, K of one and of a few steps
# (up to 8 rows of x run the streaming kernel, up to 4 rows per pass over the weights, and more rows where that is
# cheaper than a GEMM of few tiles: 17 x 4096 x 4096 streams, 17 x 11008 x 4096 does not; else the matrix-core GEMM)
# (N = 16384 and 32800: the streaming kernel with 16 and with 32 rows per workgroup)
SHAPES = [(1, 4096, 4096), (2, 16384, 128), (1, 32800, 64), (2, 96, 64), (3, 4128, 320), (4, 11008, 4096), (1, 64, 32768), (4, 32, 28672), (2, 4096, 11008),
          (5, 4096, 4096), (7, 4096, 4096), (8, 4128, 320), (6, 160, 11008), (3, 96, 32768), (9, 4096, 4096), (17, 4096, 4096), (17, 11008, 4096), (13, 256, 8192), (130, 4096, 4096), (513, 4096, 4096), (33, 96, 64), (257, 160, 192),
          (300, 4128, 320), (64, 11008, 4096), (1100, 2048, 1024)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_linear_matches_oracle(env, oracle, M, N, K):
    ops, u, torch = env
    x, W, S = _inputs(oracle, M, N, K, seed=M + N + K)
    rng = np.random.default_rng(4)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    Bt = np.ascontiguousarray(oracle.q4g32_dequant(W, S).T)  # [N, K]
    W_nk, ST = ops.q4n32_prepare(u.dev(W), u.dev(S))
    print(f"q4n32 linear M={M} N={N} K={K}", flush=True)
    got = u.host(ops.q4n32_linear(W_nk, ST, u.dev(x)))
    u.assert_close(got, oracle.nt_matmul_f32acc(Bt, x, nthreads=8), f"q4n32 {M}x{N}x{K}")
    got = u.host(ops.q4n32_linear(W_nk, ST, u.dev(x), u.dev(bias), u.dev(res)))
    u.assert_close(got, oracle.nt_matmul_f32acc(Bt, x, bias, res, nthreads=8), f"q4n32 {M}x{N}x{K} + bias + residual")


def test_one_hot_rows_select_the_reference_weight_bit_for_bit(env, oracle):
    ops, u, torch = env
    N, K = 416, 256
    _, W, S = _inputs(oracle, 1, N, K, seed=9)
    D = oracle.q4g32_dequant(W, S)  # [K, N]
    W_nk, ST = ops.q4n32_prepare(u.dev(W), u.dev(S))
    x = np.eye(K, dtype=np.float16)  # row k selects w[k, :]
    got = u.host(ops.q4n32_linear(W_nk, ST, u.dev(x)))
    assert np.array_equal(got.view(np.uint16), D.view(np.uint16))


def test_one_hot_rows_through_the_streaming_kernel(env, oracle):
    """The same with 4 rows of x per call: the decode kernel rounds x * s instead of (code - 7) * s, which for
    x = 1 is the same number."""
    ops, u, torch = env
    N, K = 160, 192
    _, W, S = _inputs(oracle, 1, N, K, seed=10)
    D = oracle.q4g32_dequant(W, S)  # [K, N]
    W_nk, ST = ops.q4n32_prepare(u.dev(W), u.dev(S))
    eye = np.eye(K, dtype=np.float16)
    for k0 in range(0, K, 4):
        got = u.host(ops.q4n32_linear(W_nk, ST, u.dev(eye[k0:k0 + 4])))
        assert np.array_equal(got.view(np.uint16), D[k0:k0 + 4].view(np.uint16)), k0


def test_every_tile_shape_gives_the_same_sums(env, oracle):
    """The tile shape is chosen from M and N; forced through the test hook, the three shapes agree with the oracle."""
    ops, u, torch = env
    from relax_amd import _lib

    M, N, K = 200, 1056, 512
    x, W, S = _inputs(oracle, M, N, K, seed=2)
    ref = oracle.nt_matmul_f32acc(np.ascontiguousarray(oracle.q4g32_dequant(W, S).T), x, nthreads=8)
    W_nk, ST = ops.q4n32_prepare(u.dev(W), u.dev(S))
    try:
        for cfg in (11, 17, 18):
            _lib.lib().wq_debug_set_gemm_config(cfg)
            u.assert_close(u.host(ops.q4n32_linear(W_nk, ST, u.dev(x))), ref, f"q4n32 tile shape {cfg}")
            # (a forced tile shape also keeps one or two rows on the GEMM)
            u.assert_close(u.host(ops.q4n32_linear(W_nk, ST, u.dev(x[:2]))), ref[:2], f"q4n32 tile shape {cfg}, 2 rows")
    finally:
        _lib.lib().wq_debug_set_gemm_config(0)


def test_arguments(env):
    ops, u, torch = env
    from relax_amd import _lib

    W_nk = torch.zeros((64, 4), dtype=torch.int32, device="cuda")   # K = 32: not a multiple of 64
    ST = torch.zeros((2, 32), dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.WqError, match="multiple of 64"):
        ops.q4n32_linear(W_nk, ST, torch.zeros((1, 32), dtype=torch.float16, device="cuda"))
    W_nk = torch.zeros((64, 8), dtype=torch.int32, device="cuda")
    ST = torch.zeros((2, 64), dtype=torch.float16, device="cuda")
    assert ops.q4n32_linear(W_nk, ST, torch.zeros((0, 64), dtype=torch.float16, device="cuda")).shape == (0, 64)
    y = ops.q4n32_linear(W_nk, ST, torch.ones((3, 64), dtype=torch.float16, device="cuda"))
    assert torch.count_nonzero(y) == 0  # zero scales
