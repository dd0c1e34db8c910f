"""GPU parity of the format-A (q4f16_1) kernels against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch

    assert torch.cuda.is_available(), "these tests need a GPU"
    from relax_amd import ops as _ops

    return _ops


@pytest.fixture(scope="module")
def u():
    from tests import gpu_util

    return gpu_util


def test_unpack_bit_exact(ops, u, oracle):
    rng = np.random.default_rng(0)
    for N, K in [(1, 8), (3, 40), (257, 4096), (4096, 4096)]:
        W = rng.integers(0, 2**32, size=(N, K // 8), dtype=np.uint64).astype(np.uint32)
        got = u.host(ops.q4_unpack(u.dev(W)))
        assert np.array_equal(got, oracle.q4_unpack(W)), (N, K)
    # each code in each slot
    W = np.array([[(c << (4 * s)) for s in range(8)] for c in range(16)], np.uint32)
    assert np.array_equal(u.host(ops.q4_unpack(u.dev(W))), oracle.q4_unpack(W))
    # empty
    assert ops.q4_unpack(u.dev(np.zeros((0, 4), np.uint32))).shape == (0, 32)


def test_dequant_exhaustive_bit_exact(ops, u, oracle):
    """all 16 codes x all 65536 fp16 scale patterns (subnormals, inf, nan included)."""
    all_s = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16)
    codes = np.tile(np.arange(16, dtype=np.uint8), 2)[None, :].repeat(65536, 0)
    W = oracle.q4_pack(codes)
    S = all_s.reshape(65536, 1)
    got = u.host(ops.q4g32_dequantize(u.dev(W), u.dev(S)))
    want = oracle.q4g32_dequant(W, S)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])
    assert np.all(np.isnan(got[nan]))


def test_dequant_random_shapes(ops, u, oracle):
    for N, K, seed in [(5, 32, 1), (64, 352, 2), (4096, 4096, 3), (300, 11008, 4)]:
        _, W, S = oracle.make_q4g32_inputs(1, N, K, seed)
        got = u.host(ops.q4g32_dequantize(u.dev(W), u.dev(S)))
        assert np.array_equal(got.view(np.uint16), oracle.q4g32_dequant(W, S).view(np.uint16)), (N, K)


GEMV_SHAPES = [  # (M, N, K)
    (1, 4096, 4096),    # the single-GEMV configuration
    (1, 12288, 4096),   # fused QKV
    (1, 22016, 4096),   # fused gate/up
    (1, 4096, 11008),   # down
    (1, 1, 32), (1, 7, 64), (1, 1001, 2080), (1, 8, 32768),
    (2, 515, 4096), (2, 300, 11008), (3, 64, 256), (4, 4096, 4096), (5, 130, 11008), (8, 4096, 4096),
]


@pytest.mark.parametrize("M,N,K", GEMV_SHAPES)
def test_gemv_vs_oracle(ops, u, oracle, M, N, K):
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=M * 1000 + N + K)
    print(f"gemv M={M} N={N} K={K}", flush=True)
    got = u.host(ops.q4g32_linear(u.dev(W), u.dev(S), u.dev(x), kernel="gemv"))
    ref = oracle.q4g32_linear(W, S, x, nthreads=8)
    u.assert_close(got, ref, f"gemv {M}x{N}x{K}")


def test_gemv_epilogue_and_invariants(ops, u, oracle):
    M, N, K = 3, 520, 1024
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=77)
    rng = np.random.default_rng(5)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    got = u.host(ops.q4g32_linear(u.dev(W), u.dev(S), u.dev(x), bias=u.dev(bias), residual=u.dev(res), kernel="gemv"))
    u.assert_close(got, oracle.q4g32_linear(W, S, x, bias=bias, residual=res), "gemv epilogue")
    # one-hot x selects a dequantized column exactly
    B = oracle.q4g32_dequant(W, S)
    for k in (0, 5, 36, 1023):
        xh = np.zeros((1, K), np.float16)
        xh[0, k] = 1
        y = u.host(ops.q4g32_linear(u.dev(W), u.dev(S), u.dev(xh), kernel="gemv"))
        assert np.array_equal(y[0].view(np.uint16), B[:, k].view(np.uint16)), k
    # codes all 7 -> zero (the decode kernel folds the zero point into a per-group
    # constant, so this is zero up to fp32 rounding of that constant, not bit-exact)
    W7 = np.full((N, K // 8), 0x77777777, np.uint32)
    assert np.abs(u.host(ops.q4g32_linear(u.dev(W7), u.dev(S), u.dev(x), kernel="gemv"))).max() <= 1e-3
    # leading batch dims are flattened like the reference's [b, 1, K] activations
    x3 = x.reshape(M, 1, K)
    y3 = ops.q4g32_linear(u.dev(W), u.dev(S), u.dev(x3), kernel="gemv")
    assert tuple(y3.shape) == (M, 1, N)


def test_argument_errors(ops, u, oracle):
    from relax_amd._lib import WqError

    x, W, S = oracle.make_q4g32_inputs(1, 8, 64, seed=0)
    with pytest.raises(ValueError):
        ops.q4g32_linear(u.dev(W), u.dev(S[:, :1].copy()), u.dev(x))
    with pytest.raises(ValueError):
        ops.q4g32_linear(u.dev(W), u.dev(S), u.dev(x[:, :32].copy()))
    # K not a multiple of the group size is rejected by the C layer
    import torch
    from relax_amd import _lib

    w = torch.zeros((4, 5), dtype=torch.int32, device="cuda")
    rc = _lib.lib().wq_q4g32_gemv(w.data_ptr(), w.data_ptr(), w.data_ptr(), 0, 0, w.data_ptr(), 1, 4, 40, 0)
    assert rc != 0 and b"multiple" in _lib.lib().wq_last_error()
    with pytest.raises(WqError):
        _lib.check(rc, "gemv")


GEMM_SMALL = [  # (M, N, K) edge shapes: ragged M/N, odd number of groups
    (16, 64, 64), (33, 100, 96), (77, 300, 352), (128, 256, 4096), (300, 520, 1024), (64, 4096, 11008),
]


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 11, 12, 13, 14, 17, 18])
@pytest.mark.parametrize("M,N,K", GEMM_SMALL)
def test_gemm_small_vs_oracle(ops, u, oracle, cfg, M, N, K):
    from relax_amd import _lib

    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=cfg + M + N + K)
    print(f"gemm cfg={cfg} M={M} N={N} K={K}", flush=True)
    _lib.lib().wq_debug_set_gemm_config(cfg)
    try:
        got = u.host(ops.q4g32_linear(u.dev(W), u.dev(S), u.dev(x), kernel="gemm"))
    finally:
        _lib.lib().wq_debug_set_gemm_config(0)
    ref = oracle.q4g32_linear(W, S, x, nthreads=8)
    u.assert_close(got, ref, f"gemm cfg{cfg} {M}x{N}x{K}")


@pytest.mark.parametrize("N,K", [(11008, 4096), (4096, 11008)])
def test_gemm_prefill_full_size_sampled_rows(ops, u, oracle, N, K):
    """M=2048 at the real prefill shapes; the oracle checks a sample of output rows
    (rows of y are independent, so this is exact parity for the sampled rows),
    linearity checks the rest."""
    M = 2048
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=N)
    print(f"gemm prefill M={M} N={N} K={K}", flush=True)
    dW, dS, dx = u.dev(W), u.dev(S), u.dev(x)
    y = ops.q4g32_linear(dW, dS, dx)
    got = u.host(y)
    rows = np.array([0, 1, 31, 32, 255, 256, 1000, 1023, 1024, 2047])
    ref = oracle.q4g32_linear(W, S, x[rows], nthreads=8)
    u.assert_close(got[rows], ref, f"prefill {N}x{K}")
    # every row agrees with the decode kernel's result for that row (independent kernel)
    import torch

    pick = torch.arange(0, M, 61, device="cuda")
    yv = ops.q4g32_linear(dW, dS, dx[pick].contiguous(), kernel="gemv")
    u.assert_close(got[::61], u.host(yv), "gemm vs gemv")
    # scaling x by 2 scales y by exactly 2 (fp32 accumulation is scale invariant)
    # (outputs that are subnormal in fp16 round differently and are left out)
    y2 = ops.q4g32_linear(dW, dS, (dx * 2).contiguous())
    normal = y.abs() >= 2.0 ** -13
    assert torch.equal(y2[normal], (y * 2)[normal])


def test_gemm_epilogue(ops, u, oracle):
    M, N, K = 130, 200, 512
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=9)
    rng = np.random.default_rng(6)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    got = u.host(ops.q4g32_linear(u.dev(W), u.dev(S), u.dev(x), bias=u.dev(bias), residual=u.dev(res), kernel="gemm"))
    u.assert_close(got, oracle.q4g32_linear(W, S, x, bias=bias, residual=res, nthreads=8), "gemm epilogue")


SMALL_BATCH = [  # (M, N, K): ragged M and N, K/64 not a multiple of the wavefronts that split K
    (2, 64, 64), (5, 100, 192), (8, 4096, 4096), (16, 1001, 320), (17, 12288, 4096),
    (32, 4096, 11008), (33, 520, 1024), (64, 22016, 4096), (9, 31, 128),
    (3, 12288, 4096), (16, 4112, 8192), (12, 5000, 5184), (7, 16, 8192),
]


@pytest.mark.parametrize("nw,waves,stages", [(1, 0, 2), (2, 0, 3), (4, 0, 5), (1, 0, 3), (2, 0, 2), (4, 0, 4), (8, 0, 3), (8, 0, 2), (0, 0, 0),
                                             (0, 1, 0), (0, 2, 0)])
@pytest.mark.parametrize("M,N,K", SMALL_BATCH)
def test_small_batch_vs_oracle(ops, u, oracle, nw, waves, stages, M, N, K):
    """the matrix-core kernels for 2 <= M <= 64, in each of their work splits (0 = automatic; waves 1: the
    ring kernel, 2: activations in registers where M <= 16 and K <= 8192)."""
    from relax_amd import _lib

    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=nw + M + N + K)
    print(f"small batch nw={nw} waves={waves} stages={stages} M={M} N={N} K={K}", flush=True)
    _lib.lib().wq_debug_set_skinny_config(nw, stages, waves)
    try:
        got = u.host(ops.q4g32_linear(u.dev(W), u.dev(S), u.dev(x), kernel="small_batch"))
    finally:
        _lib.lib().wq_debug_set_skinny_config(0, 0, 0)
    ref = oracle.q4g32_linear(W, S, x, nthreads=8)
    u.assert_close(got, ref, f"small batch nw{nw} waves{waves} {M}x{N}x{K}")


@pytest.mark.parametrize("M", [1, 2, 4, 5, 8])
def test_low_batch_fixture_shape(ops, u, oracle, M):
    """The shape of the reference's low-batch fixture (tests/python/dlight/test_gpu_low_batch_gemv.py:29-34:
    N = 4096, K = 28672, a dynamic batch) at full size: the automatic dispatch and every kernel that serves it."""
    N, K = 4096, 28672
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=M + 77)
    print(f"low-batch fixture shape M={M}", flush=True)
    ref = oracle.q4g32_linear(W, S, x, nthreads=8)
    dW, dS, dx = u.dev(W), u.dev(S), u.dev(x)
    u.assert_close(u.host(ops.q4g32_linear(dW, dS, dx)), ref, f"automatic {M}x{N}x{K}")
    u.assert_close(u.host(ops.q4g32_linear(dW, dS, dx, kernel="gemv")), ref, f"gemv {M}x{N}x{K}")
    if M >= 2:
        u.assert_close(u.host(ops.q4g32_linear(dW, dS, dx, kernel="small_batch")), ref, f"small batch {M}x{N}x{K}")
    u.assert_close(u.host(ops.q4g32_linear(dW, dS, dx, kernel="gemm")), ref, f"gemm {M}x{N}x{K}")


@pytest.mark.parametrize("M", [8, 32])
@pytest.mark.parametrize("N,K", [(12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008)])
def test_llama7b_shapes_at_decode_batches(ops, u, oracle, M, N, K):
    """The four Llama-2-7B linears at the batch sizes of the 32-layer stack, at full size: the
    small-batch kernel selected explicitly and whatever the automatic dispatch picks."""
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=M + N + K)
    print(f"llama shape M={M} N={N} K={K}", flush=True)
    ref = oracle.q4g32_linear(W, S, x, nthreads=8)
    dW, dS, dx = u.dev(W), u.dev(S), u.dev(x)
    u.assert_close(u.host(ops.q4g32_linear(dW, dS, dx, kernel="small_batch")), ref, f"small batch {M}x{N}x{K}")
    u.assert_close(u.host(ops.q4g32_linear(dW, dS, dx)), ref, f"automatic {M}x{N}x{K}")


def test_small_batch_epilogue_and_dispatch(ops, u, oracle):
    M, N, K = 24, 200, 512
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=19)
    rng = np.random.default_rng(8)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    dW, dS, dx = u.dev(W), u.dev(S), u.dev(x)
    got = u.host(ops.q4g32_linear(dW, dS, dx, bias=u.dev(bias), residual=u.dev(res), kernel="small_batch"))
    u.assert_close(got, oracle.q4g32_linear(W, S, x, bias=bias, residual=res, nthreads=8), "small batch epilogue")
    # the automatic choice at this M is this kernel: identical bits
    auto = u.host(ops.q4g32_linear(dW, dS, dx, bias=u.dev(bias), residual=u.dev(res)))
    assert np.array_equal(auto.view(np.uint16), got.view(np.uint16))
    # K % 64 != 0 is outside this kernel and is refused by it, but served by the automatic choice
    from relax_amd._lib import WqError

    x2, W2, S2 = oracle.make_q4g32_inputs(12, 40, 96, seed=3)
    with pytest.raises(WqError):
        ops.q4g32_linear(u.dev(W2), u.dev(S2), u.dev(x2), kernel="small_batch")
    u.assert_close(u.host(ops.q4g32_linear(u.dev(W2), u.dev(S2), u.dev(x2))),
                   oracle.q4g32_linear(W2, S2, x2), "K=96 fallback")


def test_two_pass_small_batch_for_mid_m(ops, u, oracle):
    """65 <= M <= 128 on a small matrix runs as two passes of the small-batch kernel."""
    M, N, K = 100, 264, 512
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=23)
    rng = np.random.default_rng(9)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    got = u.host(ops.q4g32_linear(u.dev(W), u.dev(S), u.dev(x), bias=u.dev(bias), residual=u.dev(res)))
    u.assert_close(got, oracle.q4g32_linear(W, S, x, bias=bias, residual=res, nthreads=8), "two-pass small batch")
    got = u.host(ops.q4g32_linear(u.dev(W), u.dev(S), u.dev(x)))
    u.assert_close(got, oracle.q4g32_linear(W, S, x, nthreads=8), "two-pass small batch, plain")


def test_gemm_row_wise_and_element_wise_epilogues_agree(ops, u, oracle):
    """The GEMM stores 16 bytes per lane when N % 8 == 0 and y / residual are 16-byte aligned, single
    elements otherwise: both paths, same numbers."""
    import torch

    M, N, K = 300, 520, 1024
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=31)
    rng = np.random.default_rng(10)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    ref = oracle.q4g32_linear(W, S, x, bias=bias, residual=res, nthreads=8)
    dW, dS, dx, db = u.dev(W), u.dev(S), u.dev(x), u.dev(bias)
    aligned = ops.q4g32_linear(dW, dS, dx, bias=db, residual=u.dev(res), kernel="gemm")
    u.assert_close(u.host(aligned), ref, "aligned")
    # y and residual two bytes off a 16-byte boundary
    ybuf = torch.zeros(M * N + 8, dtype=torch.float16, device="cuda")
    rbuf = torch.zeros(M * N + 8, dtype=torch.float16, device="cuda")
    rbuf[1:1 + M * N] = u.dev(res).reshape(-1)
    y = ybuf[1:1 + M * N].view(M, N)
    ops.q4g32_linear(dW, dS, dx, bias=db, residual=rbuf[1:1 + M * N].view(M, N), out=y, kernel="gemm")
    assert torch.equal(y, aligned)
    assert float(ybuf[0]) == 0.0 and float(ybuf[M * N + 1]) == 0.0  # nothing written outside


@pytest.mark.parametrize("N,K", [(1, 32), (70, 96), (4096, 4096), (1000, 11008)])
def test_kn_layout_conversion_bit_exact_and_linear(ops, u, oracle, N, K):
    """K-major checkpoints are transposed once on the device; the result is the NK form bit for bit and the
    linear layer on it agrees with the K-major oracle."""
    rng = np.random.default_rng(N + K)
    W_kn = rng.integers(0, 2**32, size=(K // 8, N), dtype=np.uint64).astype(np.uint32)
    S_kn = rng.uniform(0.005, 0.02, size=(K // 32, N)).astype(np.float16)
    W, S = ops.q4g32_kn_to_nk(u.dev(W_kn), u.dev(S_kn))
    assert np.array_equal(u.host(W).view(np.uint32), np.ascontiguousarray(W_kn.T))
    assert np.array_equal(u.host(S).view(np.uint16), np.ascontiguousarray(S_kn.T).view(np.uint16))
    if N * K <= 4096 * 4096:
        x = rng.standard_normal((3, K)).astype(np.float16)
        got = u.host(ops.q4g32_linear(W, S, u.dev(x)))
        u.assert_close(got, oracle.q4g32_kn_linear(W_kn, S_kn, x), f"kn linear {N}x{K}")
