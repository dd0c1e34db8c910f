"""GPU parity of the format-B (fp16 x int8/int4) path against the CPU oracle, through the C ABI."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden", "ft_layout_vectors.npz")


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


@pytest.mark.parametrize("case", ["int8_64x64", "int8_128x192", "int8_256x64", "int4_64x64", "int4_128x192", "int4_256x128"])
def test_device_preprocess_matches_golden(ops, u, case):
    g = np.load(GOLD)
    a, want = g[case + "_in"], g[case + "_out"]
    got = u.host(ops.ft_preprocess_weight(u.dev(a), 80, case.startswith("int4")))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("is_int4", [False, True])
def test_device_preprocess_large_and_experts(ops, u, oracle, is_int4):
    rng = np.random.default_rng(17)
    a = rng.integers(-128, 128, size=(2, 512, 320)).astype(np.int8)
    got = u.host(ops.ft_preprocess_weight(u.dev(a), 80, is_int4))
    assert np.array_equal(got, oracle.ft_preprocess(a, is_int4, 80))
    a = rng.integers(-128, 128, size=(8192, 1024 if not is_int4 else 512)).astype(np.int8)
    got = u.host(ops.ft_preprocess_weight(u.dev(a), 80, is_int4))
    assert np.array_equal(got, oracle.ft_preprocess(a, is_int4, 80))


@pytest.mark.parametrize("nbit", [8, 4])
def test_dequant_exhaustive_bit_exact(ops, u, oracle, nbit):
    """every code x every fp16 scale bit pattern, through preprocess + device dequantize."""
    all_s = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16)
    ncode = 256 if nbit == 8 else 16
    lo = -128 if nbit == 8 else -8
    K = 256  # codes repeat down the rows; K must be a multiple of 64
    codes = (np.arange(K) % ncode + lo).astype(np.int64)
    for start in range(0, 65536, 16384):
        s = all_s[start:start + 16384]
        N = s.size
        q = np.repeat(codes[:, None], N, axis=1)
        if nbit == 8:
            A = q.astype(np.int8)
        else:
            A = ((q[:, 0::2] & 15) | ((q[:, 1::2] & 15) << 4)).astype(np.uint8).view(np.int8)
        want = oracle.intb_dequant(A, s, nbit)
        P = ops.ft_preprocess_weight(u.dev(A), 80, nbit == 4)
        got = u.host(ops.intb_dequantize(P, u.dev(s), nbit))
        nan = np.isnan(want)
        assert np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])
        assert np.all(np.isnan(got[nan]))


@pytest.mark.parametrize("nbit", [8, 4])
def test_dequant_finegrained(ops, u, oracle, nbit):
    _, A, s = oracle.make_intb_inputs(1, 128, 256, nbit, seed=4, group_size=64)
    P = ops.ft_preprocess_weight(u.dev(A), 80, nbit == 4)
    got = u.host(ops.intb_dequantize(P, u.dev(s), nbit, group_size=64))
    assert np.array_equal(got.view(np.uint16), oracle.intb_dequant(A, s, nbit, 64).view(np.uint16))


def _run(ops, u, oracle, M, N, K, nbit, seed, group_size=-1, **ep):
    x, A, s = oracle.make_intb_inputs(M, N, K, nbit, seed=seed, group_size=group_size)
    rng = np.random.default_rng(seed + 1)
    kw, okw = {}, {}
    if ep.get("bias") == "row":
        b = rng.standard_normal(N).astype(np.float16)
        kw["bias"], okw["bias"] = u.dev(b), b
    elif ep.get("bias") == "full":
        b = rng.standard_normal((M, N)).astype(np.float16)
        kw["bias"], okw["bias"], okw["bias_stride"] = u.dev(b), b, N
    if ep.get("residual"):
        r = rng.standard_normal((M, N)).astype(np.float16)
        kw["residual"], okw["residual"] = u.dev(r), r
        kw["binary_op"] = okw["binary_op"] = ep.get("binary_op", "plus")
        kw["unary_op"] = okw["unary_op"] = ep.get("unary_op", "identity")
    act = ep.get("activation", "identity")
    P = ops.ft_preprocess_weight(u.dev(A), 80, nbit == 4)
    got = u.host(ops.fpA_intB_gemm(u.dev(x), P, u.dev(s), weight_nbit=nbit, activation=act, group_size=group_size, **kw))
    ref = oracle.intb_linear(x, A, s, nbit, group_size=group_size, activation=act, nthreads=8, **okw)
    u.assert_close(got, ref, f"intb nbit={nbit} M={M} N={N} K={K} g={group_size} {ep}")


@pytest.mark.parametrize("nbit", [8, 4])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 16, 33, 128, 300])
def test_gemm_vs_oracle_shapes(ops, u, oracle, nbit, M):
    print(f"intb nbit={nbit} M={M}", flush=True)
    _run(ops, u, oracle, M, 256, 512, nbit, seed=M)
    _run(ops, u, oracle, M, 64, 64, nbit, seed=M + 50)
    _run(ops, u, oracle, M, 192, 4096, nbit, seed=M + 100)


@pytest.mark.parametrize("nbit", [8, 4])
@pytest.mark.parametrize("M", [1, 4, 64])
def test_gemm_finegrained(ops, u, oracle, nbit, M):
    _run(ops, u, oracle, M, 128, 512, nbit, seed=M + 7, group_size=64)


@pytest.mark.parametrize("nbit", [8, 4])
@pytest.mark.parametrize("M", [2, 48, 100, 130])
@pytest.mark.parametrize("ep", [
    dict(bias="row"), dict(bias="full"), dict(bias="row", activation="relu"), dict(bias="row", activation="silu"),
    dict(bias="row", activation="gelu"), dict(residual=True), dict(bias="row", residual=True, binary_op="plus"),
    dict(bias="row", residual=True, binary_op="multiply", unary_op="relu"),
    dict(bias="row", activation="silu", residual=True, binary_op="plus", unary_op="relu"),
], ids=lambda d: "-".join(f"{k}={v}" for k, v in d.items()))
def test_gemm_epilogues(ops, u, oracle, nbit, M, ep):
    _run(ops, u, oracle, M, 128, 256, nbit, seed=M + 3, **ep)


@pytest.mark.parametrize("nw,stages,waves", [(1, 2, 0), (2, 3, 0), (4, 4, 0), (8, 3, 0), (0, 0, 0), (0, 0, 1), (0, 0, 2)])
@pytest.mark.parametrize("nbit", [8, 4])
@pytest.mark.parametrize("group_size", [-1, 64])
def test_small_batch_work_splits(ops, u, oracle, nbit, group_size, nw, stages, waves):
    """3 <= M <= 64 runs the matrix-core streaming kernel; every work split of it, ragged M,
    K not a multiple of its 128-k step."""
    from relax_amd import _lib

    _lib.lib().wq_debug_set_skinny_config(nw, stages, waves)
    try:
        for M, N, K in [(3, 64, 64), (8, 320, 448), (9, 128, 4096), (16, 320, 448), (24, 64, 1024),
                        (32, 2048, 512), (40, 320, 448), (64, 192, 2112), (16, 4288, 8192), (5, 8192, 5184)]:
            print(f"intb small batch nbit={nbit} g={group_size} nw={nw} waves={waves} M={M} N={N} K={K}", flush=True)
            _run(ops, u, oracle, M, N, K, nbit, seed=M + nw, group_size=group_size)
    finally:
        _lib.lib().wq_debug_set_skinny_config(0, 0, 0)


@pytest.mark.parametrize("rows", [0, 1, 2])
@pytest.mark.parametrize("nbit", [8, 4])
@pytest.mark.parametrize("group_size", [-1, 64])
def test_one_and_two_rows_on_either_kernel(ops, u, oracle, nbit, group_size, rows):
    """M <= 2: the automatic choice (the streaming kernel for wide matrices, the small-batch kernel for narrow
    ones, where whole columns per wavefront leave the machine short of wavefronts) and the streaming kernel asked
    for by the test hook, with one and two column groups per wavefront."""
    from relax_amd import _lib

    _lib.lib().wq_debug_set_gemv_config(rows, 0)
    try:
        for M, N, K in [(1, 64, 64), (2, 64, 128), (1, 320, 448), (2, 320, 4096), (1, 4096, 1024), (2, 4096, 1024),
                        (1, 16384, 256), (2, 16384, 256), (1, 1024, 11008)]:
            print(f"intb rows={rows} nbit={nbit} g={group_size} M={M} N={N} K={K}", flush=True)
            _run(ops, u, oracle, M, N, K, nbit, seed=M + N + rows, group_size=group_size, bias="row")
    finally:
        _lib.lib().wq_debug_set_gemv_config(0, 0)


@pytest.mark.parametrize("nbit", [8, 4])
def test_65_to_128_rows_in_two_small_batch_passes(ops, u, oracle, nbit):
    """65 .. 128 rows of a small matrix run as two passes of the small-batch kernel (64 rows, then the rest), wider
    ones as a tiled GEMM: both sides of the rule, with an epilogue that reads per-row operands."""
    for M, N, K, g in [(65, 4096, 256, -1), (128, 1024, 1024, 64), (96, 5120, 8192, -1), (97, 5120, 8192, -1),
                       (128, 4160, 512, 64)]:
        print(f"intb two passes nbit={nbit} M={M} N={N} K={K} g={g}", flush=True)
        _run(ops, u, oracle, M, N, K, nbit, seed=M + N, group_size=g, bias="full")
        _run(ops, u, oracle, M, N, K, nbit, seed=M + N + 1, group_size=g, bias="row", residual=True, binary_op="multiply")


@pytest.mark.parametrize("ways", [2, 4, 8])
@pytest.mark.parametrize("nbit", [8, 4])
@pytest.mark.parametrize("group_size", [-1, 64])
def test_streaming_kernel_with_k_split(ops, u, oracle, nbit, group_size, ways):
    """2, 4 or 8 wavefronts share a column group and split K (what one row of a narrow int4 matrix gets by itself):
    K shorter than the split, K that does not divide by it, one and two rows, ragged last workgroup."""
    from relax_amd import _lib

    L = _lib.lib()
    L.wq_debug_set_intb_gemv_k_split(ways)
    L.wq_debug_set_gemv_config(2, 0)
    try:
        for M, N, K in [(1, 64, 64), (2, 64, 128), (1, 320, 448), (1, 4096, 1024), (2, 1024, 4096), (1, 8192, 2112),
                        (1, 5120, 13824)]:
            print(f"intb k split {ways} nbit={nbit} g={group_size} M={M} N={N} K={K}", flush=True)
            _run(ops, u, oracle, M, N, K, nbit, seed=M + N + ways, group_size=group_size, bias="row", residual=True)
        L.wq_debug_set_gemv_config(1, 0)
        _run(ops, u, oracle, 1, 1024, 4096, nbit, seed=ways, group_size=group_size)
    finally:
        L.wq_debug_set_gemv_config(0, 0)
        L.wq_debug_set_intb_gemv_k_split(0)


@pytest.mark.parametrize("nbit", [8, 4])
def test_one_row_of_a_narrow_matrix(ops, u, oracle, nbit):
    """The automatic choice at M = 1 over widths on both sides of every threshold (int4: the streaming kernel with
    its own split of K; int8: the small-batch kernel below 8 wavefronts per CU)."""
    for N, K in [(1024, 4096), (4096, 4096), (5120, 13824), (8192, 8192), (12288, 4096), (22016, 4096)]:
        for g in (-1, 64):
            print(f"intb narrow nbit={nbit} g={g} N={N} K={K}", flush=True)
            _run(ops, u, oracle, 1, N, K, nbit, seed=N + K, group_size=g)


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 11, 12, 17, 18])
@pytest.mark.parametrize("nbit", [8, 4])
def test_gemm_tile_configurations(ops, u, oracle, nbit, cfg):
    """every tile shape of the register-staged (1-4) and the LDS-staged (11, 12, 17, 18) kernel, ragged M,
    N smaller than a tile, with and without the row-wise epilogue (bias stride not a multiple of 8)."""
    from relax_amd import _lib

    _lib.lib().wq_debug_set_gemm_config(cfg)
    try:
        for M, N, K in [(70, 64, 64), (130, 320, 448), (257, 192, 1024), (300, 576, 512)]:
            print(f"intb cfg={cfg} nbit={nbit} M={M} N={N} K={K}", flush=True)
            _run(ops, u, oracle, M, N, K, nbit, seed=M + cfg)
        _run(ops, u, oracle, 100, 128, 256, nbit, seed=cfg, bias="row", activation="gelu", residual=True,
             binary_op="multiply", unary_op="relu")
        _run(ops, u, oracle, 100, 128, 256, nbit, seed=cfg + 1, bias="full")
        # fine-grained (group-64) scales through the same tiles
        for M, N, K in [(70, 64, 64), (130, 320, 448), (300, 576, 512)]:
            print(f"intb cfg={cfg} nbit={nbit} g=64 M={M} N={N} K={K}", flush=True)
            _run(ops, u, oracle, M, N, K, nbit, seed=M + cfg + 1, group_size=64)
        _run(ops, u, oracle, 100, 128, 256, nbit, seed=cfg + 2, group_size=64, bias="row", activation="relu")
    finally:
        _lib.lib().wq_debug_set_gemm_config(0)


@pytest.mark.parametrize("M", [1, 16, 128, 256, 512])
def test_int8_full_size_sampled(ops, u, oracle, M):
    """K=8192, N=28672 int8 per-channel.  The oracle checks a sample of output columns
    (columns are independent given x), the one-hot test checks the layout end to end."""
    import torch

    K, N = 8192, 28672
    rng = np.random.default_rng(M)
    x = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
    dA = torch.randint(-127, 128, (K, N), dtype=torch.int8, device="cuda")
    s = rng.uniform(0.001, 0.01, size=N).astype(np.float16)
    print(f"int8 full size M={M}", flush=True)
    P = ops.ft_preprocess_weight(dA, 80, False)
    got = u.host(ops.fpA_intB_gemm(u.dev(x), P, u.dev(s), weight_nbit=8))
    cols = np.concatenate([np.arange(0, 64), np.arange(14000, 14064), np.arange(N - 64, N)])
    A_cols = u.host(dA[:, torch.from_numpy(cols).cuda()].contiguous())
    # rows from every row tile of the kernels that serve these M (128 x 128, 256 x 128 and 256 x 256 tiles by M)
    rows = np.unique(np.clip(np.array([0, 7, 8, 15, 31, 32, 63, 64, 127, 128, 129, 255, 256, 300, 383, 384, 511]), 0, M - 1))
    ref = oracle.intb_linear(x[rows], A_cols, s[cols], 8, nthreads=8)
    u.assert_close(got[rows][:, cols], ref, f"int8 full M={M}")
    if M > 2:
        # every 61st row against the streaming kernel (an independent kernel), all columns
        pick = np.arange(0, M, 61)
        for r in pick:
            yv = u.host(ops.fpA_intB_gemm(u.dev(x[r:r + 1]), P, u.dev(s), weight_nbit=8))
            u.assert_close(got[r:r + 1], yv, f"int8 full M={M} row {r} vs gemv")
    if M == 1:
        # the reordered layout of the whole matrix (224 MiB), bit for bit against the oracle
        want_P = oracle.ft_preprocess(u.host(dA), False, 80)
        assert np.array_equal(u.host(P), want_P)
        del want_P
        xh = np.zeros((1, K), np.float16)
        xh[0, 4321] = 1
        y = u.host(ops.fpA_intB_gemm(u.dev(xh), P, u.dev(s), weight_nbit=8))
        want = (u.host(dA[4321]).astype(np.float16) * s)
        assert np.array_equal(y[0].view(np.uint16), want.view(np.uint16))


def test_reference_fixture_chain(ops, u, oracle):
    """The reference's own small test case (tests/python/relax/test_codegen_cutlass.py:1559-1609):
    np.random.seed(0); x = randn(64,64); y = normal(0, 0.002, (128,64)); bias = randn(1,128);
    residual = randn(64,128); encode -> preprocess -> fused GEMM, compared with the UNQUANTIZED
    np.dot(x, y.T) + bias (+ residual) at the reference's rtol = atol = 1e-2."""
    np.random.seed(0)
    x = np.random.randn(64, 64).astype("float16")
    y = np.random.normal(0, 0.002, size=(128, 64)).astype("float16")
    bias = np.random.randn(1, 128).astype("float16")
    residual = np.random.randn(64, 128).astype("float16")
    for nbit, tol in ((4, 1e-2), (8, 1e-2)):
        w, s = oracle.intb_encode(y, nbit)
        P = ops.ft_preprocess_weight(u.dev(w), 80, nbit == 4)
        out = u.host(ops.fpA_intB_gemm(u.dev(x), P, u.dev(s), bias=u.dev(bias), weight_nbit=nbit))
        ref = np.dot(x, y.transpose()) + bias
        np.testing.assert_allclose(out, ref, rtol=tol, atol=tol)
        out = u.host(ops.fpA_intB_gemm(u.dev(x), P, u.dev(s), bias=u.dev(bias), residual=u.dev(residual),
                                       weight_nbit=nbit, binary_op="plus"))
        np.testing.assert_allclose(out, ref + residual, rtol=tol, atol=tol)


def test_argument_errors(ops, u, oracle):
    from relax_amd._lib import WqError

    x, A, s = oracle.make_intb_inputs(2, 64, 64, 8, seed=0)
    P = ops.ft_preprocess_weight(u.dev(A), 80, False)
    with pytest.raises(WqError, match="group_size"):
        ops.fpA_intB_gemm(u.dev(x), P, u.dev(np.tile(s, 2)), weight_nbit=8, group_size=32)
    with pytest.raises(ValueError):
        ops.fpA_intB_gemm(u.dev(x[:, :32].copy()), P, u.dev(s), weight_nbit=8)
    with pytest.raises(ValueError):
        ops.fpA_intB_gemm(u.dev(x), P, u.dev(s[:10].copy()), weight_nbit=8)


@pytest.mark.parametrize("nbit", [8, 4])
def test_grouped_gemv_with_scales_at_any_alignment(ops, u, oracle, nbit):
    """group-64 scales: the streaming kernel fetches them as 8- or 16-byte vectors when the buffer is
    16-byte aligned and one by one otherwise; both must give the same result."""
    import torch

    M, N, K = 2, 192, 512
    x, A, s = oracle.make_intb_inputs(M, N, K, nbit, seed=5, group_size=64)
    P = ops.ft_preprocess_weight(u.dev(A), 80, nbit == 4)
    ref = oracle.intb_linear(x, A, s, nbit, group_size=64)
    aligned = u.dev(s)
    backing = torch.empty(s.size + 2, dtype=torch.float16, device="cuda")
    shifted = backing[2:].view(s.shape)  # 4 bytes past a 16-byte boundary
    shifted.copy_(aligned)
    assert aligned.data_ptr() % 16 == 0 and shifted.data_ptr() % 16 == 4
    got_a = ops.fpA_intB_gemm(u.dev(x), P, aligned, weight_nbit=nbit, group_size=64)
    got_s = ops.fpA_intB_gemm(u.dev(x), P, shifted, weight_nbit=nbit, group_size=64)
    assert torch.equal(got_a, got_s)
    u.assert_close(u.host(got_a), ref, f"grouped gemv int{nbit}")
