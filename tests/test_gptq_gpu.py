"""GPU parity of the AutoGPTQ entry points against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from tests.test_gptq_oracle import _pack_kn, _pack_zeros

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


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


def _ref_linear(oracle, qw, qz, s, g_idx, x, bias=None, residual=None):
    """fp32-accumulated oracle over the bit-exact dequantized weight (the pinned [N, K] matmul)."""
    B = oracle.gptq_dequant(qw, qz, s, g_idx)
    return oracle.nt_matmul_f32acc(np.ascontiguousarray(B.T), x, bias, residual, nthreads=8)


def test_dequantize_exhaustive_bit_exact(ops, u, oracle):
    """16 codes x 16 zero points x all 65536 scale bit patterns."""
    K, N, G = 256, 65536, 16
    k = np.arange(K)
    codes = np.broadcast_to((k // 16).astype(np.uint8)[:, None], (K, N))
    zeros = np.broadcast_to(np.arange(G, dtype=np.uint8)[:, None], (G, N))
    scales = np.broadcast_to(np.arange(N, dtype=np.uint32).astype(np.uint16).view(np.float16), (G, N)).copy()
    g_idx = (k % 16).astype(np.int32)
    qw, qz = _pack_kn(codes), _pack_zeros(zeros)
    got = u.host(ops.gptq_dequantize(u.dev(qw), u.dev(qz), u.dev(scales), u.dev(g_idx)))
    want = oracle.gptq_dequant(qw, qz, scales, g_idx)
    nan = np.isnan(want)
    assert np.array_equal(_bits(got)[~nan], _bits(want)[~nan])
    assert np.all(np.isnan(got[nan]))


@pytest.mark.parametrize("K,N,gs,mode", [(64, 8, 32, "trivial"), (256, 72, 64, "act_order"), (4096, 4096, 128, "act_order"),
                                         (1024, 328, 128, "ragged_groups"), (11008, 512, 128, "trivial")])
def test_dequantize_shapes(ops, u, oracle, K, N, gs, mode):
    _, qw, qz, s, g_idx = oracle.make_gptq_inputs(1, N, K, gs, seed=K + N, act_order=(mode == "act_order"))
    if mode == "ragged_groups":  # any assignment is a valid input of the decode
        g_idx = np.random.default_rng(1).integers(0, K // gs, size=K).astype(np.int32)
    got = u.host(ops.gptq_dequantize(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx)))
    assert np.array_equal(_bits(got), _bits(oracle.gptq_dequant(qw, qz, s, g_idx)))


def test_prepare_layout(ops, u, oracle):
    for K, N, gs, act in [(256, 72, 64, True), (4096, 1024, 128, True), (512, 64, 32, False), (192, 8, 96, True)]:
        _, qw, qz, s, g_idx = oracle.make_gptq_inputs(1, N, K, gs, seed=7, act_order=act)
        w = ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
        order = np.argsort(g_idx, kind="stable")
        if act:
            assert np.array_equal(u.host(w.perm), order.astype(np.int32))
        else:
            assert w.perm is None
        codes = ((qw[np.arange(K) // 8, :] >> (4 * (np.arange(K) % 8)).astype(np.uint32)[:, None]) & 15).astype(np.uint8)
        want_w = _pack_kn(codes[order]).T  # [N, K/8]
        assert np.array_equal(u.host(w.W_nk).view(np.uint32), want_w), (K, N)
        n = np.arange(N)
        zeros = (qz[:, n // 8] >> (4 * (n % 8)).astype(np.uint32)[None, :]) & 15  # [G, N]
        sz = u.host(w.SZ)
        assert np.array_equal(_bits(sz[:, :, 0]), _bits(s.T))
        assert np.array_equal(sz[:, :, 1], (zeros.T + 1).astype(np.float16))


def test_prepare_rejects_unequal_groups(ops, u, oracle):
    from relax_amd._lib import WqError

    _, qw, qz, s, g_idx = oracle.make_gptq_inputs(1, 64, 256, 64, seed=1)
    bad = g_idx.copy()
    bad[3] = 2  # group 0 loses a row, group 2 gains one
    with pytest.raises(WqError, match="exactly K/G"):
        ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(bad))
    bad = g_idx.copy()
    bad[100] = 99  # outside [0, G)
    with pytest.raises(WqError, match="exactly K/G"):
        ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(bad))
    with pytest.raises(WqError, match="multiple of 32"):
        ops.gptq_prepare(u.dev(qw), u.dev(qz[:1].repeat(16, 0)), u.dev(s[:1].repeat(16, 0)), u.dev(g_idx))


LINEAR_CASES = [  # (M, N, K, group size, act_order)
    (1, 4096, 4096, 128, False),   # the shape of the reference's test
    (1, 4096, 4096, 128, True),
    (1, 12288, 4096, 128, True),
    (1, 4096, 11008, 128, True),
    (2, 4096, 4096, 64, True),
    (2, 520, 11008, 128, True),    # two long rows: the small-batch kernel
    (2, 72, 8224, 32, False),      # two long rows, K not a multiple of 64: the streaming kernel
    (3, 520, 1024, 32, True),
    (4, 1000, 2048, 1024, False),
    (5, 264, 4096, 4096, True),    # one group
    (8, 2048, 4096, 128, True),
    (7, 72, 96, 96, True),         # K not a multiple of 64: streaming kernel repeated
    (16, 512, 1024, 128, True),    # small-batch kernel
    (33, 1032, 4096, 128, True),
    (64, 4096, 4096, 128, False),
    (64, 264, 384, 96, True),      # three 32-code groups per scale group
    (65, 512, 1024, 128, True),    # two passes of the small-batch kernel up to 128 rows of a matrix with N <= 8192
    (128, 264, 2048, 64, True),
    (100, 8200, 256, 128, False),  # wider: the MFMA GEMM
    (16, 512, 1024, 128, False),
    (40, 264, 1152, 192, True),
    (130, 1096, 2048, 64, True),
    (512, 2048, 4096, 128, True),
    (700, 1024, 1024, 256, False),
    (20, 136, 288, 96, True),      # large M, group size not a multiple of 64: streaming kernel repeated
    (1, 72, 32768, 128, True),     # the longest supported row: 64 KB of activations staged / gathered through LDS
    (3, 72, 32768, 256, True),
    (70, 136, 32768, 2048, True),
]


@pytest.mark.parametrize("M,N,K,gs,act", LINEAR_CASES)
def test_linear_matches_oracle(ops, u, oracle, M, N, K, gs, act):
    x, qw, qz, s, g_idx = oracle.make_gptq_inputs(M, N, K, gs, seed=M + N + K + gs, act_order=act)
    rng = np.random.default_rng(9)
    res = rng.standard_normal((M, N)).astype(np.float16)
    w = ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
    assert (w.perm is not None) == (not np.array_equal(np.argsort(g_idx, kind="stable"), np.arange(K)))
    got = u.host(ops.gptq_linear(w, u.dev(x), residual=u.dev(res)))
    u.assert_close(got, _ref_linear(oracle, qw, qz, s, g_idx, x, None, res), f"gptq {M}x{N}x{K} gs={gs}")


@pytest.mark.parametrize("M", [1, 4, 48, 400])
def test_linear_bias_and_plain(ops, u, oracle, M):
    N, K, gs = 776, 2048, 128
    x, qw, qz, s, g_idx = oracle.make_gptq_inputs(M, N, K, gs, seed=M, act_order=True)
    bias = np.random.default_rng(2).standard_normal(N).astype(np.float16)
    w = ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
    u.assert_close(u.host(ops.gptq_linear(w, u.dev(x))), _ref_linear(oracle, qw, qz, s, g_idx, x), "plain")
    u.assert_close(u.host(ops.gptq_linear(w, u.dev(x), bias=u.dev(bias))),
                   _ref_linear(oracle, qw, qz, s, g_idx, x, bias), "bias")


@pytest.mark.parametrize("M", [1, 8, 64, 100])
def test_one_hot_rows_reproduce_the_dequantized_weight(ops, u, oracle, M):
    """x = e_k selects row k of the weight: exact in the small-batch kernel and the GEMM (they multiply
    the reference's fp16 weights), one fp16 ulp in the streaming kernel (it applies the scale after the sum)."""
    N, K, gs = 256, 512, 128
    _, qw, qz, s, g_idx = oracle.make_gptq_inputs(1, N, K, gs, seed=11, act_order=True)
    B = oracle.gptq_dequant(qw, qz, s, g_idx)
    ks = np.random.default_rng(3).integers(0, K, size=M)
    x = np.zeros((M, K), np.float16)
    x[np.arange(M), ks] = 1
    w = ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
    got = u.host(ops.gptq_linear(w, u.dev(x)))
    if M > 2:
        assert np.array_equal(_bits(got), _bits(B[ks]))
    else:
        assert np.max(np.abs(got.astype(np.float64) - B[ks].astype(np.float64))) <= 2.0**-10 * np.max(np.abs(B))


def test_linear_argument_errors(ops, u, oracle):
    from relax_amd import _lib
    from relax_amd._lib import WqError
    import torch

    x, qw, qz, s, g_idx = oracle.make_gptq_inputs(16, 64, 256, 64, seed=1, act_order=True)
    w = ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
    assert ops.gptq_workspace_bytes(16, 256, True) == 16 * 256 * 2
    assert ops.gptq_workspace_bytes(16, 256, False) == 0 and ops.gptq_workspace_bytes(1, 256, True) == 512
    with pytest.raises(WqError, match="workspace"):
        ops.gptq_linear(w, u.dev(x), workspace=torch.empty(16, dtype=torch.uint8, device="cuda"))
    with pytest.raises(ValueError):
        ops.gptq_linear(w, u.dev(x[:, :128]))
    assert ops.gptq_linear(w, u.dev(x[:0])).shape == (0, 64)
    y = torch.empty(16, 64, dtype=torch.float16, device="cuda")
    rc = _lib.lib().wq_gptq_linear(w.W_nk.data_ptr(), w.SZ.data_ptr(), 0, u.dev(x).data_ptr(), 0, 0, y.data_ptr(),
                                   16, 64, 256, 3, 0, 0, 0)
    assert rc != 0 and b"groups" in _lib.lib().wq_last_error()


# ---- any g_idx: groups of unequal size (wq_gptq_prepare_padded / wq_gptq_linear_padded) ----
def _unequal_g_idx(K, G, seed, kind):
    rng = np.random.default_rng(seed)
    if kind == "random":        # every row picks a group at random: sizes differ, some may be empty
        return rng.integers(0, G, size=K).astype(np.int32)
    if kind == "runs":          # contiguous runs of different lengths, not multiples of 32
        cuts = np.sort(rng.choice(np.arange(1, K), size=G - 1, replace=False))
        return np.repeat(np.arange(G), np.diff(np.concatenate([[0], cuts, [K]]))).astype(np.int32)
    if kind == "one_big":       # one group holds nearly everything, one is empty
        g = np.zeros(K, np.int32)
        g[:5] = 1
        g[-3:] = G - 1
        return g
    raise ValueError(kind)


@pytest.mark.parametrize("kind", ["random", "runs", "one_big"])
@pytest.mark.parametrize("M,N,K,G", [(1, 256, 1024, 8), (2, 64, 4096, 32), (5, 520, 2048, 16), (40, 128, 1024, 4), (200, 256, 512, 4)])
def test_unequal_groups_linear_matches_oracle(ops, u, oracle, kind, M, N, K, G):
    x, qw, qz, s, _ = oracle.make_gptq_inputs(M, N, K, K // G, seed=M + N + K)
    g_idx = _unequal_g_idx(K, G, seed=K + G, kind=kind)
    sizes = np.bincount(g_idx, minlength=G)
    assert len(set(sizes.tolist())) > 1  # really unequal
    w = ops.gptq_prepare_padded(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
    assert w.K_padded % 64 == 0 and w.K_padded >= int(((sizes + 31) // 32 * 32).sum())
    # layout: position k' holds row perm[k'] of the checkpoint, rows of a group in ascending k, padding = -1
    perm = u.host(w.perm)
    real = perm[perm >= 0]
    assert np.array_equal(np.sort(real), np.arange(K))
    assert np.array_equal(g_idx[real], np.sort(g_idx, kind="stable")) and np.array_equal(real, np.argsort(g_idx, kind="stable"))
    rng = np.random.default_rng(3)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    got = u.host(ops.gptq_linear(w, u.dev(x), bias=u.dev(bias), residual=u.dev(res)))
    u.assert_close(got, _ref_linear(oracle, qw, qz, s, g_idx, x, bias, res), f"gptq unequal {kind} {M}x{N}x{K} G={G}")


def test_unequal_groups_one_hot_rows_reproduce_the_dequantized_weight(ops, u, oracle):
    N, K, G = 64, 512, 8
    _, qw, qz, s, _ = oracle.make_gptq_inputs(1, N, K, K // G, seed=5)
    g_idx = _unequal_g_idx(K, G, seed=9, kind="random")
    B = oracle.gptq_dequant(qw, qz, s, g_idx)  # [K, N]
    rows = [0, 1, 31, 32, 100, 255, 256, 511]
    x = np.zeros((len(rows), K), np.float16)
    for m, k in enumerate(rows):
        x[m, k] = 1
    w = ops.gptq_prepare_padded(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
    got = u.host(ops.gptq_linear(w, u.dev(x)))
    for m, k in enumerate(rows):
        assert np.array_equal(_bits(got[m]), _bits(B[k])), (m, k)


def test_prepare_padded_errors(ops, u, oracle):
    from relax_amd._lib import WqError

    _, qw, qz, s, g_idx = oracle.make_gptq_inputs(1, 64, 256, 64, seed=1)
    bad = g_idx.copy()
    bad[3] = 4  # outside [0, G)
    with pytest.raises(WqError, match="outside"):
        ops.gptq_prepare_padded(u.dev(qw), u.dev(qz), u.dev(s), u.dev(bad))
