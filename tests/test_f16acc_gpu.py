"""The decode GEMV with the reference's fp16 accumulation (tests/python/dlight/test_gpu_reduction.py:44-51,
test_gpu_gemv.py:199-206) against the CPU oracle, through the C ABI.

The reference fixes WHAT is rounded (every product and every partial sum, to fp16) but not the ORDER of the
sum: its schedules split the reduction over lanes.  Two checks follow from that:
  * bit-exact against a numpy model that applies the oracle's fp16 multiply and add in the kernel's order
    (per lane over its scale groups, two interleaved chains, then a tree over the 64 lanes);
  * against the oracle's sequential sum within the error bound of fp16 accumulation, stated below.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

EPS = 2.0 ** -11  # unit roundoff of fp16


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


def kernel_order_model(B: np.ndarray, x: np.ndarray) -> np.ndarray:
    """y[n] for one activation row: fp16 products and sums in the order the kernel adds them."""
    N, K = B.shape
    G = K // 32
    h = np.float16
    lanes = np.zeros((N, 64, 2), h)  # the two chains of a lane: elements j < 4 and j >= 4 of each word
    with np.errstate(over="ignore", invalid="ignore"):
        for g in range(G):
            lane = g % 64
            for c in range(4):
                for i in range(4):
                    for half in range(2):
                        k = g * 32 + c * 8 + i + 4 * half
                        p = (B[:, k] * x[k]).astype(h)
                        lanes[:, lane, half] = (lanes[:, lane, half] + p).astype(h)
        v = (lanes[:, :, 0] + lanes[:, :, 1]).astype(h)  # [N, 64]
        for sh in (1, 2, 4, 8):  # within rows of 16 lanes
            src = np.zeros_like(v)
            for row in range(4):
                src[:, row * 16 + sh:(row + 1) * 16] = v[:, row * 16:(row + 1) * 16 - sh]
            v = (v + src).astype(h)
        r = v[:, 15::16]  # the four row sums
        return ((r[:, 3] + r[:, 2]).astype(h) + (r[:, 1] + r[:, 0]).astype(h)).astype(h)


SHAPES = [(1, 8, 32), (1, 37, 64), (1, 64, 4096), (2, 129, 2048 + 32), (1, 256, 11008), (3, 5, 160),
          # the reference's low-batch fixture (test_gpu_low_batch_gemv.py:29-34: N = 4096, K = 28672, fp16 accumulation)
          (1, 4096, 28672), (5, 64, 28672),
          # several rows of x in one pass over the weights (4, 4 + 2 + 1, 4 + 4): every row as if alone
          (4, 300, 11008), (7, 37, 2048 + 32), (8, 64, 4096)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_f16acc_bit_exact_in_kernel_order(ops, u, oracle, M, N, K):
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=N + K)
    B = oracle.q4g32_dequant(W, S)
    got = u.host(ops.q4g32_gemv_f16acc(u.dev(W), u.dev(S), u.dev(x)))
    assert got.shape == (M, N)
    for m in range(M):
        want = kernel_order_model(B, x[m])
        assert np.array_equal(got[m].view(np.uint16), want.view(np.uint16)), (m, N, K)


@pytest.mark.parametrize("M,N,K", [(1, 64, 4096), (1, 300, 11008), (2, 4096, 4096)])
def test_f16acc_against_sequential_oracle_within_fp16_bound(ops, u, oracle, M, N, K):
    """|fl(sum) - sum| <= depth * eps * sum|x w| (first order) for any order whose longest chain of
    roundings is `depth` (product included): depth K + 1 for the oracle's sequential sum, 16 * ceil(K / 2048)
    + 8 for the kernel's tree.  Tolerance of the comparison: 1.1 x the sum of both bounds."""
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=5)
    B = oracle.q4g32_dequant(W, S)
    got = u.host(ops.q4g32_gemv_f16acc(u.dev(W), u.dev(S), u.dev(x))).astype(np.float64)
    rows = np.arange(0, N, max(1, N // 64))  # the sequential oracle is slow: a sample of rows
    seq = oracle.nt_matmul_f16acc(B[rows], x).astype(np.float64)
    exact = x.astype(np.float64) @ B[rows].astype(np.float64).T
    mag = np.abs(x).astype(np.float64) @ np.abs(B[rows]).astype(np.float64).T
    depth_kernel = 16 * -(-K // 2048) + 8
    assert np.all(np.abs(got[:, rows] - exact) <= 1.1 * depth_kernel * EPS * mag + 1e-7)
    assert np.all(np.abs(got[:, rows] - seq) <= 1.1 * (depth_kernel + K + 1) * EPS * mag + 1e-7)
    # and the tree is the more accurate of the two on average
    assert np.mean(np.abs(got[:, rows] - exact)) <= np.mean(np.abs(seq - exact))


def test_f16acc_differs_from_fp32_accumulation(ops, u, oracle):
    """The entry point really rounds the partial sums: on a long row its result differs from the fp32-accumulate
    kernel's in a good share of the outputs (both are within their own bounds of the exact value)."""
    x, W, S = oracle.make_q4g32_inputs(1, 512, 8192, seed=11)
    a = u.host(ops.q4g32_gemv_f16acc(u.dev(W), u.dev(S), u.dev(x)))
    b = u.host(ops.q4g32_linear(u.dev(W), u.dev(S), u.dev(x)))
    assert np.mean(a.view(np.uint16) != b.view(np.uint16)) > 0.25


def test_f16acc_edges_and_errors(ops, u):
    import torch

    from relax_amd._lib import WqError

    W = torch.zeros((0, 4), dtype=torch.int32, device="cuda")
    S = torch.zeros((0, 1), dtype=torch.float16, device="cuda")
    x = torch.zeros((1, 32), dtype=torch.float16, device="cuda")
    assert ops.q4g32_gemv_f16acc(W, S, x).shape == (1, 0)
    W = torch.zeros((4, 4), dtype=torch.int32, device="cuda")
    S = torch.zeros((4, 1), dtype=torch.float16, device="cuda")
    assert ops.q4g32_gemv_f16acc(W, S, x[:0]).shape == (0, 4)
    with pytest.raises(ValueError):
        ops.q4g32_gemv_f16acc(W, S, torch.zeros((1, 64), dtype=torch.float16, device="cuda"))
    with pytest.raises(WqError):  # x not 16-byte aligned
        xx = torch.zeros(40, dtype=torch.float16, device="cuda")[1:33].view(1, 32)
        ops.q4g32_gemv_f16acc(W, S, xx)
