"""Device quantizers against the CPU oracle (bit-exact codes and scales), and the whole on-device
preparation chain encode -> preprocess -> fused GEMM against the unquantized product, the way the
reference's own end-to-end tests check it (tests/python/relax/test_codegen_cutlass.py:1586-1611)."""
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


def _weights(N, K, seed):
    rng = np.random.default_rng(seed)
    w = (rng.normal(0, 0.02, size=(N, K)) * rng.uniform(0.05, 5, size=(N, 1))).astype(np.float16)
    w[1, : min(K, 64)] = 0          # an all-zero group / row prefix
    w[2, 3] = np.float16(60000.0)    # a huge outlier
    w[N - 1] = 0                     # an all-zero row: the 1e-4 floor
    return w


@pytest.mark.parametrize("nbit", [8, 4])
@pytest.mark.parametrize("N,K", [(64, 64), (128, 448), (320, 1024), (4096, 4096)])
def test_intb_encode_per_channel_bit_exact(ops, u, oracle, nbit, N, K):
    Wf = _weights(N, K, seed=N + K + nbit)
    w, s = ops.intb_encode(u.dev(Wf), nbit)
    w_ref, s_ref = oracle.intb_encode(Wf, nbit)
    assert np.array_equal(u.host(s).view(np.uint16), s_ref.view(np.uint16))
    assert np.array_equal(u.host(w), w_ref)


@pytest.mark.parametrize("nbit", [8, 4])
@pytest.mark.parametrize("N,K", [(64, 64), (128, 448), (1024, 2048)])
def test_intb_encode_group64_bit_exact(ops, u, oracle, nbit, N, K):
    Wf = _weights(N, K, seed=N + K + nbit + 1)
    w, s = ops.intb_encode(u.dev(Wf), nbit, group_size=64)
    if K == 64:  # one group per row is the per-channel form
        w_ref, s_ref = oracle.intb_encode(Wf, nbit)
        assert tuple(s.shape) == (N,)
    else:
        w_ref, s_ref = oracle.intb_encode_grouped(Wf, nbit)
        assert tuple(s.shape) == (K // 64, N)
    assert np.array_equal(u.host(s).view(np.uint16), s_ref.view(np.uint16))
    assert np.array_equal(u.host(w), w_ref)


@pytest.mark.parametrize("N,K", [(1, 32), (7, 96), (300, 1024), (4096, 4096)])
def test_q4g32_encode_bit_exact_and_round_trip(ops, u, oracle, N, K):
    Wf = _weights(max(N, 3), K, seed=N + K)[:N] if N >= 3 else _weights(3, K, seed=N + K)[:N]
    W, S = ops.q4g32_encode(u.dev(Wf))
    W_ref, S_ref = oracle.q4g32_encode(Wf)
    assert np.array_equal(u.host(S).view(np.uint16), S_ref.view(np.uint16))
    assert np.array_equal(u.host(W).view(np.uint32), W_ref)
    # decode(encode(w)) stays within half a quantization step of w
    deq = u.host(ops.q4g32_dequantize(W, S)).astype(np.float64)
    step = np.repeat(S_ref.astype(np.float64), 32, axis=1)
    assert np.all(np.abs(deq - Wf.astype(np.float64)) <= 0.5 * step * 1.01 + 1e-7)


@pytest.mark.parametrize("nbit,group_size", [(8, -1), (4, -1), (8, 64), (4, 64)])
def test_encode_preprocess_gemm_chain_vs_unquantized(ops, u, oracle, nbit, group_size):
    """x @ w^T through the quantized path agrees with the unquantized fp16 product to the accuracy the
    quantizer allows (the reference asserts rtol = atol = 1e-2 for int8 at these magnitudes)."""
    rng = np.random.default_rng(nbit + group_size)
    M, N, K = 64, 128, 256
    x = rng.standard_normal((M, K)).astype(np.float16)
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    q, s = ops.intb_encode(u.dev(w), nbit, group_size=group_size)
    P = ops.ft_preprocess_weight(q, 80, nbit == 4)
    got = u.host(ops.fpA_intB_gemm(u.dev(x), P, s, weight_nbit=nbit, group_size=group_size)).astype(np.float64)
    # exact parity with the oracle on the same quantized weights ...
    ref = oracle.intb_linear(x, u.host(q), u.host(s), nbit, group_size=group_size)
    u.assert_close(got, ref, "quantized chain")
    # ... and closeness to the unquantized product
    full = x.astype(np.float64) @ w.astype(np.float64).T
    err = np.abs(got - full).max() / np.abs(full).max()
    assert err < (0.02 if nbit == 8 else 0.2), err


def test_q4g32_encode_linear_chain_vs_unquantized(ops, u, oracle):
    rng = np.random.default_rng(12)
    M, N, K = 16, 256, 512
    x = rng.standard_normal((M, K)).astype(np.float16)
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    W, S = ops.q4g32_encode(u.dev(w))
    got = u.host(ops.q4g32_linear(W, S, u.dev(x))).astype(np.float64)
    u.assert_close(got, oracle.q4g32_linear(u.host(W).view(np.uint32), u.host(S), x), "encoded linear")
    full = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(got - full).max() / np.abs(full).max() < 0.2


def test_encode_argument_errors(ops, u):
    import torch

    from relax_amd._lib import WqError

    with pytest.raises(WqError):
        ops.intb_encode(torch.zeros((60, 64), dtype=torch.float16, device="cuda"), 8)
    with pytest.raises(WqError):
        ops.intb_encode(torch.zeros((64, 64), dtype=torch.float16, device="cuda"), 3)
    with pytest.raises(WqError):
        ops.intb_encode(torch.zeros((64, 128), dtype=torch.float16, device="cuda"), 8, group_size=32)
    with pytest.raises(ValueError):
        ops.q4g32_encode(torch.zeros((4, 40), dtype=torch.float16, device="cuda"))
