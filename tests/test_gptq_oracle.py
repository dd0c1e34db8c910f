"""Pins the oracle's AutoGPTQ functions against independent evidence (no GPU)."""
import numpy as np
import pytest


def _pack_kn(codes):
    """codes uint8 [K, N] -> uint32 [K/8, N], code k%8 of a word in bits 4*(k%8).."""
    K, N = codes.shape
    c = codes.reshape(K // 8, 8, N).astype(np.uint32)
    w = np.zeros((K // 8, N), np.uint32)
    for i in range(8):
        w |= c[:, i, :] << np.uint32(4 * i)
    return w


def _pack_zeros(z):
    """z uint8 [G, N] -> uint32 [G, N/8], zero n%8 of a word in bits 4*(n%8).."""
    G, N = z.shape
    c = z.reshape(G, N // 8, 8).astype(np.uint32)
    w = np.zeros((G, N // 8), np.uint32)
    for i in range(8):
        w |= c[:, :, i] << np.uint32(4 * i)
    return w


def test_gptq_dequant_hand_case(oracle):
    K, N, G = 8, 8, 2
    qweight = np.zeros((1, N), np.uint32)
    qweight[0, 3] = 0xFEDCBA98  # codes 8, 9, ..., 15 for k = 0..7 of column 3
    qzeros = np.zeros((G, 1), np.uint32)
    qzeros[0, 0] = 0x00005000  # column 3, group 0: zero 5 -> subtract 6
    qzeros[1, 0] = 0x00002000  # column 3, group 1: zero 2 -> subtract 3
    scales = np.ones((G, N), np.float16)
    scales[0, 3], scales[1, 3] = 0.5, 0.25
    g_idx = np.array([0, 1, 0, 1, 1, 0, 0, 1], np.int32)
    B = oracle.gptq_dequant(qweight, qzeros, scales, g_idx)
    assert B[:, 3].tolist() == [1.0, 1.5, 2.0, 2.0, 2.25, 3.5, 4.0, 3.0]
    # the other columns hold code 0 and zero 0 with scale 1: 0 - (0 + 1) = -1
    assert np.all(np.delete(B, 3, axis=1) == -1.0)


def test_gptq_dequant_exhaustive(oracle):
    # every (code, zero) pair against every scale bit pattern: k = 16*code + zero, group = zero
    K, N, G = 256, 65536, 16
    k = np.arange(K)
    codes = np.broadcast_to((k // 16).astype(np.uint8)[:, None], (K, N))
    zeros = np.broadcast_to(np.arange(G, dtype=np.uint8)[:, None], (G, N))
    scales = np.broadcast_to(np.arange(N, dtype=np.uint32).astype(np.uint16).view(np.float16), (G, N)).copy()
    g_idx = (k % 16).astype(np.int32)
    got = oracle.gptq_dequant(_pack_kn(codes), _pack_zeros(zeros), scales, g_idx)
    with np.errstate(over="ignore", invalid="ignore"):
        zp = zeros[g_idx].astype(np.float16) + np.float16(1)
        want = (codes.astype(np.float16) - zp) * scales[g_idx]
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])
    assert np.all(np.isnan(got[nan]))


def test_gptq_dequant_reduces_to_k_major_q4f16_1(oracle):
    # zero 6 everywhere and groups of 32 consecutive k: (q - 7) * s, the K-major q4f16_1 decode
    rng = np.random.default_rng(5)
    K, N = 128, 48
    G = K // 32
    qweight = rng.integers(0, 2**32, size=(K // 8, N), dtype=np.uint64).astype(np.uint32)
    scales = rng.uniform(0.005, 0.02, size=(G, N)).astype(np.float16)
    qzeros = np.full((G, N // 8), 0x66666666, np.uint32)
    g_idx = (np.arange(K) // 32).astype(np.int32)
    got = oracle.gptq_dequant(qweight, qzeros, scales, g_idx)
    assert np.array_equal(got.view(np.uint16), oracle.q4g32_kn_dequant(qweight, scales).view(np.uint16))


def test_gptq_dequant_row_permutation(oracle):
    rng = np.random.default_rng(6)
    K, N, G = 64, 24, 4
    codes = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    zeros = rng.integers(0, 16, size=(G, N), dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, size=(G, N)).astype(np.float16)
    g_idx = rng.integers(0, G, size=K).astype(np.int32)  # unequal group sizes on purpose
    base = oracle.gptq_dequant(_pack_kn(codes), _pack_zeros(zeros), scales, g_idx)
    perm = rng.permutation(K)
    moved = oracle.gptq_dequant(_pack_kn(codes[perm]), _pack_zeros(zeros), scales, np.ascontiguousarray(g_idx[perm]))
    assert np.array_equal(moved.view(np.uint16), base[perm].view(np.uint16))
    # and the value itself, element by element in python
    for kk in (0, 17, 63):
        for n in (0, 9, 23):
            g = g_idx[kk]
            want = (np.float16(codes[kk, n]) - (np.float16(zeros[g, n]) + np.float16(1))) * scales[g, n]
            assert base[kk, n] == want


def test_gptq_dequant_rejects_bad_group(oracle):
    K, N, G = 8, 8, 1
    with pytest.raises(ValueError):
        oracle.gptq_dequant(np.zeros((1, N), np.uint32), np.zeros((G, 1), np.uint32), np.ones((G, N), np.float16),
                            np.array([0, 0, 0, 1, 0, 0, 0, 0], np.int32))


def test_kn_matmul_modes(oracle):
    rng = np.random.default_rng(7)
    M, K, N = 3, 96, 40
    B = (rng.standard_normal((K, N)) * 0.05).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    # fp32 mode: one rounding away from the float64 product, then the fp16 residual add
    y32 = oracle.kn_matmul(B, x, None, f32acc=True)
    exact = x.astype(np.float64) @ B.astype(np.float64)
    assert np.max(np.abs(y32.astype(np.float64) - exact)) <= 2.0**-11 * np.max(np.abs(exact)) + 1e-4
    y32r = oracle.kn_matmul(B, x, res, f32acc=True)
    assert np.array_equal(y32r.view(np.uint16), (res + y32).view(np.uint16))
    # fp16 mode: the reference's sequence, replayed with numpy.float16 scalars
    y16 = oracle.kn_matmul(B, x, res, f32acc=False)
    for m in range(M):
        for n in range(0, N, 7):
            acc = np.float16(0)
            for k in range(K):
                acc = np.float16(acc + np.float16(x[m, k] * B[k, n]))
            assert y16[m, n] == np.float16(res[m, n] + acc)
    # a one-hot activation selects a row of B in both modes
    e = np.zeros((1, K), np.float16)
    e[0, 37] = 1
    for mode in (True, False):
        assert np.array_equal(oracle.kn_matmul(B, e, None, f32acc=mode)[0].view(np.uint16), B[37].view(np.uint16))


def test_gptq_linear_against_float64(oracle):
    x, qw, qz, s, g_idx = oracle.make_gptq_inputs(2, 64, 256, 64, seed=3, act_order=True)
    y = oracle.gptq_linear(qw, qz, s, g_idx, x)
    B = oracle.gptq_dequant(qw, qz, s, g_idx).astype(np.float64)
    exact = x.astype(np.float64) @ B
    assert np.max(np.abs(y.astype(np.float64) - exact)) <= 2.0**-10 * np.max(np.abs(exact))
    counts = np.bincount(g_idx, minlength=4)
    assert counts.tolist() == [64] * 4 and not np.array_equal(g_idx, np.arange(256) // 64)
