"""Pins the CPU oracle against independent evidence (no GPU).

numpy's float16 is the independent library for rounding and fp16 arithmetic;
float64 matmul, one-hot selection and algebraic invariants fix the matmuls.
"""
import numpy as np
import pytest


def test_f16_to_f32_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    for portable in (False, True):
        got = oracle.f16_to_f32(bits, portable=portable)
        assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
        assert np.all(np.isnan(got[nan]))  # the F16C path quiets signalling NaNs


def _interesting_f32():
    rng = np.random.default_rng(0)
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    h = bits.view(np.float16).astype(np.float32)
    pieces = [h]
    # midpoints between neighbouring halves (ties) and their float32 neighbours
    fin = np.sort(h[np.isfinite(h)])
    mid = ((fin[:-1].astype(np.float64) + fin[1:].astype(np.float64)) / 2).astype(np.float32)
    pieces += [mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))]
    pieces.append(rng.integers(0, 2**32, size=4_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32))
    pieces.append(np.array([65504, 65519.99, 65520, 65535, 65536, 1e30, 2.0**-24, 2.0**-25,
                            np.nextafter(np.float32(2.0**-25), np.float32(1)), 2.0**-26, 0.0, -0.0,
                            np.inf, -np.inf], np.float32))
    return np.concatenate(pieces)


def test_f32_to_f16_rne_dense(oracle):
    f = _interesting_f32()
    with np.errstate(over="ignore", invalid="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    nan = np.isnan(f)
    for portable in (False, True):
        got = oracle.f32_to_f16(f, portable=portable)
        assert np.array_equal(got[~nan], want[~nan])
        # NaNs stay NaNs (payload conventions differ between libraries)
        assert np.all(np.isnan(got[nan].view(np.float16)))


def test_q4_unpack_bruteforce(oracle):
    # every code in every slot, one at a time
    for slot in range(8):
        for code in range(16):
            W = np.array([[np.uint32(code) << np.uint32(4 * slot)]], np.uint32)
            q = oracle.q4_unpack(W)
            want = np.zeros(8, np.uint8)
            want[slot] = code
            assert np.array_equal(q[0], want)
    # hand-written word: nibble i holds i+1
    W = np.array([[0x87654321, 0xFEDCBA90]], np.uint32)
    assert oracle.q4_unpack(W)[0].tolist() == [1, 2, 3, 4, 5, 6, 7, 8, 0, 9, 10, 11, 12, 13, 14, 15]
    rng = np.random.default_rng(1)
    q = rng.integers(0, 16, size=(7, 64)).astype(np.uint8)
    assert np.array_equal(oracle.q4_unpack(oracle.q4_pack(q)), q)
    W = rng.integers(0, 2**32, size=(5, 12), dtype=np.uint64).astype(np.uint32)
    assert np.array_equal(oracle.q4_pack(oracle.q4_unpack(W)), W)


def test_q4g32_dequant_exhaustive(oracle):
    """16 codes x all 65536 fp16 scale bit patterns, against numpy float16 arithmetic."""
    all_s = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16)
    # row n holds scale n for its single group; the 32 codes of the group cover 0..15 twice
    codes = np.tile(np.arange(16, dtype=np.uint8), 2)[None, :].repeat(65536, 0)
    W = oracle.q4_pack(codes)
    S = all_s.reshape(65536, 1)
    got = oracle.q4g32_dequant(W, S)
    with np.errstate(all="ignore"):
        want = (codes.astype(np.float16) - np.float16(7)) * S
    g, w = got.view(np.uint16), want.view(np.uint16)
    nan = np.isnan(want)
    assert np.array_equal(g[~nan], w[~nan])
    assert np.all(np.isnan(got[nan]))


@pytest.mark.parametrize("nbit", [8, 4])
def test_intb_dequant_exhaustive(oracle, nbit):
    all_s = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16)
    ncode = 256 if nbit == 8 else 16
    lo = -128 if nbit == 8 else -8
    codes = np.arange(lo, lo + ncode, dtype=np.int64)
    # columns n = scale index (in chunks to bound memory), rows k = code
    for start in range(0, 65536, 8192):
        s = all_s[start:start + 8192]
        N = s.size
        q = np.repeat(codes[:, None], N, axis=1)
        if nbit == 8:
            A = q.astype(np.int8)
        else:
            A = ((q[:, 0::2] & 15) | ((q[:, 1::2] & 15) << 4)).astype(np.uint8).view(np.int8)
        assert np.array_equal(oracle.intb_unpack(A, nbit), q.astype(np.int8))
        got = oracle.intb_dequant(A, s, nbit)
        with np.errstate(all="ignore"):
            want = q.astype(np.float16) * s[None, :]
        nan = np.isnan(want)
        assert np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])
        assert np.all(np.isnan(got[nan]))


def test_intb_finegrained_scale_indexing(oracle):
    x, A, s = oracle.make_intb_inputs(1, 64, 256, 8, seed=3, group_size=64)
    got = oracle.intb_dequant(A, s, 8, group_size=64)
    want = A.astype(np.float16) * np.repeat(s, 64, axis=0)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_nt_matmul_against_float64(oracle):
    x, W, S = oracle.make_q4g32_inputs(3, 96, 512, seed=11)
    B = oracle.q4g32_dequant(W, S)
    y = oracle.nt_matmul_f32acc(B, x).astype(np.float64)
    ref = x.astype(np.float64) @ B.astype(np.float64).T
    assert np.max(np.abs(y - ref)) <= 2e-3 * np.max(np.abs(ref))
    # the fused entry gives the same bits as decode followed by matmul
    assert np.array_equal(oracle.q4g32_linear(W, S, x).view(np.uint16), oracle.nt_matmul_f32acc(B, x).view(np.uint16))
    # threads only split rows: same bits
    assert np.array_equal(oracle.q4g32_linear(W, S, x, nthreads=4).view(np.uint16),
                          oracle.q4g32_linear(W, S, x).view(np.uint16))


def test_nt_matmul_invariants(oracle):
    N, K = 64, 256
    _, W, S = oracle.make_q4g32_inputs(1, N, K, seed=5)
    B = oracle.q4g32_dequant(W, S)
    # one-hot x selects a dequantized column exactly (a transposed operand would fail this)
    for k in (0, 1, 7, 8, 31, 32, 255):
        x = np.zeros((1, K), np.float16)
        x[0, k] = 1
        assert np.array_equal(oracle.q4g32_linear(W, S, x)[0].view(np.uint16), B[:, k].view(np.uint16))
    # all codes 7 -> exact zeros whatever the scales
    W7 = np.full((N, K // 8), 0x77777777, np.uint32)
    x = np.random.default_rng(0).standard_normal((2, K)).astype(np.float16)
    assert not np.any(oracle.q4g32_linear(W7, S, x))
    # scaling x by a power of two scales y exactly
    y1 = oracle.q4g32_linear(W, S, x)
    y2 = oracle.q4g32_linear(W, S, (x * np.float16(4)).astype(np.float16))
    assert np.array_equal((y1 * np.float16(4)).view(np.uint16), y2.view(np.uint16))


def test_nt_epilogue_bias_residual(oracle):
    x, W, S = oracle.make_q4g32_inputs(4, 32, 128, seed=2)
    rng = np.random.default_rng(4)
    bias = rng.standard_normal(32).astype(np.float16)
    res = rng.standard_normal((4, 32)).astype(np.float16)
    B = oracle.q4g32_dequant(W, S)
    acc = x.astype(np.float64) @ B.astype(np.float64).T
    want = (acc + bias.astype(np.float64)).astype(np.float16) + res
    got = oracle.q4g32_linear(W, S, x, bias=bias, residual=res)
    assert np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))) <= 4e-3 * np.max(np.abs(want))


def test_f16acc_matmul_matches_numpy_sequence(oracle):
    x, W, S = oracle.make_q4g32_inputs(1, 8, 64, seed=9)
    B = oracle.q4g32_dequant(W, S)
    got = oracle.nt_matmul_f16acc(B, x)
    want = np.zeros((1, 8), np.float16)
    for n in range(8):
        acc = np.float16(0)
        for k in range(64):
            acc = np.float16(acc + np.float16(x[0, k] * B[n, k]))
        want[0, n] = acc
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("nbit", [8, 4])
def test_nn_matmul_and_epilogues(oracle, nbit):
    from scipy.special import erf

    M, N, K = 5, 64, 128
    x, A, s = oracle.make_intb_inputs(M, N, K, nbit, seed=21)
    Wd = oracle.intb_dequant(A, s, nbit)
    rng = np.random.default_rng(8)
    bias = rng.standard_normal(N).astype(np.float16)
    bias2 = rng.standard_normal((M, N)).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    acc = x.astype(np.float64) @ Wd.astype(np.float64)

    def close(got, want):
        want = np.asarray(want, np.float64)
        assert np.max(np.abs(got.astype(np.float64) - want)) <= 2e-3 * max(1.0, np.max(np.abs(want)))

    close(oracle.intb_linear(x, A, s, nbit), acc)
    close(oracle.intb_linear(x, A, s, nbit, bias=bias), acc + bias)
    close(oracle.intb_linear(x, A, s, nbit, bias=bias2, bias_stride=N), acc + bias2)
    close(oracle.intb_linear(x, A, s, nbit, bias=bias, activation="relu"), np.maximum(acc + bias, 0))
    v = acc + bias
    close(oracle.intb_linear(x, A, s, nbit, bias=bias, activation="silu"), v / (1 + np.exp(-v)))
    close(oracle.intb_linear(x, A, s, nbit, bias=bias, activation="gelu"), 0.5 * v * (1 + erf(v / np.sqrt(2))))
    close(oracle.intb_linear(x, A, s, nbit, bias=bias, residual=res, binary_op="plus"), v + res)
    close(oracle.intb_linear(x, A, s, nbit, bias=bias, residual=res, binary_op="multiply", unary_op="relu"),
          np.maximum(v * res, 0))
    # one-hot row of x selects a dequantized weight row exactly
    xh = np.zeros((1, K), np.float16)
    xh[0, 77] = 1
    assert np.array_equal(oracle.intb_linear(xh, A, s, nbit)[0].view(np.uint16), Wd[77].view(np.uint16))


@pytest.mark.parametrize("nbit", [8, 4])
def test_intb_encode_closed_form(oracle, nbit):
    rng = np.random.default_rng(0)
    N, K = 128, 64
    Wf = rng.normal(0, 0.002, size=(N, K)).astype(np.float16)
    w, s = oracle.intb_encode(Wf, nbit)
    q = oracle.intb_unpack(w, nbit).astype(np.int64)  # [K,N]
    c = 0.125 if nbit == 4 else 0.0078125
    scale = np.maximum(np.abs(Wf).max(axis=1).astype(np.float32), np.float32(1e-4)) * np.float32(c)
    assert np.array_equal(s.view(np.uint16), scale.astype(np.float16).view(np.uint16))
    r = Wf.astype(np.float32) / scale[:, None]
    want = np.clip(np.sign(r) * np.floor(np.abs(r) + np.float32(0.5)), -8 if nbit == 4 else -128, 7 if nbit == 4 else 127)
    assert np.array_equal(q, want.T.astype(np.int64))
    # the largest element of every row maps to +-full scale (8 clips to 7 for int4)
    top = np.abs(q).max(axis=0)
    assert np.all(top >= (7 if nbit == 4 else 127))


def _round_half_away(r):
    return np.sign(r) * np.floor(np.abs(r) + np.float32(0.5))


@pytest.mark.parametrize("nbit", [8, 4])
def test_intb_encode_grouped_closed_form(oracle, nbit):
    """group-64 quantizer (tests/python/relax/test_codegen_cutlass.py:2044-2109) against a numpy
    restatement in float32, and against the per-channel one where they must agree (K = 64)."""
    rng = np.random.default_rng(3)
    N, K = 64, 256
    Wf = (rng.normal(0, 0.02, size=(N, K)) * rng.uniform(0.1, 4, size=(N, 1))).astype(np.float16)
    Wf[5, 64:128] = 0  # an all-zero group takes the 1e-4 floor
    w, s = oracle.intb_encode_grouped(Wf, nbit)
    q = oracle.intb_unpack(w, nbit).astype(np.int64)  # [K, N]
    c = np.float32(0.125 if nbit == 4 else 0.0078125)
    lo, hi = (-8, 7) if nbit == 4 else (-128, 127)
    g = Wf.reshape(N, K // 64, 64)
    scale = np.maximum(np.abs(g).max(axis=2).astype(np.float32), np.float32(1e-4)) * c  # [N, K/64]
    assert np.array_equal(s.view(np.uint16), scale.T.astype(np.float16).view(np.uint16))
    want = np.clip(_round_half_away(g.astype(np.float32) / scale[:, :, None]), lo, hi).reshape(N, K)
    assert np.array_equal(q, want.T.astype(np.int64))
    assert np.all(q[64:128, 5] == 0)
    w1, s1 = oracle.intb_encode(Wf[:, :64].copy(), nbit)
    wg, sg = oracle.intb_encode_grouped(Wf[:, :64].copy(), nbit)
    assert np.array_equal(w1, wg) and np.array_equal(s1.view(np.uint16), sg[0].view(np.uint16))


def test_q4g32_encode_definition_and_round_trip(oracle):
    """The format-A quantizer has no counterpart in the reference tree (parity unpinned): checked are
    the stated definition (numpy restatement), the code range, the error bound of decode(encode(w))
    and that weights which are already on a quantization grid survive unchanged."""
    rng = np.random.default_rng(4)
    N, K = 48, 256
    Wf = (rng.normal(0, 0.05, size=(N, K)) * rng.uniform(0.05, 8, size=(N, 1))).astype(np.float16)
    Wf[3, 32:64] = 0
    W, S = oracle.q4g32_encode(Wf)
    q = oracle.q4_unpack(W).astype(np.int64)
    assert q.min() >= 0 and q.max() <= 14
    g = Wf.reshape(N, K // 32, 32)
    m = np.abs(g).max(axis=2).astype(np.float32)
    s_want = (np.maximum(m, np.float32(1e-4)) / np.float32(7)).astype(np.float16)
    assert np.array_equal(S.view(np.uint16), s_want.view(np.uint16))
    r = g.astype(np.float32) / s_want.astype(np.float32)[:, :, None]
    want = np.clip(_round_half_away(r) + 7, 0, 14).reshape(N, K)
    assert np.array_equal(q, want.astype(np.int64))
    assert np.all(q[3, 32:64] == 7)
    # error bound: half a step, plus the fp16 roundings of scale and product
    deq = oracle.q4g32_dequant(W, S).astype(np.float64)
    step = np.repeat(S.astype(np.float64), 32, axis=1)
    assert np.all(np.abs(deq - Wf.astype(np.float64)) <= 0.5 * step * 1.01 + 1e-7)
    # every group reaches full scale on one side
    qq = q.reshape(N, K // 32, 32)
    nz = m > 1e-4
    assert np.all(((qq.min(axis=2) == 0) | (qq.max(axis=2) == 14))[nz])
    # grid weights: codes with full-scale groups and power-of-two scales are reproduced exactly
    codes = rng.integers(0, 15, size=(N, K)).astype(np.uint8)
    codes[:, ::32] = 14
    W0 = oracle.q4_pack(codes)
    S0 = np.full((N, K // 32), 2.0 ** -6, np.float16)
    Wgrid = oracle.q4g32_dequant(W0, S0)
    W1, S1 = oracle.q4g32_encode(Wgrid)
    assert np.array_equal(oracle.q4g32_dequant(W1, S1).view(np.uint16), Wgrid.view(np.uint16))


def test_kn_layout_oracle_matches_loops_and_nk_form(oracle):
    """K-major q4f16_1: brute-force loops over the TIR expression on a small case, and equality with the
    NK oracle on the transposed arrays (a word holds the same 8 k of one column in both layouts)."""
    rng = np.random.default_rng(6)
    N, K = 5, 64
    W_kn = rng.integers(0, 2**32, size=(K // 8, N), dtype=np.uint64).astype(np.uint32)
    S_kn = rng.uniform(0.005, 0.02, size=(K // 32, N)).astype(np.float16)
    B = oracle.q4g32_kn_dequant(W_kn, S_kn)
    for k in range(K):
        for n in range(N):
            q = (int(W_kn[k // 8, n]) >> (4 * (k % 8))) & 15
            want = (np.float16(q) - np.float16(7)) * S_kn[k // 32, n]
            assert B[k, n].view(np.uint16) == np.float16(want).view(np.uint16)
    nk = oracle.q4g32_dequant(np.ascontiguousarray(W_kn.T), np.ascontiguousarray(S_kn.T))
    assert np.array_equal(nk.view(np.uint16), np.ascontiguousarray(B.T).view(np.uint16))
    x = rng.standard_normal((3, K)).astype(np.float16)
    y = oracle.q4g32_kn_linear(W_kn, S_kn, x)
    y_nk = oracle.q4g32_linear(np.ascontiguousarray(W_kn.T), np.ascontiguousarray(S_kn.T), x)
    assert np.allclose(y.astype(np.float32), y_nk.astype(np.float32), rtol=2e-3, atol=2e-3)


def test_weights_packed_along_n_are_format_a_with_the_dimensions_exchanged(oracle):
    """The decode block of tests/python/dlight/test_gpu_matmul.py:366-377, written out index by index
    (D[i, j] from W[i, j // 8] and S[i, j // 32]), and its matmul (:378-383, D[k, n]) in float64: the oracle the GPU
    tests of that layout use — wqo_q4g32_dequant on the same two arrays, then the NT matmul over the transpose."""
    K, N, M = 24, 96, 3
    rng = np.random.default_rng(17)
    W = rng.integers(0, 2**32, size=(K, N // 8), dtype=np.uint64).astype(np.uint32)
    S = rng.uniform(0.005, 0.02, size=(K, N // 32)).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    D = np.zeros((K, N), np.float16)
    for i in range(K):
        for j in range(N):
            code = (int(W[i, j // 8]) >> ((j % 8) * 4)) & 15
            D[i, j] = np.float16(np.float16(code) - np.float16(7)) * S[i, j // 32]
    got = oracle.q4g32_dequant(W, S)
    assert got.shape == (K, N) and np.array_equal(got.view(np.uint16), D.view(np.uint16))
    y = oracle.nt_matmul_f32acc(np.ascontiguousarray(got.T), x)
    want = x.astype(np.float64) @ D.astype(np.float64)
    assert np.allclose(y.astype(np.float64), want, rtol=2e-3, atol=2e-3)
