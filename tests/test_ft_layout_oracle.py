"""Pins the oracle's weight-reordering against golden vectors (no GPU).

tests/golden/ft_layout_vectors.npz was produced by tests/golden/make_ft_layout_vectors.py
from PyTorch's own restatement of the layout (an independent implementation).
"""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden", "ft_layout_vectors.npz")
CASES = ["int8_64x64", "int8_128x192", "int8_256x64", "int4_64x64", "int4_128x192", "int4_256x128"]


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD)


@pytest.mark.parametrize("case", CASES)
def test_preprocess_matches_golden(oracle, gold, case):
    a, want = gold[case + "_in"], gold[case + "_out"]
    got = oracle.ft_preprocess(a, is_int4=case.startswith("int4"), sm=80)
    assert got.shape == want.shape and got.dtype == np.int8
    assert np.array_equal(got, want)


@pytest.mark.parametrize("case", CASES)
def test_unprocess_inverts_golden(oracle, gold, case):
    a, out = gold[case + "_in"], gold[case + "_out"]
    assert np.array_equal(oracle.ft_unprocess(out, is_int4=case.startswith("int4"), sm=80), a)


@pytest.mark.parametrize("is_int4", [False, True])
def test_preprocess_invariants(oracle, is_int4):
    rng = np.random.default_rng(12)
    K, N = 128, 128
    cols = N // 2 if is_int4 else N
    a = rng.integers(-128, 128, size=(K, cols)).astype(np.int8)
    p = oracle.ft_preprocess(a, is_int4, 80)
    # same multiset of codes, shifted by the bias
    if is_int4:
        nib = lambda z: np.concatenate([(z.view(np.uint8) & 15).ravel(), (z.view(np.uint8) >> 4).ravel()])
        src = (nib(a).astype(np.int64) ^ 8)  # two's complement nibble + 8  ==  flip the top bit
        assert np.array_equal(np.sort(src), np.sort(nib(p).astype(np.int64)))
    else:
        assert np.array_equal(np.sort((a.astype(np.int64) + 128).ravel()), np.sort(p.view(np.uint8).astype(np.int64).ravel()))
    # a single marked element lands in exactly one place (bijection), and the round trip restores it
    assert np.array_equal(oracle.ft_unprocess(p, is_int4, 80), a)
    # every sm of the family gives the same layout; others are refused
    for sm in (75, 80, 86, 89):
        assert np.array_equal(oracle.ft_preprocess(a, is_int4, sm), p)
    for sm in (70, 90):
        with pytest.raises(ValueError):
            oracle.ft_preprocess(a, is_int4, sm)
    # stacked experts are processed independently
    e = np.stack([a, a[::-1].copy()])
    pe = oracle.ft_preprocess(e, is_int4, 80)
    assert np.array_equal(pe[0], p) and np.array_equal(pe[1], oracle.ft_preprocess(a[::-1].copy(), is_int4, 80))


def test_int8_layout_closed_form(oracle):
    """Independent closed form of the int8 result: column pairs are interleaved per
    64-row tile, and inside each 16-row block the bytes appear in the order
    0,8,1,9,2,10,...,7,15 (the order one tensor-core lane consumes them)."""
    rng = np.random.default_rng(3)
    K, N = 128, 64
    a = rng.integers(-128, 128, size=(K, N)).astype(np.int8)
    p = oracle.ft_preprocess(a, False, 80).view(np.uint8).ravel()
    order = [0, 8, 1, 9, 2, 10, 3, 11, 4, 12, 5, 13, 6, 14, 7, 15]
    want = np.empty(K * N, np.uint8)
    pos = 0
    for pair in range(N // 2):
        for tile in range(K // 64):
            for c in range(2):
                for blk in range(4):
                    for o in order:
                        want[pos] = (int(a[tile * 64 + blk * 16 + o, 2 * pair + c]) + 128) & 255
                        pos += 1
    assert np.array_equal(p, want)
