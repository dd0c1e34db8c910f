"""ctypes front end of the CPU oracle (``oracle/wq_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by the tests, by the smoke check and by the
benchmark's ``cpu_baseline`` leg, always as the checker.  The product package
never imports this module.

All arrays are numpy; fp16 tensors are passed as ``np.float16`` and viewed as
``uint16`` at the C boundary.  Shapes follow the reference's fixtures:

* format A (q4f16_1):  ``W uint32 [N, K/8]``, ``S float16 [N, K/32]``, ``x float16 [M, K]``
  (tests/python/dlight/test_gpu_reduction.py:33-51, 400-424)
* format B (fpA_intB): ``A int8 [K, N]`` or ``[K, N/2]``, ``scales float16 [N]`` or ``[K/g, N]``
  (tests/python/relax/test_codegen_cutlass.py:1359-1389, 1616-1628, 2030-2041)
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libwq_oracle.so")

ACTIVATIONS = {"identity": 0, "relu": 1, "silu": 2, "gelu": 3}
BINARY_OPS = {"none": 0, "plus": 1, "multiply": 2}
UNARY_OPS = {"identity": 0, "relu": 1}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a few seconds)."""
    src = os.path.join(_HERE, "wq_oracle.c")
    stale = (not os.path.exists(_LIB_PATH)) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src)
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B", "libwq_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.wqo_ft_preprocess.restype = ctypes.c_int
        _lib.wqo_ft_unprocess.restype = ctypes.c_int
    return _lib


def _p(a: np.ndarray):
    return ctypes.c_void_p(a.ctypes.data)


def _opt(a):
    return ctypes.c_void_p(0) if a is None else _p(a)


def _c(a, dtype):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.dtype(dtype), (a.dtype, dtype)
    return a


i64 = ctypes.c_int64
cint = ctypes.c_int

# ----------------------------------------------------------------- fp16


def f16_to_f32(h_bits: np.ndarray, portable: bool = False) -> np.ndarray:
    h_bits = _c(h_bits, np.uint16)
    out = np.empty(h_bits.shape, np.float32)
    lib().wqo_f16_to_f32_array(_p(h_bits), _p(out), i64(h_bits.size), cint(int(portable)))
    return out


def f32_to_f16(f: np.ndarray, portable: bool = False) -> np.ndarray:
    f = _c(f, np.float32)
    out = np.empty(f.shape, np.uint16)
    lib().wqo_f32_to_f16_array(_p(f), _p(out), i64(f.size), cint(int(portable)))
    return out


# ------------------------------------------------------------- format A


def q4_unpack(W: np.ndarray) -> np.ndarray:
    W = _c(W, np.uint32)
    N, kw = W.shape
    q = np.empty((N, kw * 8), np.uint8)
    lib().wqo_q4_unpack(_p(W), _p(q), i64(N), i64(kw * 8))
    return q


def q4_pack(q: np.ndarray) -> np.ndarray:
    q = _c(q, np.uint8)
    N, K = q.shape
    W = np.empty((N, K // 8), np.uint32)
    lib().wqo_q4_pack(_p(q), _p(W), i64(N), i64(K))
    return W


def q4g32_dequant(W: np.ndarray, S: np.ndarray) -> np.ndarray:
    W = _c(W, np.uint32)
    S = _c(S, np.float16)
    N, kw = W.shape
    K = kw * 8
    assert S.shape == (N, K // 32)
    out = np.empty((N, K), np.float16)
    lib().wqo_q4g32_dequant(_p(W), _p(S), _p(out), i64(N), i64(K))
    return out


def nt_matmul_f32acc(Bdeq, X, bias=None, residual=None, nthreads: int = 1) -> np.ndarray:
    Bdeq = _c(Bdeq, np.float16)
    X = _c(X, np.float16)
    N, K = Bdeq.shape
    M = X.shape[0]
    assert X.shape == (M, K)
    bias = None if bias is None else _c(bias, np.float16).reshape(N)
    residual = None if residual is None else _c(residual, np.float16).reshape(M, N)
    Y = np.empty((M, N), np.float16)
    lib().wqo_nt_matmul_f32acc(_p(Bdeq), _p(X), _opt(bias), _opt(residual), _p(Y), i64(M), i64(N), i64(K), cint(nthreads))
    return Y


def nt_matmul_f16acc(Bdeq, X) -> np.ndarray:
    Bdeq = _c(Bdeq, np.float16)
    X = _c(X, np.float16)
    N, K = Bdeq.shape
    M = X.shape[0]
    Y = np.empty((M, N), np.float16)
    lib().wqo_nt_matmul_f16acc(_p(Bdeq), _p(X), _p(Y), i64(M), i64(N), i64(K))
    return Y


def q4g32_linear(W, S, X, bias=None, residual=None, nthreads: int = 1) -> np.ndarray:
    """decode + NT matmul, fp32 accumulate, fp16 out — the reference CPU path."""
    W = _c(W, np.uint32)
    S = _c(S, np.float16)
    X = _c(X, np.float16)
    N, kw = W.shape
    K = kw * 8
    M = X.shape[0]
    assert X.shape == (M, K) and S.shape == (N, K // 32)
    bias = None if bias is None else _c(bias, np.float16).reshape(N)
    residual = None if residual is None else _c(residual, np.float16).reshape(M, N)
    Y = np.empty((M, N), np.float16)
    lib().wqo_q4g32_linear(_p(W), _p(S), _p(X), _opt(bias), _opt(residual), _p(Y), i64(M), i64(N), i64(K), cint(nthreads))
    return Y


# ------------------------------------------------------------- format B


def _intb_dims(A: np.ndarray, nbit: int):
    K, c = A.shape
    return K, c * (2 if nbit == 4 else 1)


def intb_unpack(A: np.ndarray, nbit: int) -> np.ndarray:
    A = _c(A, np.int8)
    K, N = _intb_dims(A, nbit)
    q = np.empty((K, N), np.int8)
    lib().wqo_intb_unpack(_p(A), _p(q), i64(K), i64(N), cint(nbit))
    return q


def intb_dequant(A: np.ndarray, scales: np.ndarray, nbit: int, group_size: int = -1) -> np.ndarray:
    A = _c(A, np.int8)
    scales = _c(scales, np.float16)
    K, N = _intb_dims(A, nbit)
    assert scales.size == (N if group_size <= 0 else (K // group_size) * N)
    out = np.empty((K, N), np.float16)
    lib().wqo_intb_dequant(_p(A), _p(scales), _p(out), i64(K), i64(N), cint(nbit), i64(group_size))
    return out


def nn_matmul_f32acc(X, Wdeq, bias=None, residual=None, activation="identity", binary_op="none",
                     unary_op="identity", bias_stride: int = 0, nthreads: int = 1) -> np.ndarray:
    X = _c(X, np.float16)
    Wdeq = _c(Wdeq, np.float16)
    M, K = X.shape
    N = Wdeq.shape[1]
    bias = None if bias is None else _c(bias, np.float16)
    residual = None if residual is None else _c(residual, np.float16).reshape(M, N)
    C = np.empty((M, N), np.float16)
    lib().wqo_nn_matmul_f32acc(_p(X), _p(Wdeq), _opt(bias), _opt(residual), _p(C), i64(M), i64(N), i64(K),
                               cint(ACTIVATIONS[activation]), cint(BINARY_OPS[binary_op]),
                               cint(UNARY_OPS[unary_op]), i64(bias_stride), cint(nthreads))
    return C


def intb_linear(X, A, scales, nbit, bias=None, residual=None, group_size=-1, activation="identity",
                binary_op="none", unary_op="identity", bias_stride=0, nthreads=1) -> np.ndarray:
    """decode + NN matmul with the fused epilogue — the reference CPU path for format B.
    ``A`` is the packed weight BEFORE preprocessing."""
    X = _c(X, np.float16)
    A = _c(A, np.int8)
    scales = _c(scales, np.float16)
    M, K = X.shape
    K2, N = _intb_dims(A, nbit)
    assert K == K2
    bias = None if bias is None else _c(bias, np.float16)
    residual = None if residual is None else _c(residual, np.float16).reshape(M, N)
    C = np.empty((M, N), np.float16)
    lib().wqo_intb_linear(_p(X), _p(A), _p(scales), _opt(bias), _opt(residual), _p(C), i64(M), i64(N), i64(K),
                          cint(nbit), i64(group_size), cint(ACTIVATIONS[activation]),
                          cint(BINARY_OPS[binary_op]), cint(UNARY_OPS[unary_op]), i64(bias_stride), cint(nthreads))
    return C


def ft_preprocess(A: np.ndarray, is_int4: bool, sm: int = 80) -> np.ndarray:
    """cutlass.ft_preprocess_weight on a host array: int8 [K,N] | [K,N/2] | [E,K,N(/2)]."""
    A = _c(A, np.int8)
    if A.ndim == 2:
        E, (rows, c) = 1, A.shape
    else:
        E, rows, c = A.shape
    cols = c * 2 if is_int4 else c
    out = np.empty_like(A)
    rc = lib().wqo_ft_preprocess(_p(out), _p(A), i64(E), i64(rows), i64(cols), cint(int(is_int4)), cint(sm))
    if rc != 0:
        raise ValueError(f"unsupported preprocess request sm={sm} rows={rows} cols={cols}")
    return out


def ft_unprocess(A: np.ndarray, is_int4: bool, sm: int = 80) -> np.ndarray:
    A = _c(A, np.int8)
    if A.ndim == 2:
        E, (rows, c) = 1, A.shape
    else:
        E, rows, c = A.shape
    cols = c * 2 if is_int4 else c
    out = np.empty_like(A)
    rc = lib().wqo_ft_unprocess(_p(out), _p(A), i64(E), i64(rows), i64(cols), cint(int(is_int4)), cint(sm))
    if rc != 0:
        raise ValueError("unsupported unprocess request")
    return out


def intb_encode(Wf: np.ndarray, nbit: int):
    """The fixtures' per-channel quantizer: fp16 [N,K] -> (int8 [K,N] | [K,N/2], fp16 [N])."""
    Wf = _c(Wf, np.float16)
    N, K = Wf.shape
    w = np.zeros((K, N if nbit == 8 else N // 2), np.int8)
    s = np.empty((N,), np.float16)
    lib().wqo_intb_encode(_p(Wf), _p(w), _p(s), i64(N), i64(K), cint(nbit))
    return w, s


def intb_encode_grouped(Wf: np.ndarray, nbit: int):
    """The fixtures' group-64 quantizer: fp16 [N,K] -> (int8 [K,N] | [K,N/2], fp16 [K/64,N])."""
    Wf = _c(Wf, np.float16)
    N, K = Wf.shape
    assert K % 64 == 0
    w = np.zeros((K, N if nbit == 8 else N // 2), np.int8)
    s = np.empty((K // 64, N), np.float16)
    lib().wqo_intb_encode_grouped(_p(Wf), _p(w), _p(s), i64(N), i64(K), cint(nbit))
    return w, s


def q4g32_encode(Wf: np.ndarray):
    """q4f16_1 quantizer (a definition: the reference tree has none): fp16 [N,K] -> (uint32 [N,K/8], fp16 [N,K/32])."""
    Wf = _c(Wf, np.float16)
    N, K = Wf.shape
    assert K % 32 == 0
    W = np.empty((N, K // 8), np.uint32)
    S = np.empty((N, K // 32), np.float16)
    lib().wqo_q4g32_encode(_p(Wf), _p(W), _p(S), i64(N), i64(K))
    return W, S


def q4g32_kn_dequant(W_kn: np.ndarray, S_kn: np.ndarray) -> np.ndarray:
    """K-major form of the same scheme (tests/python/dlight/test_gpu_reduction.py:112-120):
    B[k, n] = (fp16((W[k // 8, n] >> 4 * (k % 8)) & 15) - 7) * S[k // 32, n], fp16 [K, N].  numpy restatement."""
    W_kn = _c(W_kn, np.uint32)
    S_kn = _c(S_kn, np.float16)
    k8, N = W_kn.shape
    K = k8 * 8
    k = np.arange(K)
    q = (W_kn[k // 8, :] >> (4 * (k % 8)).astype(np.uint32)[:, None]) & np.uint32(15)
    return (q.astype(np.float16) - np.float16(7)) * S_kn[k // 32, :]


def q4g32_kn_linear(W_kn: np.ndarray, S_kn: np.ndarray, x: np.ndarray) -> np.ndarray:
    """y[m, n] = sum_k x[m, k] * B[k, n], float32 accumulation over the fp16 weights, fp16 result
    (test_gpu_reduction.py:121-128 with the accumulate mode the build implements)."""
    B = q4g32_kn_dequant(W_kn, S_kn).astype(np.float32)
    x = _c(x, np.float16).astype(np.float32)
    return (x.reshape(-1, x.shape[-1]) @ B).astype(np.float16)


# ------------------------------------------------- synthetic inputs (shared)


def make_q4g32_inputs(M: int, N: int, K: int, seed: int):
    """Inputs with the distributions the benchmark configuration names:
    x ~ N(0,1) fp16, codes uniform 0..15 packed 8 per uint32 along K,
    scales ~ U(0.005, 0.02) fp16."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
    W = rng.integers(0, 2**32, size=(N, K // 8), dtype=np.uint64).astype(np.uint32)
    S = rng.uniform(0.005, 0.02, size=(N, K // 32)).astype(np.float16)
    return x, W, S


def make_intb_inputs(M: int, N: int, K: int, nbit: int, seed: int, group_size: int = -1):
    """x ~ N(0,1) fp16; int8 codes uniform -127..127 laid out [K,N] (int4: -8..7 packed two per
    byte along N, low nibble = even n); per-channel scales ~ U(0.001, 0.01) fp16."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
    if nbit == 8:
        A = rng.integers(-127, 128, size=(K, N), dtype=np.int64).astype(np.int8)
    else:
        q = rng.integers(-8, 8, size=(K, N), dtype=np.int64)
        A = ((q[:, 0::2] & 15) | ((q[:, 1::2] & 15) << 4)).astype(np.uint8).view(np.int8)
    shape = (N,) if group_size <= 0 else (K // group_size, N)
    s = rng.uniform(0.001, 0.01, size=shape).astype(np.float16)
    return x, A, s


# ------------------------------------------------- AutoGPTQ layout (K-major, zero points, g_idx)


def gptq_dequant(qweight: np.ndarray, qzeros: np.ndarray, scales: np.ndarray, g_idx: np.ndarray) -> np.ndarray:
    """B[k, n] = (fp16(code) - (fp16(zero) + 1)) * scales[g_idx[k], n], fp16 [K, N]
    (tests/python/dlight/test_gpu_gemv.py:636-652).  qweight uint32 [K/8, N], qzeros uint32 [G, N/8],
    scales fp16 [G, N], g_idx int32 [K]."""
    qweight = _c(qweight, np.uint32)
    qzeros = _c(qzeros, np.uint32)
    scales = _c(scales, np.float16)
    g_idx = _c(g_idx, np.int32)
    k8, N = qweight.shape
    K, G = k8 * 8, scales.shape[0]
    assert qzeros.shape == (G, N // 8) and scales.shape == (G, N) and g_idx.shape == (K,)
    out = np.empty((K, N), np.float16)
    rc = lib().wqo_gptq_dequant(_p(qweight), _p(qzeros), _p(scales.view(np.uint16)), _p(g_idx),
                                _p(out.view(np.uint16)), i64(K), i64(N), i64(G))
    if rc != 0:
        raise ValueError("g_idx entry outside [0, G)")
    return out


def kn_matmul(Bdeq: np.ndarray, x: np.ndarray, residual=None, f32acc: bool = True) -> np.ndarray:
    """y[m, n] = residual[m, n] + sum_k x[m, k] * B[k, n] (test_gpu_gemv.py:653-665); ``f32acc=False`` is the
    reference's fp16 accumulation, ``True`` the fp32 accumulation the GPU build implements."""
    Bdeq = _c(Bdeq, np.float16)
    x = _c(x, np.float16)
    K, N = Bdeq.shape
    x2 = x.reshape(-1, K)
    M = x2.shape[0]
    res = None if residual is None else _c(residual, np.float16).reshape(M, N)
    y = np.empty((M, N), np.float16)
    lib().wqo_kn_matmul(_p(Bdeq.view(np.uint16)), _p(x2.view(np.uint16)),
                        _opt(None if res is None else res.view(np.uint16)), _p(y.view(np.uint16)),
                        i64(M), i64(N), i64(K), cint(1 if f32acc else 0))
    return y


def gptq_linear(qweight, qzeros, scales, g_idx, x, residual=None, f32acc: bool = True) -> np.ndarray:
    return kn_matmul(gptq_dequant(qweight, qzeros, scales, g_idx), x, residual, f32acc)


def make_gptq_inputs(M: int, N: int, K: int, group_size: int, seed: int, act_order: bool = False):
    """x ~ N(0,1) fp16; codes and zero points uniform 0..15; scales ~ U(0.005, 0.02) fp16;
    g_idx[k] = k // group_size, or (``act_order``) a random permutation of that assignment, which is
    what AutoGPTQ's desc_act option produces: every group keeps exactly ``group_size`` members."""
    rng = np.random.default_rng(seed)
    G = K // group_size
    x = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
    qweight = rng.integers(0, 2**32, size=(K // 8, N), dtype=np.uint64).astype(np.uint32)
    qzeros = rng.integers(0, 2**32, size=(G, N // 8), dtype=np.uint64).astype(np.uint32)
    scales = rng.uniform(0.005, 0.02, size=(G, N)).astype(np.float16)
    g_idx = (np.arange(K) // group_size).astype(np.int32)
    if act_order:
        g_idx = g_idx[rng.permutation(K)]
    return x, qweight, qzeros, scales, np.ascontiguousarray(g_idx)
