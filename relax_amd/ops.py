"""torch-tensor front end of the C ABI.

torch is used for device memory and streams only: every function validates its
arguments, takes ``data_ptr()`` of each tensor and calls the C entry point on
torch's current stream.  Argument names and orders follow the reference's
PrimFuncs / PackedFuncs:

* format A: ``(W uint32[N,K/8], S fp16[N,K/32], x fp16[...,K]) -> y fp16[...,N]``
  (tests/python/dlight/test_gpu_gemv.py:189, test_gpu_low_batch_gemv.py:30-34)
* format B: ``(x, w_preprocessed, scales, [bias], [residual]) -> out``
  (tests/python/relax/test_codegen_cutlass.py:1474-1520)
* AutoGPTQ: ``(qweight uint32[K/8,N], qzeros uint32[G,N/8], scales fp16[G,N], g_idx int32[K], x, residual) -> y``
  (tests/python/dlight/test_gpu_gemv.py:636-665)
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib
from ._lib import check

ACTIVATIONS = {"identity": 0, "relu": 1, "silu": 2, "gelu": 3}
BINARY_OPS = {"none": 0, "plus": 1, "multiply": 2}
UNARY_OPS = {"identity": 0, "relu": 1}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, dtype, name: str) -> torch.Tensor:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise ValueError(f"{name} must be a device tensor")
    if t.dtype != dtype:
        raise ValueError(f"{name} must have dtype {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be compact (contiguous)")
    return t


def _ptr(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


# torch has no uint32 arithmetic; packed weights may arrive as int32 or uint32 (same bytes)
def _w32(W: torch.Tensor) -> torch.Tensor:
    if W.dtype not in (torch.int32, torch.uint32):
        raise ValueError(f"packed weight must be 32-bit integers, got {W.dtype}")
    return _dev(W, W.dtype, "W")


# ----------------------------------------------------------------- format A


def q4_unpack(W: torch.Tensor) -> torch.Tensor:
    """codes uint8 [N, K] of a packed ``uint32 [N, K/8]`` weight."""
    W = _w32(W)
    N, kw = W.shape
    q = torch.empty((N, kw * 8), dtype=torch.uint8, device=W.device)
    check(_lib.lib().wq_q4_unpack(_ptr(W), _ptr(q), N, kw * 8, _stream()), "wq_q4_unpack")
    return q


def q4g32_dequantize(W: torch.Tensor, S: torch.Tensor) -> torch.Tensor:
    """fp16 [N, K] dequantized weight, bit-identical to the reference's ``decode`` block."""
    W = _w32(W)
    S = _dev(S, torch.float16, "S")
    N, kw = W.shape
    K = kw * 8
    if tuple(S.shape) != (N, K // 32) or K % 32:
        raise ValueError(f"S must be [N, K/32] = [{N}, {K // 32}], got {tuple(S.shape)}")
    out = torch.empty((N, K), dtype=torch.float16, device=W.device)
    check(_lib.lib().wq_q4g32_dequantize(_ptr(W), _ptr(S), _ptr(out), N, K, _stream()), "wq_q4g32_dequantize")
    return out


def q4g32_linear(W: torch.Tensor, S: torch.Tensor, x: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                 kernel: str = "auto") -> torch.Tensor:
    """``y[..., n] = sum_k x[..., k] * dequant(W, S)[n, k]`` (+bias, +residual), fp32 accumulate.

    ``kernel``: "auto" (by M), "gemv" or "gemm".  ``out`` makes the call destination-passing.
    """
    W = _w32(W)
    S = _dev(S, torch.float16, "S")
    x = _dev(x, torch.float16, "x")
    N, kw = W.shape
    K = kw * 8
    if x.shape[-1] != K:
        raise ValueError(f"x last dim {x.shape[-1]} != K {K}")
    if K % 32 or tuple(S.shape) != (N, K // 32):
        raise ValueError(f"S must be [N, K/32] = [{N}, {K // 32}], got {tuple(S.shape)}")
    M = x.numel() // K if K else 0
    oshape = tuple(x.shape[:-1]) + (N,)
    if bias is not None:
        bias = _dev(bias, torch.float16, "bias")
        if bias.numel() != N:
            raise ValueError("bias must have N elements")
    if residual is not None:
        residual = _dev(residual, torch.float16, "residual")
        if residual.numel() != M * N:
            raise ValueError("residual must have M*N elements")
    if out is None:
        out = torch.empty(oshape, dtype=torch.float16, device=x.device)
    else:
        out = _dev(out, torch.float16, "out")
        if out.numel() != M * N:
            raise ValueError("out must have M*N elements")
    fn = {"auto": _lib.lib().wq_q4g32_linear, "gemv": _lib.lib().wq_q4g32_gemv,
          "gemm": _lib.lib().wq_q4g32_gemm, "small_batch": _lib.lib().wq_q4g32_small_batch}[kernel]
    check(fn(_ptr(W), _ptr(S), _ptr(x), _ptr(bias), _ptr(residual), _ptr(out), M, N, K, _stream()),
          f"wq_q4g32_{kernel}")
    return out


def q4g32_gemv_f16acc(W: torch.Tensor, S: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """The decode GEMV with fp16 accumulation (the reference's `NT_matmul += x * decode` with every
    buffer fp16: tests/python/dlight/test_gpu_reduction.py:44-51): each product and each partial sum
    is rounded to fp16; the sum is a tree (per lane, then over the wavefront)."""
    W = _w32(W)
    S = _dev(S, torch.float16, "S")
    x = _dev(x, torch.float16, "x")
    N, kw = W.shape
    K = kw * 8
    if x.shape[-1] != K:
        raise ValueError(f"x last dim {x.shape[-1]} != K {K}")
    if K % 32 or tuple(S.shape) != (N, K // 32):
        raise ValueError(f"S must be [N, K/32] = [{N}, {K // 32}], got {tuple(S.shape)}")
    M = x.numel() // K if K else 0
    out = torch.empty(tuple(x.shape[:-1]) + (N,), dtype=torch.float16, device=x.device)
    check(_lib.lib().wq_q4g32_gemv_f16acc(_ptr(W), _ptr(S), _ptr(x), _ptr(out), M, N, K, _stream()),
          "wq_q4g32_gemv_f16acc")
    return out


class GemvDesc(ctypes.Structure):
    """``wq_q4g32_gemv_desc`` of include/relax_amd_wq.h."""
    _fields_ = [("W", ctypes.c_void_p), ("S", ctypes.c_void_p), ("x", ctypes.c_void_p), ("bias", ctypes.c_void_p),
                ("residual", ctypes.c_void_p), ("y", ctypes.c_void_p), ("N", ctypes.c_int64), ("K", ctypes.c_int64)]


class Q4G32GemvList:
    """A list of decode linears (M = 1 each) run as ONE launch (``wq_q4g32_gemv_list_*``).

    ``linears``: sequence of ``(W, S, x, y)`` or ``(W, S, x, y, bias, residual)`` device tensors; a linear
    whose ``x`` is the ``y`` of an earlier one waits for it on the device.  The tensors are kept alive by
    this object; the descriptor table and the counters live in a workspace allocated here, once.
    ``M`` (1 .. 32): rows of activations of every linear of the list (x ``[M, K]``, y and residual ``[M, N]``).
    """

    def __init__(self, linears, M: int = 1):
        self._l = _lib.lib()
        n = len(linears)
        arr = (GemvDesc * max(1, n))()
        self._keep = []
        for i, lin in enumerate(linears):
            W, S, x, y = lin[:4]
            bias = lin[4] if len(lin) > 4 else None
            residual = lin[5] if len(lin) > 5 else None
            W = _w32(W)
            S = _dev(S, torch.float16, "S")
            x = _dev(x, torch.float16, "x")
            y = _dev(y, torch.float16, "y")
            N, kw = W.shape
            K = kw * 8
            if K % 32 or tuple(S.shape) != (N, K // 32):
                raise ValueError(f"linear {i}: S must be [N, K/32] = [{N}, {K // 32}], got {tuple(S.shape)}")
            if x.numel() != M * K or y.numel() != M * N:
                raise ValueError(f"linear {i}: x must hold M*K={M * K} and y M*N={M * N} elements")
            for t, name, want in ((bias, "bias", N), (residual, "residual", M * N)):
                if t is not None and _dev(t, torch.float16, name).numel() != want:
                    raise ValueError(f"linear {i}: {name} must hold {want} elements")
            arr[i] = GemvDesc(_ptr(W), _ptr(S), _ptr(x), _ptr(bias), _ptr(residual), _ptr(y), N, K)
            self._keep.append((W, S, x, y, bias, residual))
        need = self._l.wq_q4g32_gemv_list_workspace_bytes(n)
        self._workspace = torch.zeros(max(int(need), 256), dtype=torch.uint8, device="cuda")
        self.M = M
        self._h = self._l.wq_q4g32_gemv_list_create_batched(arr, n, M, self._workspace.data_ptr(),
                                                            self._workspace.numel(), _stream())
        if not self._h:
            raise _lib.WqError("wq_q4g32_gemv_list_create failed: " + self._l.wq_last_error().decode())

    def __del__(self):
        if getattr(self, "_h", None):
            self._l.wq_q4g32_gemv_list_destroy(self._h)
            self._h = None

    def run(self) -> None:
        """One asynchronous launch on torch's current stream."""
        check(self._l.wq_q4g32_gemv_list_run(self._h, _stream()), "wq_q4g32_gemv_list_run")

    def status(self) -> None:
        """Synchronises and raises if a device-side wait of an earlier launch timed out."""
        check(self._l.wq_q4g32_gemv_list_status(self._h, _stream()), "wq_q4g32_gemv_list_status")

    def poll(self, word: torch.Tensor) -> None:
        """Enqueues an asynchronous copy of the error word into ``word`` (a pinned int32 host tensor of one
        element) behind the work on torch's current stream; no synchronisation.  Non-zero once the stream has
        passed: a wait of an earlier launch ran out (then :meth:`status` says which)."""
        if word.dtype != torch.int32 or word.numel() != 1 or word.is_cuda or not word.is_pinned():
            raise ValueError("word must be a pinned int32 host tensor of one element")
        check(self._l.wq_q4g32_gemv_list_poll(self._h, word.data_ptr(), _stream()), "wq_q4g32_gemv_list_poll")

    def info(self):
        """(linears that wait for an earlier one, of which for the one directly in front)."""
        a, b = ctypes.c_int(0), ctypes.c_int(0)
        check(self._l.wq_q4g32_gemv_list_info(self._h, ctypes.byref(a), ctypes.byref(b)), "wq_q4g32_gemv_list_info")
        return a.value, b.value

    def set_spin_limit(self, ticks: int) -> None:
        check(self._l.wq_q4g32_gemv_list_set_spin_limit(self._h, ticks), "wq_q4g32_gemv_list_set_spin_limit")


# ----------------------------------------------------------------- format B


def ft_preprocess_weight(packed_weight: torch.Tensor, sm: int, is_int4: bool) -> torch.Tensor:
    """``cutlass.ft_preprocess_weight(packed_weight, sm, is_int4)``
    (src/runtime/contrib/cutlass/weight_preprocess.cc:38-59): returns a new tensor of the same
    shape, dtype and device holding the reordered weight.  ``packed_weight`` is int8 ``[K, N]``,
    ``[K, N/2]`` (int4) or ``[E, K, N(/2)]``.  Host tensors are reordered on the host, device
    tensors by a device kernel (no round trip through host memory)."""
    w = packed_weight
    if not isinstance(w, torch.Tensor) or w.dtype != torch.int8:
        raise ValueError("packed_weight must be an int8 tensor")
    if w.dim() not in (2, 3):
        raise ValueError("packed_weight must be [K, N] or [E, K, N]")
    if not w.is_contiguous():
        raise ValueError("packed_weight must be compact (contiguous)")
    E = 1 if w.dim() == 2 else w.shape[0]
    rows, cols = w.shape[-2], w.shape[-1] * (2 if is_int4 else 1)
    out = torch.empty_like(w)
    if w.is_cuda:
        check(_lib.lib().wq_ft_preprocess_weight(_ptr(out), _ptr(w), E, rows, cols, int(bool(is_int4)), int(sm),
                                                 _stream()), "wq_ft_preprocess_weight")
    else:
        check(_lib.lib().wq_ft_preprocess_weight_host(_ptr(out), _ptr(w), E, rows, cols, int(bool(is_int4)),
                                                      int(sm)), "wq_ft_preprocess_weight_host")
    return out


def _intb_dims(B: torch.Tensor, nbit: int):
    if nbit not in (4, 8):
        raise ValueError("weight_nbit must be 4 or 8")
    B = _dev(B, torch.int8, "B")
    if B.dim() != 2:
        raise ValueError("B must be [K, N] or [K, N/2]")
    K, c = B.shape
    return B, K, c * (2 if nbit == 4 else 1)


def intb_dequantize(B: torch.Tensor, scales: torch.Tensor, weight_nbit: int, group_size: int = -1) -> torch.Tensor:
    """fp16 ``[K, N]`` dequantized weight from the PREPROCESSED layout, bit-identical to the
    reference's ``decode`` PrimFunc applied to the original packed weight."""
    B, K, N = _intb_dims(B, weight_nbit)
    scales = _dev(scales, torch.float16, "scales")
    want = N if group_size <= 0 or group_size == K else (K // group_size) * N
    if scales.numel() != want:
        raise ValueError(f"scales must have {want} elements, got {scales.numel()}")
    out = torch.empty((K, N), dtype=torch.float16, device=B.device)
    check(_lib.lib().wq_intb_dequantize(_ptr(B), _ptr(scales), _ptr(out), K, N, weight_nbit, group_size, _stream()),
          "wq_intb_dequantize")
    return out


def fpA_intB_gemm(x: torch.Tensor, B: torch.Tensor, scales: torch.Tensor, bias: Optional[torch.Tensor] = None,
                  residual: Optional[torch.Tensor] = None, *, weight_nbit: int, activation: str = "identity",
                  binary_op: str = "plus", unary_op: str = "identity", group_size: int = -1,
                  out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The fused ``decode -> matmul [-> bias] [-> activation] [-> residual op [-> relu]]`` composite
    (python/tvm/relax/backend/contrib/cutlass.py:271-314, 344-372), arguments in the composite's
    order ``(x, w_preprocessed, scales, [bias], [residual])``.  ``m = prod(x.shape[:-1])``,
    ``bias_stride = 0`` for a bias that only varies along N, else ``bias.shape[-1]``
    (python/tvm/contrib/cutlass/build.py:722-734)."""
    B, K, N = _intb_dims(B, weight_nbit)
    x = _dev(x, torch.float16, "x")
    scales = _dev(scales, torch.float16, "scales")
    if x.shape[-1] != K:
        raise ValueError(f"x last dim {x.shape[-1]} != K {K}")
    M = x.numel() // K
    want = N if group_size <= 0 or group_size == K else (K // group_size) * N
    if scales.numel() != want:
        raise ValueError(f"scales must have {want} elements, got {scales.numel()}")
    bias_stride = 0
    if bias is not None:
        bias = _dev(bias, torch.float16, "bias")
        if bias.shape[-1] != N:
            raise ValueError("bias last dim must be N")
        if bias.numel() != N:
            if bias.numel() != M * N:
                raise ValueError("bias must have N or M*N elements")
            bias_stride = N
    if residual is not None:
        residual = _dev(residual, torch.float16, "residual")
        if residual.numel() != M * N:
            raise ValueError("residual must have M*N elements")
    if out is None:
        out = torch.empty(tuple(x.shape[:-1]) + (N,), dtype=torch.float16, device=x.device)
    else:
        out = _dev(out, torch.float16, "out")
        if out.numel() != M * N:
            raise ValueError("out must have M*N elements")
    L = _lib.lib()
    if residual is None:
        check(L.wq_fpA_intB_gemm(_ptr(x), _ptr(B), _ptr(scales), _ptr(bias), _ptr(out), ACTIVATIONS[activation],
                                 M, N, K, group_size, bias_stride, weight_nbit, 0, 0, _stream()), "wq_fpA_intB_gemm")
    else:
        if bias_stride:
            raise ValueError("the residual form takes a bias that only varies along N")
        check(L.wq_fpA_intB_gemm_residual(_ptr(x), _ptr(B), _ptr(scales), _ptr(bias), _ptr(residual), _ptr(out),
                                          ACTIVATIONS[activation], BINARY_OPS[binary_op], UNARY_OPS[unary_op],
                                          M, N, K, group_size, weight_nbit, 0, 0, _stream()),
              "wq_fpA_intB_gemm_residual")
    return out


def intb_encode(Wf: torch.Tensor, weight_nbit: int, group_size: int = -1):
    """The reference fixtures' quantizer (tests/python/relax/test_codegen_cutlass.py:1392-1457, 1631-1676,
    2044-2109): fp16 ``[N, K]`` -> ``(int8 [K, N] | packed int4 [K, N/2], fp16 scales [N] | [K/64, N])``.
    The codes are not yet in the GEMM's layout: pass them through :func:`ft_preprocess_weight`."""
    Wf = _dev(Wf, torch.float16, "Wf")
    if Wf.dim() != 2:
        raise ValueError("Wf must be [N, K]")
    N, K = Wf.shape
    grouped = group_size == 64 and group_size != K
    w = torch.empty((K, N if weight_nbit == 8 else N // 2), dtype=torch.int8, device=Wf.device)
    s = torch.empty((K // 64, N) if grouped else (N,), dtype=torch.float16, device=Wf.device)
    scratch = None if grouped else torch.empty((N,), dtype=torch.float32, device=Wf.device)
    check(_lib.lib().wq_intb_encode(_ptr(Wf), _ptr(w), _ptr(s), _ptr(scratch), N, K, group_size, weight_nbit,
                                    _stream()), "wq_intb_encode")
    return w, s


def q4g32_encode(Wf: torch.Tensor):
    """q4f16_1 quantizer: fp16 ``[N, K]`` -> ``(W int32 [N, K/8] (uint32 bits), S fp16 [N, K/32])``."""
    Wf = _dev(Wf, torch.float16, "Wf")
    if Wf.dim() != 2 or Wf.shape[1] % 32:
        raise ValueError("Wf must be [N, K] with K a multiple of 32")
    N, K = Wf.shape
    W = torch.empty((N, K // 8), dtype=torch.int32, device=Wf.device)
    S = torch.empty((N, K // 32), dtype=torch.float16, device=Wf.device)
    check(_lib.lib().wq_q4g32_encode(_ptr(Wf), _ptr(W), _ptr(S), N, K, _stream()), "wq_q4g32_encode")
    return W, S


def q4g32_kn_to_nk(W_kn: torch.Tensor, S_kn: torch.Tensor):
    """K-major q4f16_1 weights (``W [K/8, N]``, ``S [K/32, N]``; tests/python/dlight/test_gpu_reduction.py:102-120)
    -> the ``[N, K/8]`` / ``[N, K/32]`` layout of :func:`q4g32_linear`.  Run once when a checkpoint is loaded."""
    W_kn = _w32(W_kn)
    S_kn = _dev(S_kn, torch.float16, "S_kn")
    k8, N = W_kn.shape
    K = k8 * 8
    if K % 32 or tuple(S_kn.shape) != (K // 32, N):
        raise ValueError(f"S_kn must be [K/32, N] = [{K // 32}, {N}], got {tuple(S_kn.shape)}")
    W = torch.empty((N, k8), dtype=W_kn.dtype, device=W_kn.device)
    S = torch.empty((N, K // 32), dtype=torch.float16, device=W_kn.device)
    check(_lib.lib().wq_q4g32_kn_to_nk(_ptr(W_kn), _ptr(S_kn), _ptr(W), _ptr(S), N, K, _stream()), "wq_q4g32_kn_to_nk")
    return W, S


KN_GEMV_MAX_M = 16


def q4g32_kn_gemv(W_kn: torch.Tensor, S_kn: torch.Tensor, x: torch.Tensor, bias: Optional[torch.Tensor] = None,
                  residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                  workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The decode linear over a K-major q4f16_1 checkpoint used in place (``W [K/8, N]``, ``S [K/32, N]``;
    tests/python/dlight/test_gpu_reduction.py:102-165), ``M <= 16`` rows.  ``workspace`` (uint8, see
    ``wq_q4g32_kn_gemv_workspace_bytes``) is allocated here when not given."""
    W_kn = _w32(W_kn)
    S_kn = _dev(S_kn, torch.float16, "S_kn")
    x = _dev(x, torch.float16, "x")
    k8, N = W_kn.shape
    K = k8 * 8
    if K % 32 or tuple(S_kn.shape) != (K // 32, N):
        raise ValueError(f"S_kn must be [K/32, N] = [{K // 32}, {N}], got {tuple(S_kn.shape)}")
    if x.shape[-1] != K:
        raise ValueError(f"x last dim {x.shape[-1]} != K {K}")
    M = x.numel() // K if K else 0
    if bias is not None:
        bias = _dev(bias, torch.float16, "bias")
        if bias.numel() != N:
            raise ValueError("bias must have N elements")
    if residual is not None:
        residual = _dev(residual, torch.float16, "residual")
        if residual.numel() != M * N:
            raise ValueError("residual must have M*N elements")
    if out is None:
        out = torch.empty(tuple(x.shape[:-1]) + (N,), dtype=torch.float16, device=x.device)
    else:
        out = _dev(out, torch.float16, "out")
        if out.numel() != M * N:
            raise ValueError("out must have M*N elements")
    L = _lib.lib()
    need = int(L.wq_q4g32_kn_gemv_workspace_bytes(M, N, K))
    if workspace is None and need:
        workspace = torch.empty((need,), dtype=torch.uint8, device=x.device)
    check(L.wq_q4g32_kn_gemv(_ptr(W_kn), _ptr(S_kn), _ptr(x), _ptr(bias), _ptr(residual), _ptr(out), M, N, K,
                             _ptr(workspace), workspace.numel() if workspace is not None else 0, _stream()),
          "wq_q4g32_kn_gemv")
    return out


# ------------------------------------------------------------------ q4f16_1 packed along N


def q4n32_prepare(W: torch.Tensor, S: torch.Tensor):
    """Load-time rearrangement of q4f16_1 weights packed along N (``W`` uint32 ``[K, N/8]``, ``S`` fp16
    ``[K, N/32]``; tests/python/dlight/test_gpu_matmul.py:366-377) for :func:`q4n32_linear`: returns
    ``(W_nk [N, K/8], ST [N/32, K])``."""
    W = _w32(W)
    S = _dev(S, torch.float16, "S")
    K, n8 = W.shape
    N = n8 * 8
    if N % 32 or tuple(S.shape) != (K, N // 32):
        raise ValueError(f"S must be [K, N/32] = [{K}, {N // 32}], got {tuple(S.shape)}")
    W_nk = torch.empty((N, K // 8), dtype=W.dtype, device=W.device)
    ST = torch.empty((N // 32, K), dtype=torch.float16, device=W.device)
    check(_lib.lib().wq_q4n32_prepare(_ptr(W), _ptr(S), _ptr(W_nk), _ptr(ST), K, N, _stream()), "wq_q4n32_prepare")
    return W_nk, ST


def q4n32_linear(W_nk: torch.Tensor, ST: torch.Tensor, x: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``y = residual + fp16(x . w + bias)`` over operands of :func:`q4n32_prepare` (test_gpu_matmul.py:352-401);
    ``x`` fp16 ``[..., K]``."""
    W_nk = _w32(W_nk)
    ST = _dev(ST, torch.float16, "ST")
    x = _dev(x, torch.float16, "x")
    N, K = W_nk.shape[0], W_nk.shape[1] * 8
    if tuple(ST.shape) != (N // 32, K) or x.shape[-1] != K:
        raise ValueError(f"expected ST [N/32, K] = [{N // 32}, {K}] and x [..., {K}]; got {tuple(ST.shape)}, {tuple(x.shape)}")
    M = x.numel() // K if K else 0
    if bias is not None and _dev(bias, torch.float16, "bias").numel() != N:
        raise ValueError("bias must have N elements")
    if residual is not None and _dev(residual, torch.float16, "residual").numel() != M * N:
        raise ValueError("residual must have M*N elements")
    if out is None:
        out = torch.empty((*x.shape[:-1], N), dtype=torch.float16, device=x.device)
    elif not out.is_contiguous() or out.numel() != M * N or out.dtype != torch.float16:
        raise ValueError("out must be a contiguous fp16 tensor of M*N elements")
    check(_lib.lib().wq_q4n32_linear(_ptr(W_nk), _ptr(ST), _ptr(x), _ptr(bias), _ptr(residual), _ptr(out), M, N, K,
                                     _stream()), "wq_q4n32_linear")
    return out


# ------------------------------------------------------------------ AutoGPTQ checkpoints


def _gptq_dims(qweight, qzeros, scales, g_idx):
    qweight, qzeros = _w32(qweight), _w32(qzeros)
    scales = _dev(scales, torch.float16, "scales")
    g_idx = _dev(g_idx, torch.int32, "g_idx")
    k8, N = qweight.shape
    K, G = k8 * 8, scales.shape[0]
    if N % 8 or tuple(qzeros.shape) != (G, N // 8) or tuple(scales.shape) != (G, N) or tuple(g_idx.shape) != (K,):
        raise ValueError(f"expected qzeros [G, N/8], scales [G, N], g_idx [K] for qweight [K/8, N] = [{k8}, {N}]; got "
                         f"{tuple(qzeros.shape)}, {tuple(scales.shape)}, {tuple(g_idx.shape)}")
    return qweight, qzeros, scales, g_idx, K, N, G


def gptq_dequantize(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor,
                    g_idx: torch.Tensor) -> torch.Tensor:
    """fp16 ``[K, N]`` weight of an AutoGPTQ layer, bit for bit
    (tests/python/dlight/test_gpu_gemv.py:636-652): ``(code - (zero + 1)) * scales[g_idx[k], n]``."""
    qweight, qzeros, scales, g_idx, K, N, G = _gptq_dims(qweight, qzeros, scales, g_idx)
    out = torch.empty((K, N), dtype=torch.float16, device=qweight.device)
    check(_lib.lib().wq_gptq_dequantize(_ptr(qweight), _ptr(qzeros), _ptr(scales), _ptr(g_idx), _ptr(out), K, N, G,
                                        _stream()), "wq_gptq_dequantize")
    return out


class GptqWeight:
    """An AutoGPTQ layer converted for :func:`gptq_linear` (see :func:`gptq_prepare`)."""

    def __init__(self, W_nk, SZ, perm, K, N, G):
        self.W_nk, self.SZ, self.perm, self.K, self.N, self.G = W_nk, SZ, perm, K, N, G


def gptq_prepare(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor, g_idx: torch.Tensor) -> GptqWeight:
    """Load-time conversion of an AutoGPTQ layer: rows sorted by group, words transposed to ``[N, K/8]``,
    ``(scale, zero + 1)`` pairs ``[N, G, 2]``.  ``perm`` is kept only when the sorted order is not the identity
    (checkpoints written with ``desc_act``)."""
    qweight, qzeros, scales, g_idx, K, N, G = _gptq_dims(qweight, qzeros, scales, g_idx)
    dev = qweight.device
    W_nk = torch.empty((N, K // 8), dtype=qweight.dtype, device=dev)
    SZ = torch.empty((N, G, 2), dtype=torch.float16, device=dev)
    perm = torch.empty((K,), dtype=torch.int32, device=dev)
    status = torch.empty((1,), dtype=torch.int32, device=dev)
    needs = ctypes.c_int(0)
    check(_lib.lib().wq_gptq_prepare(_ptr(qweight), _ptr(qzeros), _ptr(scales), _ptr(g_idx), _ptr(W_nk), _ptr(SZ),
                                     _ptr(perm), _ptr(status), ctypes.byref(needs), K, N, G, _stream()),
          "wq_gptq_prepare")
    return GptqWeight(W_nk, SZ, perm if needs.value else None, K, N, G)


def gptq_prepare_padded(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor, g_idx: torch.Tensor) -> GptqWeight:
    """:func:`gptq_prepare` for ANY ``g_idx`` (groups of unequal size): every group padded to a multiple of 32
    rows (``wq_gptq_prepare_padded``); the result carries ``K_padded`` and is run by :func:`gptq_linear`."""
    qweight, qzeros, scales, g_idx, K, N, G = _gptq_dims(qweight, qzeros, scales, g_idx)
    dev = qweight.device
    cap = int(_lib.lib().wq_gptq_padded_k_bound(K, G))
    W_nk = torch.empty((N, cap // 8), dtype=qweight.dtype, device=dev)
    SZ = torch.empty((N, cap // 32, 2), dtype=torch.float16, device=dev)
    perm = torch.empty((cap,), dtype=torch.int32, device=dev)
    kp = ctypes.c_int64(0)
    check(_lib.lib().wq_gptq_prepare_padded(_ptr(qweight), _ptr(qzeros), _ptr(scales), _ptr(g_idx), _ptr(W_nk),
                                            _ptr(SZ), _ptr(perm), cap, ctypes.byref(kp), K, N, G, _stream()),
          "wq_gptq_prepare_padded")
    KP = int(kp.value)
    # the prepared operands are compact for K_padded rows (they occupy the front of the buffers)
    w = GptqWeight(W_nk.view(-1)[: N * (KP // 8)].view(N, KP // 8), SZ.view(-1)[: N * (KP // 32) * 2].view(N, KP // 32, 2),
                   perm[:KP], K, N, G)
    w.K_padded = KP
    return w


def gptq_linear(w: GptqWeight, x: torch.Tensor, bias: Optional[torch.Tensor] = None,
                residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``y = residual + fp16(x . w + bias)`` for a prepared AutoGPTQ layer; ``x`` fp16 ``[..., K]``.
    A workspace (uint8, :func:`gptq_workspace_bytes`) is allocated when needed and not given."""
    x = _dev(x, torch.float16, "x")
    if x.shape[-1] != w.K:
        raise ValueError(f"x must end in K={w.K}, got {tuple(x.shape)}")
    M = x.numel() // w.K
    if bias is not None:
        bias = _dev(bias, torch.float16, "bias")
    if residual is not None:
        residual = _dev(residual, torch.float16, "residual")
        if residual.numel() != M * w.N:
            raise ValueError("residual must have M*N elements")
    if out is None:
        out = torch.empty((*x.shape[:-1], w.N), dtype=torch.float16, device=x.device)
    elif not out.is_contiguous() or out.numel() != M * w.N or out.dtype != torch.float16:
        raise ValueError("out must be a contiguous fp16 tensor of M*N elements")
    KP = getattr(w, "K_padded", 0)
    if KP:
        need = _lib.lib().wq_gptq_padded_workspace_bytes(M, KP)
        if workspace is None:
            workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=x.device)
        check(_lib.lib().wq_gptq_linear_padded(_ptr(w.W_nk), _ptr(w.SZ), _ptr(w.perm), _ptr(x), _ptr(bias),
                                               _ptr(residual), _ptr(out), M, w.N, w.K, KP, _ptr(workspace),
                                               workspace.numel() * workspace.element_size(), _stream()),
              "wq_gptq_linear_padded")
        return out
    need = _lib.lib().wq_gptq_workspace_bytes(M, w.K, 1 if w.perm is not None else 0)
    if need and workspace is None:
        workspace = torch.empty((need,), dtype=torch.uint8, device=x.device)
    check(_lib.lib().wq_gptq_linear(_ptr(w.W_nk), _ptr(w.SZ), _ptr(w.perm), _ptr(x), _ptr(bias), _ptr(residual),
                                    _ptr(out), M, w.N, w.K, w.G, _ptr(workspace),
                                    0 if workspace is None else workspace.numel() * workspace.element_size(),
                                    _stream()), "wq_gptq_linear")
    return out


def gptq_workspace_bytes(M: int, K: int, has_perm: bool) -> int:
    return int(_lib.lib().wq_gptq_workspace_bytes(M, K, 1 if has_perm else 0))


class GptqGemvDesc(ctypes.Structure):
    """``wq_gptq_gemv_desc`` of include/relax_amd_wq.h."""
    _fields_ = [("W_nk", ctypes.c_void_p), ("SZ", ctypes.c_void_p), ("perm", ctypes.c_void_p), ("x", ctypes.c_void_p), ("bias", ctypes.c_void_p),
                ("residual", ctypes.c_void_p), ("y", ctypes.c_void_p), ("N", ctypes.c_int64), ("K", ctypes.c_int64),
                ("G", ctypes.c_int64)]


class GptqGemvList(Q4G32GemvList):
    """A list of prepared AutoGPTQ layers at M = 1 run as ONE launch (``wq_gptq_gemv_list_create``; run, status,
    poll, info as :class:`Q4G32GemvList`).

    ``linears``: sequence of ``(w, x, y)`` or ``(w, x, y, bias, residual)`` with ``w`` a :class:`GptqWeight` from
    :func:`gptq_prepare` (with or without a row order; not :func:`gptq_prepare_padded`)."""

    def __init__(self, linears, gather_in_front: bool = True):
        """``gather_in_front=False`` gives the list the plain workspace only, so that every row order is applied
        inside the list kernel (otherwise layers whose x comes from outside the list are gathered by a small kernel
        launched in front of it)."""
        self._l = _lib.lib()
        n = len(linears)
        arr = (GptqGemvDesc * max(1, n))()
        self._keep = []
        for i, lin in enumerate(linears):
            w, x, y = lin[:3]
            bias = lin[3] if len(lin) > 3 else None
            residual = lin[4] if len(lin) > 4 else None
            if getattr(w, "K_padded", 0):
                raise ValueError(f"linear {i}: a layer prepared with padded groups cannot be a member of a list")
            x = _dev(x, torch.float16, "x")
            y = _dev(y, torch.float16, "y")
            if x.numel() != w.K or y.numel() != w.N:
                raise ValueError(f"linear {i}: x must hold K={w.K} and y N={w.N} elements")
            for t, name in ((bias, "bias"), (residual, "residual")):
                if t is not None and _dev(t, torch.float16, name).numel() != w.N:
                    raise ValueError(f"linear {i}: {name} must hold {w.N} elements")
            arr[i] = GptqGemvDesc(_ptr(w.W_nk), _ptr(w.SZ), _ptr(w.perm), _ptr(x), _ptr(bias), _ptr(residual), _ptr(y), w.N, w.K, w.G)
            self._keep.append((w, x, y, bias, residual))
        need = (self._l.wq_gptq_gemv_list_workspace_bytes(arr, n) if gather_in_front
                else self._l.wq_q4g32_gemv_list_workspace_bytes(n))
        self._workspace = torch.zeros(max(int(need), 256), dtype=torch.uint8, device="cuda")
        self.M = 1
        self._h = self._l.wq_gptq_gemv_list_create(arr, n, self._workspace.data_ptr(), self._workspace.numel(), _stream())
        if not self._h:
            raise _lib.WqError("wq_gptq_gemv_list_create failed: " + self._l.wq_last_error().decode())
