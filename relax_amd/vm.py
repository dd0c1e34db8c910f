"""Instruction-list executor for the library's PackedFuncs (``include/relax_amd_vm.h``) with torch tensors.

Mirrors what a built Relax module does around the quantized linears: every op is a
``call_dps_packed`` (src/runtime/relax_vm/vm.cc:691-775), intermediates live in one planned
workspace (StaticPlanBlockMemory) and the whole list is replayed as one HIP graph
(RewriteCUDAGraph, python/tvm/relax/pipeline.py:90-91).
"""
from __future__ import annotations

import ctypes
from typing import Dict, List, Sequence, Tuple, Union

import torch

from . import _lib
from ._lib import check

_DTYPES = {torch.float16: (2, 16), torch.float32: (2, 32), torch.int8: (0, 8), torch.uint8: (1, 8),
           torch.int32: (0, 32), torch.int64: (0, 64)}
kDLCPU, kDLROCM = 1, 10


class Reg(int):
    """A tensor register of a :class:`DpsProgram`."""


class DpsProgram:
    def __init__(self):
        self._l = _lib.lib()
        self._p = self._l.wq_program_create()
        self._keep: Dict[int, torch.Tensor] = {}  # register -> the tensor that owns its storage
        self._shapes: Dict[int, Tuple[Tuple[int, ...], torch.dtype]] = {}
        self._workspace = None

    def __del__(self):
        if getattr(self, "_p", None):
            self._l.wq_program_destroy(self._p)
            self._p = None

    # ---- registers ----
    def external(self, t: torch.Tensor, as_uint32: bool = False) -> Reg:
        """A tensor that owns its storage (weights, inputs, kept outputs).  ``as_uint32`` declares an
        int32 tensor as uint32 (torch has no uint32 arithmetic; the bytes are the same)."""
        if not t.is_contiguous():
            raise ValueError("tensors must be contiguous")
        code, bits = _DTYPES[t.dtype]
        if as_uint32:
            if t.dtype != torch.int32:
                raise ValueError("as_uint32 needs an int32 tensor")
            code = 1
        shape = (ctypes.c_int64 * max(1, t.dim()))(*t.shape)
        r = self._l.wq_program_add_external(self._p, code, bits, t.dim(), shape, t.data_ptr(),
                                            kDLROCM if t.is_cuda else kDLCPU)
        check(min(r, 0), "wq_program_add_external")
        self._keep[r] = t
        self._shapes[r] = (tuple(t.shape), t.dtype)
        return Reg(r)

    def planned(self, shape: Sequence[int], dtype: torch.dtype = torch.float16, as_uint32: bool = False) -> Reg:
        """An intermediate whose storage the memory plan assigns (``as_uint32``: declare int32 as uint32)."""
        code, bits = _DTYPES[dtype]
        if as_uint32:
            if dtype != torch.int32:
                raise ValueError("as_uint32 needs dtype int32")
            code = 1
        shp = (ctypes.c_int64 * max(1, len(shape)))(*shape)
        r = self._l.wq_program_add_planned(self._p, code, bits, len(shape), shp)
        check(min(r, 0), "wq_program_add_planned")
        self._shapes[r] = (tuple(shape), dtype)
        return Reg(r)

    def rebind(self, reg: Reg, t: torch.Tensor) -> None:
        shape, dtype = self._shapes[int(reg)]
        if tuple(t.shape) != shape or t.dtype != dtype or not t.is_contiguous():
            raise ValueError("rebind needs a contiguous tensor of the declared shape and dtype")
        check(self._l.wq_program_rebind(self._p, int(reg), t.data_ptr()), "wq_program_rebind")
        self._keep[int(reg)] = t  # the previous tensor of this register is released

    # ---- instructions ----
    def call(self, func: str, *args: Union[Reg, int, None]) -> None:
        """``call_dps_packed(func, inputs..., outputs...)``; ``Reg`` arguments are tensors, plain ints immediates,
        ``None`` a null handle (an optional tensor that is absent)."""
        n = len(args)
        vals = (ctypes.c_int64 * max(1, n))(*[0 if a is None else int(a) for a in args])
        kinds = (ctypes.c_int * max(1, n))(*[2 if a is None else 1 if isinstance(a, Reg) else 0 for a in args])
        check(self._l.wq_program_add_call(self._p, func.encode(), n, vals, kinds), f"wq_program_add_call({func})")

    # ---- memory plan ----
    def plan(self, device: str = "cuda") -> int:
        """Plans the workspace, allocates it (once, here — never while running) and returns its size in bytes."""
        need = self._l.wq_program_plan(self._p)
        check(min(need, 0), "wq_program_plan")
        self._workspace = torch.zeros(max(need, 256), dtype=torch.uint8, device=device)
        # the fill runs on torch's current stream, the program on whatever stream run / capture are given
        torch.cuda.current_stream().synchronize()
        check(self._l.wq_program_set_workspace(self._p, self._workspace.data_ptr(), self._workspace.numel()),
              "wq_program_set_workspace")
        return int(need)

    @property
    def unplanned_bytes(self) -> int:
        return int(self._l.wq_program_unplanned_bytes(self._p))

    @property
    def num_instructions(self) -> int:
        return int(self._l.wq_program_num_instructions(self._p))

    # ---- fused decode linears ----
    def set_option(self, name: str, value: int) -> None:
        """``fuse_decode`` (default 1): run consecutive decode linears as one launch; set before :meth:`plan`.
        ``spin_limit_us``: the longest a fused run may wait for a producer linear (default 2 s)."""
        check(self._l.wq_program_set_option(self._p, name.encode(), int(value)), "wq_program_set_option")

    @property
    def num_fused_groups(self) -> int:
        return int(self._l.wq_program_num_fused_groups(self._p))

    def fused_order(self, group: int = 0) -> List[int]:
        n = self._l.wq_program_fused_order(self._p, group, (ctypes.c_int * 1)(), 0)
        check(min(n, 0), "wq_program_fused_order")
        buf = (ctypes.c_int * max(1, n))()
        self._l.wq_program_fused_order(self._p, group, buf, n)
        return list(buf[:n])

    def status(self, stream: torch.cuda.Stream = None) -> None:
        """Synchronises and raises if a device-side wait of a fused run timed out."""
        s = (stream or torch.cuda.current_stream()).cuda_stream
        check(self._l.wq_program_status(self._p, s), "wq_program_status")

    def poll(self, words: torch.Tensor, stream: torch.cuda.Stream = None) -> int:
        """Asynchronous copies of the fused runs' error words into ``words`` (pinned int32 host tensor), no
        synchronisation; returns the number of fused runs.  All zero once the stream has passed: no wait ran out."""
        if words.dtype != torch.int32 or words.is_cuda or not words.is_pinned():
            raise ValueError("words must be a pinned int32 host tensor")
        s = (stream or torch.cuda.current_stream()).cuda_stream
        n = int(self._l.wq_program_poll(self._p, words.data_ptr(), int(words.numel()), s))
        if n < 0:
            check(n, "wq_program_poll")
        return n

    # ---- execution ----
    def run(self, stream: torch.cuda.Stream = None) -> None:
        s = (stream or torch.cuda.current_stream()).cuda_stream
        check(self._l.wq_program_run(self._p, s), "wq_program_run")

    def capture(self, stream: torch.cuda.Stream) -> None:
        check(self._l.wq_program_capture(self._p, stream.cuda_stream), "wq_program_capture")

    def replay(self, stream: torch.cuda.Stream) -> None:
        check(self._l.wq_program_replay(self._p, stream.cuda_stream), "wq_program_replay")


# The four quantized linears of one Llama-2-7B decoder layer, as (name, N, K).
LLAMA7B_LINEARS = (("qkv_proj", 12288, 4096), ("o_proj", 4096, 4096), ("gate_up_proj", 22016, 4096),
                   ("down_proj", 4096, 11008))


def llama_linear_stack(weights, M: int, hidden: torch.Tensor, attn_out: torch.Tensor, mlp_act: torch.Tensor,
                       out: torch.Tensor, linears=LLAMA7B_LINEARS, taps=None) -> DpsProgram:
    """Program of ``len(weights)`` decoder layers' quantized linears (q4f16_1), batch ``M``.

    ``weights[l][name] = (W int32 [N, K/8], S fp16 [N, K/32])``.  Only the linears are present, so two
    inputs stand in for what the missing ops would produce: ``attn_out`` [M, 4096] feeds every o_proj
    and ``mlp_act`` [M, 11008] every down_proj.  ``hidden`` [M, 4096] enters layer 0; each layer's
    down_proj output is the next layer's hidden state; the last one lands in ``out``.
    ``taps`` maps ``(layer, name)`` to a tensor [M, N] that receives that linear's output instead of
    planned storage (to look at an intermediate of the stack).
    """
    taps = taps or {}

    def dest(l, name):
        t = taps.get((l, name))
        return p.external(t) if t is not None else p.planned((M, dims[name][0]))

    p = DpsProgram()
    h = p.external(hidden)
    a = p.external(attn_out)
    g = p.external(mlp_act)
    dims = {name: (n, k) for name, n, k in linears}
    L = len(weights)
    for l, layer in enumerate(weights):
        regs = {name: (p.external(w, as_uint32=True), p.external(s)) for name, (w, s) in layer.items()}
        qkv = dest(l, "qkv_proj")
        p.call("relax_amd.q4f16_1_matmul", *regs["qkv_proj"], h, qkv)
        o = dest(l, "o_proj")
        p.call("relax_amd.q4f16_1_matmul", *regs["o_proj"], a, o)
        gu = dest(l, "gate_up_proj")
        p.call("relax_amd.q4f16_1_matmul", *regs["gate_up_proj"], o, gu)
        nxt = p.external(out) if l == L - 1 else dest(l, "down_proj")
        p.call("relax_amd.q4f16_1_matmul", *regs["down_proj"], g, nxt)
        h = nxt
    return p


def llama_autogptq_stack(weights, hidden: torch.Tensor, attn_out: torch.Tensor, mlp_act: torch.Tensor,
                         out: torch.Tensor, linears=LLAMA7B_LINEARS) -> DpsProgram:
    """:func:`llama_linear_stack` for AutoGPTQ layers at one row of activations: ``weights[l][name]`` is a
    prepared layer (``ops.GptqWeight`` from ``ops.gptq_prepare``, with or without a row order); every linear is a
    ``relax_amd.autogptq_matmul`` call without residual, and a layer with a row order gets a planned gather
    workspace (which a fused run does not use)."""
    from . import ops

    p = DpsProgram()
    h = p.external(hidden)
    a = p.external(attn_out)
    g = p.external(mlp_act)
    dims = {name: (n, k) for name, n, k in linears}
    L = len(weights)

    def call(w, x, y):
        regs = (p.external(w.W_nk, as_uint32=True), p.external(w.SZ), p.external(w.perm) if w.perm is not None else None)
        if w.perm is not None:
            p.call("relax_amd.autogptq_matmul", *regs, x, None, y, p.planned((ops.gptq_workspace_bytes(1, w.K, True),), torch.uint8))
        else:
            p.call("relax_amd.autogptq_matmul", *regs, x, None, y)

    for l, layer in enumerate(weights):
        qkv = p.planned((1, dims["qkv_proj"][0]))
        call(layer["qkv_proj"], h, qkv)
        o = p.planned((1, dims["o_proj"][0]))
        call(layer["o_proj"], a, o)
        gu = p.planned((1, dims["gate_up_proj"][0]))
        call(layer["gate_up_proj"], o, gu)
        nxt = p.external(out) if l == L - 1 else p.planned((1, dims["down_proj"][0]))
        call(layer["down_proj"], g, nxt)
        h = nxt
    return p
