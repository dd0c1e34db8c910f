"""MI355X-native weight-only quantized linear path (q4f16_1 group-quant and fpA_intB).

The compute lives in ``librelax_amd_wq.so`` (hand-written HIP for gfx950) behind the C ABI
of ``include/relax_amd_wq.h``; :mod:`relax_amd.ops` is a thin torch-tensor front end that
passes device pointers through ctypes.
"""
from . import _lib  # noqa: F401

__all__ = ["_lib"]
