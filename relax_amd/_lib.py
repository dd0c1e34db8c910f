"""Loads ``librelax_amd_wq.so`` and declares the C ABI of ``include/relax_amd_wq.h`` and ``include/relax_amd_vm.h``.

There is no fallback: if the library is missing or a symbol is absent the import
fails with an error that says how to build it.
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "librelax_amd_wq.so")

_i64, _int, _vp, _sz = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t

# name -> argument types (all return int unless listed in _RESTYPES)
SIGNATURES = {
    "wq_last_error": [],
    "wq_abi_version": [],
    "wq_target_arch": [],
    "wq_q4_unpack": [_vp, _vp, _i64, _i64, _vp],
    "wq_q4g32_dequantize": [_vp, _vp, _vp, _i64, _i64, _vp],
    "wq_q4g32_linear": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "wq_q4g32_gemv": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "wq_q4g32_gemm": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "wq_q4g32_small_batch": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "wq_q4g32_gemv_f16acc": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "wq_q4g32_gemv_list_workspace_bytes": [_int],
    "wq_q4g32_gemv_list_create": [_vp, _int, _vp, _sz, _vp],
    "wq_q4g32_gemv_list_create_batched": [_vp, _int, _int, _vp, _sz, _vp],
    "wq_gptq_gemv_list_create": [_vp, _int, _vp, _sz, _vp],
    "wq_gptq_gemv_list_workspace_bytes": [_vp, _int],
    "wq_q4g32_gemv_list_run": [_vp, _vp],
    "wq_q4g32_gemv_list_status": [_vp, _vp],
    "wq_q4g32_gemv_list_poll": [_vp, _vp, _vp],
    "wq_q4g32_gemv_list_destroy": [_vp],
    "wq_q4g32_gemv_list_info": [_vp, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)],
    "wq_q4g32_gemv_list_set_spin_limit": [_vp, ctypes.c_longlong],
    "wq_ft_preprocess_weight_host": [_vp, _vp, _i64, _i64, _i64, _int, _int],
    "wq_ft_preprocess_weight": [_vp, _vp, _i64, _i64, _i64, _int, _int, _vp],
    "wq_intb_dequantize": [_vp, _vp, _vp, _i64, _i64, _int, _i64, _vp],
    "wq_fpA_intB_gemm": [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _i64, _int, _vp, _sz, _vp],
    "wq_fpA_intB_gemm_residual": [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _i64, _i64, _i64, _i64, _int, _vp, _sz, _vp],
    "wq_q4g32_kn_to_nk": [_vp, _vp, _vp, _vp, _i64, _i64, _vp],
    "wq_q4g32_kn_gemv_workspace_bytes": [_i64, _i64, _i64],
    "wq_q4g32_kn_gemv": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp],
    "wq_q4n32_prepare": [_vp, _vp, _vp, _vp, _i64, _i64, _vp],
    "wq_q4n32_linear": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "wq_gptq_dequantize": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "wq_gptq_prepare": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.POINTER(ctypes.c_int), _i64, _i64, _i64, _vp],
    "wq_gptq_workspace_bytes": [_i64, _i64, _int],
    "wq_gptq_padded_k_bound": [_i64, _i64],
    "wq_gptq_prepare_padded": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, ctypes.POINTER(_i64), _i64, _i64, _i64, _vp],
    "wq_gptq_padded_workspace_bytes": [_i64, _i64],
    "wq_gptq_linear_padded": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _sz, _vp],
    "wq_gptq_linear": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _sz, _vp],
    "wq_gptq_linear_noalloc": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "wq_intb_encode": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp],
    "wq_q4g32_encode": [_vp, _vp, _vp, _i64, _i64, _vp],
    "wq_program_create": [],
    "wq_program_destroy": [_vp],
    "wq_program_add_external": [_vp, _int, _int, _int, ctypes.POINTER(_i64), _vp, _int],
    "wq_program_add_planned": [_vp, _int, _int, _int, ctypes.POINTER(_i64)],
    "wq_program_rebind": [_vp, _int, _vp],
    "wq_program_add_call": [_vp, ctypes.c_char_p, _int, ctypes.POINTER(_i64), ctypes.POINTER(_int)],
    "wq_program_plan": [_vp],
    "wq_program_unplanned_bytes": [_vp],
    "wq_program_set_workspace": [_vp, _vp, _i64],
    "wq_program_run": [_vp, _vp],
    "wq_program_capture": [_vp, _vp],
    "wq_program_replay": [_vp, _vp],
    "wq_program_num_instructions": [_vp],
    "wq_program_set_option": [_vp, ctypes.c_char_p, _int],
    "wq_program_num_fused_groups": [_vp],
    "wq_program_fused_order": [_vp, _int, ctypes.POINTER(_int), _int],
    "wq_program_status": [_vp, _vp],
    "wq_program_unfused_reason": [_vp, _int],
    "wq_program_poll": [_vp, _vp, _int, _vp],
    "wq_activation_from_string": [ctypes.c_char_p],
    "wq_binary_op_from_string": [ctypes.c_char_p],
    "wq_unary_op_from_string": [ctypes.c_char_p],
}
_RESTYPES = {"wq_program_unfused_reason": ctypes.c_char_p, "wq_last_error": ctypes.c_char_p, "wq_target_arch": ctypes.c_char_p, "wq_program_create": _vp,
             "wq_program_destroy": None, "wq_program_plan": _i64, "wq_program_unplanned_bytes": _i64,
             "wq_gptq_workspace_bytes": _sz, "wq_q4g32_kn_gemv_workspace_bytes": _sz, "wq_gptq_padded_workspace_bytes": _sz, "wq_gptq_padded_k_bound": _i64, "wq_q4g32_gemv_list_workspace_bytes": _sz,
             "wq_q4g32_gemv_list_create": _vp, "wq_q4g32_gemv_list_create_batched": _vp, "wq_gptq_gemv_list_create": _vp, "wq_gptq_gemv_list_workspace_bytes": _sz, "wq_q4g32_gemv_list_destroy": None}

# include/relax_amd_wq_testing.h: the work-split overrides of the calling thread (void) and one query (int)
TESTING_SIGNATURES = {
    "wq_debug_set_gemm_config": [_int],
    "wq_debug_set_gemm_tail_split": [_int],
    "wq_debug_set_gemv_config": [_int, _int],
    "wq_debug_set_gemv_blocks_per_cu": [_int],
    "wq_debug_set_skinny_config": [_int, _int, _int],
    "wq_debug_set_intb_gemv_k_split": [_int],
    "wq_debug_gemv_list_groups": [_vp],
}
# ... and the calibration kernels of librelax_amd_wq_calibrate.so
CALIBRATE_LIB_PATH = os.path.join(HERE, "librelax_amd_wq_calibrate.so")
CALIBRATE_SIGNATURES = {
    "wq_calibrate_mfma_f16": [_vp, _i64, _int, ctypes.POINTER(ctypes.c_double), _vp],
    "wq_calibrate_read": [_vp, _i64, _vp, _vp],
}

_lib = None
_calibrate_lib = None


class WqError(RuntimeError):
    """A C-ABI call returned a non-zero status."""


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m relax_amd.build` "
                "(hipcc, --offload-arch=gfx950). There is no CPU fallback."
            )
        # torch goes first: it ships its own HIP runtime (same soname as the system
        # one), and whichever copy is mapped first serves the whole process.  The
        # tensors this package receives live in torch's runtime, so the kernels must too.
        import torch  # noqa: F401

        l = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(l, name)  # AttributeError if the symbol is not exported
            fn.argtypes = argtypes
            fn.restype = _RESTYPES.get(name, ctypes.c_int)
        for name, argtypes in TESTING_SIGNATURES.items():
            fn = getattr(l, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int if name == "wq_debug_gemv_list_groups" else None
        _lib = l
    return _lib


def calibrate_lib() -> ctypes.CDLL:
    """The measurement-only library (streaming-read and MFMA-issue ceilings)."""
    global _calibrate_lib
    if _calibrate_lib is None:
        if not os.path.exists(CALIBRATE_LIB_PATH):
            raise ImportError(f"{CALIBRATE_LIB_PATH} is missing: build it with `python -m relax_amd.build`")
        import torch  # noqa: F401  (same reason as in lib())

        l = ctypes.CDLL(CALIBRATE_LIB_PATH)
        for name, argtypes in CALIBRATE_SIGNATURES.items():
            fn = getattr(l, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        _calibrate_lib = l
    return _calibrate_lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().wq_last_error()
        raise WqError(f"{what} failed ({rc}): {msg.decode() if msg else ''}")
