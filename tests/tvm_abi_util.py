"""ctypes mirror of the TVM C ABI structs (include/relax_amd_tvm_abi.h) for the tests:
builds TVMValue / type-code arrays the way the Relax VM does (src/runtime/relax_vm/vm.cc:691-775)."""
import ctypes

import numpy as np

kDLCPU, kDLROCM = 1, 10
kDLInt, kDLUInt, kDLFloat = 0, 1, 2
kTVMArgInt, kTVMNullptr, kTVMDLTensorHandle, kTVMNDArrayHandle = 0, 4, 7, 13


class DLDevice(ctypes.Structure):
    _fields_ = [("device_type", ctypes.c_int32), ("device_id", ctypes.c_int32)]


class DLDataType(ctypes.Structure):
    _fields_ = [("code", ctypes.c_uint8), ("bits", ctypes.c_uint8), ("lanes", ctypes.c_uint16)]


class DLTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("device", DLDevice), ("ndim", ctypes.c_int32), ("dtype", DLDataType),
                ("shape", ctypes.POINTER(ctypes.c_int64)), ("strides", ctypes.POINTER(ctypes.c_int64)),
                ("byte_offset", ctypes.c_uint64)]


class TVMValue(ctypes.Union):
    _fields_ = [("v_int64", ctypes.c_int64), ("v_float64", ctypes.c_double), ("v_handle", ctypes.c_void_p)]


_DT = {"int8": (kDLInt, 8), "uint8": (kDLUInt, 8), "uint32": (kDLUInt, 32), "int32": (kDLInt, 32),
       "float16": (kDLFloat, 16), "float32": (kDLFloat, 32)}


def dltensor(ptr, shape, dtype, device_type, byte_offset=0, strides=None):
    """Returns (DLTensor, keepalive)."""
    code, bits = _DT[dtype]
    shp = (ctypes.c_int64 * max(1, len(shape)))(*shape)
    t = DLTensor()
    t.data = ptr
    t.device = DLDevice(device_type, 0)
    t.ndim = len(shape)
    t.dtype = DLDataType(code, bits, 1)
    t.shape = ctypes.cast(shp, ctypes.POINTER(ctypes.c_int64))
    keep = [shp]
    if strides is not None:
        st = (ctypes.c_int64 * len(strides))(*strides)
        t.strides = ctypes.cast(st, ctypes.POINTER(ctypes.c_int64))
        keep.append(st)
    t.byte_offset = byte_offset
    return t, keep


def from_numpy(a: np.ndarray, dtype=None):
    a = np.ascontiguousarray(a)
    t, keep = dltensor(a.ctypes.data, a.shape, dtype or str(a.dtype), kDLCPU)
    return t, keep + [a]


def from_torch(t, dtype=None):
    names = {"torch.int8": "int8", "torch.int32": "int32", "torch.float16": "float16", "torch.uint8": "uint8"}
    d, keep = dltensor(t.data_ptr(), tuple(t.shape), dtype or names[str(t.dtype)], kDLROCM)
    return d, keep + [t]


def pack(*items):
    """items: DLTensor (passed as NDArray handle, what the VM does), int or None (a null handle).  Returns (values, tcodes, n, keep)."""
    n = len(items)
    vals = (TVMValue * n)()
    codes = (ctypes.c_int * n)()
    for i, it in enumerate(items):
        if isinstance(it, DLTensor):
            vals[i].v_handle = ctypes.addressof(it)
            codes[i] = kTVMNDArrayHandle
        elif it is None:
            vals[i].v_handle = None
            codes[i] = kTVMNullptr
        else:
            vals[i].v_int64 = int(it)
            codes[i] = kTVMArgInt
    return vals, codes, n


def call(fn, *items):
    """Calls an exported PackedFunc symbol; returns (rc, ret_value, ret_tcode)."""
    vals, codes, n = pack(*items)
    rv = TVMValue()
    rc_code = ctypes.c_int(kTVMNullptr)
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.POINTER(TVMValue), ctypes.POINTER(ctypes.c_int), ctypes.c_int,
                   ctypes.POINTER(TVMValue), ctypes.POINTER(ctypes.c_int), ctypes.c_void_p]
    rc = fn(vals, codes, n, ctypes.byref(rv), ctypes.byref(rc_code), None)
    return rc, rv, rc_code.value
