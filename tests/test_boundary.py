"""The drop-in boundary without a GPU: the library loads, exports every symbol the
headers declare, and the PackedFunc layer speaks the TVM calling convention."""
import ctypes
import os
import re
import subprocess
import sys
import textwrap

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")
GOLD = os.path.join(ROOT, "tests", "golden", "ft_layout_vectors.npz")


@pytest.fixture(scope="module")
def lib():
    from relax_amd import _lib

    return _lib.lib()


def _declared_symbols(headers=("relax_amd_wq.h", "relax_amd_tvm.h", "relax_amd_vm.h")):
    names = set()
    for h in headers:
        text = open(os.path.join(INC, h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"^\s*(?:const\s+char\*|int|void|int64_t|size_t|wq_program_t\*|wq_gemv_list_t\*)\s+(wq_\w+)\s*\(", text, flags=re.M))
        names |= set(re.findall(r"^WQ_PACKED\((\w+)\);", text, flags=re.M))
    names.discard("name")
    return sorted(names)


def test_every_declared_symbol_is_exported(lib):
    names = _declared_symbols()
    assert len(names) >= 45, names
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    # and the ctypes front end declares the compute entry points it uses
    from relax_amd import _lib

    assert set(_lib.SIGNATURES) <= set(names)
    # the product headers hold no test hook and no calibration kernel
    assert not [n for n in names if n.startswith(("wq_debug_", "wq_calibrate_"))]


def test_testing_header_symbols(lib):
    """include/relax_amd_wq_testing.h: the thread-local overrides live in the product library, the
    calibration kernels in a library of their own."""
    from relax_amd import _lib

    names = _declared_symbols(("relax_amd_wq_testing.h",))
    hooks = sorted(n for n in names if n.startswith("wq_debug_"))
    calib = sorted(n for n in names if n.startswith("wq_calibrate_"))
    assert hooks == sorted(_lib.TESTING_SIGNATURES) and calib == sorted(_lib.CALIBRATE_SIGNATURES)
    assert sorted(names) == hooks + calib or set(names) == set(hooks) | set(calib)
    for n in hooks:
        assert hasattr(lib, n), n
    c = _lib.calibrate_lib()
    for n in calib:
        assert hasattr(c, n) and not hasattr(lib, n), n
    # an override belongs to the thread that set it: an unknown tile configuration is refused before
    # anything touches a device, and the message names the configuration of the CALLING thread
    import threading

    W = np.zeros((64, 8), np.uint32)
    S = np.zeros((64, 2), np.float16)
    x = np.zeros((64, 64), np.float16)
    y = np.zeros((64, 64), np.float16)

    def call():
        rc = lib.wq_q4g32_gemm(W.ctypes.data, S.ctypes.data, x.ctypes.data, None, None, y.ctypes.data, 64, 64, 64, None)
        return rc, lib.wq_last_error().decode()

    seen = {}

    def other():
        lib.wq_debug_set_gemm_config(99)
        seen["other"] = call()
        lib.wq_debug_set_gemm_config(0)

    lib.wq_debug_set_gemm_config(98)
    try:
        t = threading.Thread(target=other)
        t.start()
        t.join()
        seen["main"] = call()
    finally:
        lib.wq_debug_set_gemm_config(0)
    assert seen["other"][0] == -1 and "configuration 99" in seen["other"][1], seen
    assert seen["main"][0] == -1 and "configuration 98" in seen["main"][1], seen


def test_function_table(lib):
    lib.wq_tvm_function_name.restype = ctypes.c_char_p
    lib.wq_tvm_function_symbol.restype = ctypes.c_char_p
    n = lib.wq_tvm_num_functions()
    table = {lib.wq_tvm_function_name(i).decode(): lib.wq_tvm_function_symbol(i).decode() for i in range(n)}
    assert table["cutlass.ft_preprocess_weight"] == "cutlass_ft_preprocess_weight"
    # one entry per decode_matmul pattern of the reference's pattern table (6 base + 16 residual)
    dm = [k for k in table if k.startswith("relax_amd.decode_matmul")]
    assert len(dm) == 22
    for name, sym in table.items():
        assert hasattr(lib, sym), sym
    # no TVM runtime in this process: nothing to register with
    assert lib.wq_tvm_register_globals() == 0


def test_preprocess_dps_on_host_tensors(lib):
    from tests import tvm_abi_util as T

    g = np.load(GOLD)
    for case, is_int4 in (("int8_128x192", 0), ("int4_128x192", 1)):
        a, want = g[case + "_in"], g[case + "_out"]
        out = np.zeros_like(a)
        ta, k1 = T.from_numpy(a)
        to, k2 = T.from_numpy(out)
        out = k2[-1]
        rc, _, _ = T.call(lib.relax_amd_ft_preprocess_weight_dps, ta, 80, is_int4, to)
        assert rc == 0, lib.wq_last_error()
        assert np.array_equal(out, want)
    # byte_offset is honoured
    a, want = g["int8_64x64_in"], g["int8_64x64_out"]
    buf = np.zeros(a.size + 64, np.int8)
    buf[64:] = a.ravel()
    ta, k1 = T.dltensor(buf.ctypes.data, a.shape, "int8", T.kDLCPU, byte_offset=64)
    out = np.zeros_like(a)
    to, k2 = T.from_numpy(out)
    rc, _, _ = T.call(lib.relax_amd_ft_preprocess_weight_dps, ta, 80, 0, to)
    assert rc == 0 and np.array_equal(k2[-1], want)


def test_packed_errors_are_reported_not_fatal(lib):
    from tests import tvm_abi_util as T

    a = np.zeros((64, 64), np.int8)
    ta, k1 = T.from_numpy(a)
    to, k2 = T.from_numpy(np.zeros_like(a))
    # wrong arity
    rc, _, _ = T.call(lib.relax_amd_ft_preprocess_weight_dps, ta, 80)
    assert rc == -1 and b"expected" in lib.wq_last_error()
    # unsupported layout family
    rc, _, _ = T.call(lib.relax_amd_ft_preprocess_weight_dps, ta, 70, 0, to)
    assert rc == -1 and b"sm=70" in lib.wq_last_error()
    # wrong dtype
    tf, k3 = T.from_numpy(np.zeros((64, 64), np.float32))
    rc, _, _ = T.call(lib.relax_amd_ft_preprocess_weight_dps, tf, 80, 0, to)
    assert rc == -1 and b"dtype" in lib.wq_last_error()
    # non-compact strides
    ts, k4 = T.dltensor(a.ctypes.data, (64, 32), "int8", T.kDLCPU, strides=(64, 1))
    rc, _, _ = T.call(lib.relax_amd_ft_preprocess_weight_dps, ts, 80, 0, to)
    assert rc == -1 and b"compact" in lib.wq_last_error()
    # the allocating form needs a runtime to allocate from
    rc, _, _ = T.call(lib.cutlass_ft_preprocess_weight, ta, 80, 0)
    assert rc == -1 and b"no TVM runtime" in lib.wq_last_error()
    # compute entry points refuse host tensors instead of dereferencing them on the GPU
    tw, k5 = T.from_numpy(np.zeros((8, 8), np.uint32))
    tsx, k6 = T.from_numpy(np.zeros((8, 2), np.float16))
    tx, k7 = T.from_numpy(np.zeros((1, 64), np.float16))
    ty, k8 = T.from_numpy(np.zeros((1, 8), np.float16))
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_matmul, tw, tsx, tx, ty)
    assert rc == -1 and b"ROCm device tensor" in lib.wq_last_error()


def test_c_abi_argument_checks_without_gpu(lib):
    # every check below fails before any device call is made
    assert lib.wq_q4g32_gemv(1, 1, 1, 0, 0, 1, 1, 8, 40, 0) != 0 and b"multiple" in lib.wq_last_error()
    assert lib.wq_fpA_intB_gemm(16, 16, 16, 0, 16, 0, 1, 64, 100, -1, 0, 8, 0, 0, 0) != 0
    assert b"multiples of 64" in lib.wq_last_error()
    assert lib.wq_fpA_intB_gemm(16, 16, 16, 0, 16, 9, 1, 64, 64, -1, 0, 8, 0, 0, 0) != 0
    assert b"activation" in lib.wq_last_error()
    assert lib.wq_fpA_intB_gemm(16, 16, 16, 0, 16, 0, 1, 64, 64, -1, 0, 3, 0, 0, 0) != 0
    assert b"weight_nbit" in lib.wq_last_error()
    assert lib.wq_activation_from_string(b"gelu") == 3 and lib.wq_activation_from_string(b"tanh") == -1
    assert lib.wq_binary_op_from_string(b"multiply") == 2 and lib.wq_unary_op_from_string(b"relu") == 1
    # zero-sized problems are accepted without touching memory
    assert lib.wq_q4g32_linear(0, 0, 0, 0, 0, 0, 0, 64, 64, 0) == 0


def test_registers_with_a_tvm_runtime_when_present(tmp_path):
    """In a fresh process: load a stand-in runtime first, then the library; the library's
    load-time hook must register its global names, and 'cutlass.ft_preprocess_weight' called
    through the registry must return a freshly allocated, correctly reordered NDArray."""
    fake = tmp_path / "libfake_tvm_runtime.so"
    subprocess.check_call(["gcc", "-shared", "-fPIC", "-O1", "-o", str(fake), os.path.join(ROOT, "tests", "fake_tvm_runtime.c")])
    script = textwrap.dedent(f"""
        import ctypes, sys, numpy as np
        sys.path.insert(0, {ROOT!r})
        fake = ctypes.CDLL({str(fake)!r}, mode=ctypes.RTLD_GLOBAL)
        from relax_amd import _lib
        lib = _lib.lib()
        from tests import tvm_abi_util as T
        fake.fake_registered_name.restype = ctypes.c_char_p
        names = [fake.fake_registered_name(i).decode() for i in range(fake.fake_num_registered())]
        assert "cutlass.ft_preprocess_weight" in names and "relax_amd.decode_matmul_bias_gelu" in names, names
        assert len(names) == lib.wq_tvm_num_functions()
        g = np.load({GOLD!r})
        a, want = g["int4_256x128_in"], g["int4_256x128_out"]
        ta, keep = T.from_numpy(a)
        f = ctypes.c_void_p()
        assert fake.TVMFuncGetGlobal(b"cutlass.ft_preprocess_weight", ctypes.byref(f)) == 0 and f.value
        vals, codes, n = T.pack(ta, 80, 1)
        rv, rc_code = T.TVMValue(), ctypes.c_int(0)
        fake.TVMFuncCall.argtypes = [ctypes.c_void_p, ctypes.POINTER(T.TVMValue), ctypes.POINTER(ctypes.c_int),
                                     ctypes.c_int, ctypes.POINTER(T.TVMValue), ctypes.POINTER(ctypes.c_int)]
        assert fake.TVMFuncCall(f, vals, codes, n, ctypes.byref(rv), ctypes.byref(rc_code)) == 0
        assert rc_code.value == T.kTVMNDArrayHandle
        out = ctypes.cast(rv.v_handle, ctypes.POINTER(T.DLTensor)).contents
        assert out.ndim == 2 and out.shape[0] == a.shape[0] and out.shape[1] == a.shape[1]
        assert out.data != a.ctypes.data
        got = np.ctypeslib.as_array(ctypes.cast(out.data, ctypes.POINTER(ctypes.c_int8)), shape=a.shape)
        assert np.array_equal(got, want)
        # an error inside a registry call reaches the runtime's last-error slot
        vals, codes, n = T.pack(ta, 95, 1)
        assert fake.TVMFuncCall(f, vals, codes, n, ctypes.byref(rv), ctypes.byref(rc_code)) == -1
        fake.TVMGetLastError.restype = ctypes.c_char_p
        assert b"sm=95" in fake.TVMGetLastError()
        # the array allocated for the failed call went back to the runtime: only the first result is live
        assert fake.fake_live_arrays() == 1, fake.fake_live_arrays()
        print("registry ok", len(names))
    """)
    out = subprocess.run([sys.executable, "-c", script], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "registry ok" in out.stdout


def test_host_keeps_its_own_ft_preprocess_weight(tmp_path):
    """A host whose registry already holds 'cutlass.ft_preprocess_weight' (a TVM built with its CUTLASS
    back end) keeps it: the library registers its own 'relax_amd.*' names only."""
    fake = tmp_path / "libfake_tvm_runtime.so"
    subprocess.check_call(["gcc", "-shared", "-fPIC", "-O1", "-o", str(fake), os.path.join(ROOT, "tests", "fake_tvm_runtime.c")])
    script = textwrap.dedent(f"""
        import ctypes, sys
        sys.path.insert(0, {ROOT!r})
        fake = ctypes.CDLL({str(fake)!r}, mode=ctypes.RTLD_GLOBAL)
        assert fake.fake_register_host_function(b"cutlass.ft_preprocess_weight") == 0
        from relax_amd import _lib
        lib = _lib.lib()
        fake.fake_registered_name.restype = ctypes.c_char_p
        names = [fake.fake_registered_name(i).decode() for i in range(fake.fake_num_registered())]
        assert fake.fake_is_host_function(b"cutlass.ft_preprocess_weight") == 1
        assert names.count("cutlass.ft_preprocess_weight") == 1
        assert "relax_amd.ft_preprocess_weight_dps" in names and "relax_amd.q4f16_1_matmul" in names
        assert len(names) == lib.wq_tvm_num_functions()
        # a second registration replaces the library's own names and still leaves the host's alone
        assert lib.wq_tvm_register_globals() == lib.wq_tvm_num_functions() - 1
        assert fake.fake_is_host_function(b"cutlass.ft_preprocess_weight") == 1
        print("policy ok")
    """)
    out = subprocess.run([sys.executable, "-c", script], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "policy ok" in out.stdout


def test_source_compatible_headers_compile_and_run(tmp_path, lib):
    """Host code written against cutlass_kernels/*.h of the reference's external library
    compiles against include/ and links the shared library (host-only call, no GPU)."""
    exe = tmp_path / "ft_api_host"
    libdir = os.path.join(ROOT, "relax_amd")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-I", INC, os.path.join(ROOT, "tests", "cpp", "ft_api_host.cc"),
                           "-o", str(exe), "-L", libdir, "-lrelax_amd_wq", f"-Wl,-rpath,{libdir}",
                           "-Wl,-rpath,/opt/rocm/lib"])
    g = np.load(GOLD)
    for case, is_int4 in (("int8_256x64", 0), ("int4_256x128", 1)):
        a, want = g[case + "_in"], g[case + "_out"]
        fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
        a.tofile(fin)
        rows, cols = a.shape[0], a.shape[1] * (2 if is_int4 else 1)
        r = subprocess.run([str(exe), str(fin), str(fout), str(rows), str(cols), str(is_int4)], capture_output=True, text=True)
        assert r.returncode == 0, r.stdout + r.stderr
        assert np.array_equal(np.fromfile(fout, np.int8).reshape(a.shape), want)
