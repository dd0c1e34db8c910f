"""The PackedFunc symbols on device tensors: arguments marshalled as the Relax VM does
(TVMValue[] + type codes, NDArray handles), results against the CPU oracle."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch

    assert torch.cuda.is_available()
    from relax_amd import _lib
    from tests import gpu_util, tvm_abi_util

    lib = _lib.lib()
    # kernels go to torch's current stream, supplied through the stream-getter hook
    getter_t = ctypes.CFUNCTYPE(ctypes.c_void_p)
    getter = getter_t(lambda: torch.cuda.current_stream().cuda_stream)
    lib.wq_tvm_set_stream_getter(getter)
    yield lib, gpu_util, tvm_abi_util, torch
    lib.wq_tvm_set_stream_getter(None)


def test_q4f16_1_matmul_family(env, oracle):
    lib, u, T, torch = env
    M, N, K = 3, 200, 512
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=3)
    rng = np.random.default_rng(1)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    dW, dS, dx, db, dr = u.dev(W), u.dev(S), u.dev(x.reshape(M, 1, K)), u.dev(bias), u.dev(res.reshape(M, 1, N))
    y = torch.empty((M, 1, N), dtype=torch.float16, device="cuda")
    tW, _ = T.from_torch(dW, "uint32")
    tS, _ = T.from_torch(dS)
    tx, _ = T.from_torch(dx)
    tb, _ = T.from_torch(db)
    tr, _ = T.from_torch(dr)
    ty, _ = T.from_torch(y)
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_matmul, tW, tS, tx, ty)
    assert rc == 0, lib.wq_last_error()
    u.assert_close(u.host(y).reshape(M, N), oracle.q4g32_linear(W, S, x), "packed q4 matmul")
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_matmul_bias_residual, tW, tS, tx, tb, tr, ty)
    assert rc == 0, lib.wq_last_error()
    u.assert_close(u.host(y).reshape(M, N), oracle.q4g32_linear(W, S, x, bias=bias, residual=res), "packed q4 epilogue")
    # prefill-sized M goes to the MFMA kernel through the same symbol
    M2 = 96
    x2 = rng.standard_normal((M2, K)).astype(np.float16)
    dx2 = u.dev(x2)
    y2 = torch.empty((M2, N), dtype=torch.float16, device="cuda")
    tx2, _ = T.from_torch(dx2)
    ty2, _ = T.from_torch(y2)
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_matmul_bias, tW, tS, tx2, tb, ty2)
    assert rc == 0, lib.wq_last_error()
    u.assert_close(u.host(y2), oracle.q4g32_linear(W, S, x2, bias=bias, nthreads=4), "packed q4 prefill")
    # decode alone, bit-exact
    dq = torch.empty((N, K), dtype=torch.float16, device="cuda")
    tq, _ = T.from_torch(dq)
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_decode, tW, tS, tq)
    assert rc == 0
    assert np.array_equal(u.host(dq).view(np.uint16), oracle.q4g32_dequant(W, S).view(np.uint16))
    # shape errors come back as -1 with a message
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_matmul, tW, tS, tx2, ty)
    assert rc == -1 and b"inconsistent" in lib.wq_last_error()


def _decode_matmul_names():
    """The 22 composite names of python/tvm/relax/backend/contrib/cutlass.py:305-312 (6 plain) and
    :344-372 (16 residual blocks: {bias, bias_gelu} x {cast, no cast} x {add, multiply} x {relu, none})."""
    names = ["decode_matmul", "decode_matmul_bias", "decode_matmul_cast", "decode_matmul_cast_bias",
             "decode_matmul_bias_gelu", "decode_matmul_cast_bias_gelu"]
    for cast in ("", "_cast"):
        for act in ("", "_gelu"):
            for op in ("add", "multiply"):
                for relu in ("", "_relu"):
                    names.append(f"decode_matmul{cast}_bias{act}_residual_{op}{relu}")
    return names


def test_decode_matmul_name_table_is_complete(env):
    lib = env[0]
    lib.wq_tvm_function_name.restype = ctypes.c_char_p
    have = {lib.wq_tvm_function_name(i).decode() for i in range(lib.wq_tvm_num_functions())}
    want = {"relax_amd." + n for n in _decode_matmul_names()}
    assert len(want) == 22
    assert want == {n for n in have if n.startswith("relax_amd.decode_matmul")}


@pytest.mark.parametrize("nbit", [8, 4])
@pytest.mark.parametrize("name", _decode_matmul_names())
def test_decode_matmul_composites(env, oracle, name, nbit):
    """Every composite PackedFunc, epilogue derived from its name, against the oracle; M = 48 runs the
    small-batch kernel, M = 200 the MFMA GEMM."""
    from relax_amd import ops

    lib, u, T, torch = env
    N, K = 128, 256
    okw = {}
    if "_bias" in name:
        okw["bias"] = True
    if "_gelu" in name:
        okw["activation"] = "gelu"
    if "_residual_add" in name:
        okw["binary_op"] = "plus"
    if "_residual_multiply" in name:
        okw["binary_op"] = "multiply"
    if name.endswith("_relu"):
        okw["unary_op"] = "relu"
    sym = getattr(lib, "relax_amd_" + name)
    for M in (48, 200):
        x, A, s = oracle.make_intb_inputs(M, N, K, nbit, seed=nbit + M)
        rng = np.random.default_rng(2 + M)
        bias = rng.standard_normal((1, N)).astype(np.float16)
        res = rng.standard_normal((M, N)).astype(np.float16)
        P = ops.ft_preprocess_weight(u.dev(A), 80, nbit == 4)
        out = torch.empty((M, N), dtype=torch.float16, device="cuda")
        held = [u.dev(x), P, u.dev(s.reshape(1, N))]  # device tensors stay referenced during the call
        kw = dict(okw)
        if "bias" in kw:
            held.append(u.dev(bias))
            kw["bias"] = bias.reshape(-1)
        if "binary_op" in kw:
            held.append(u.dev(res))
            kw["residual"] = res
        held.append(out)
        packed = [T.from_torch(t) for t in held]
        tens = [t for t, _ in packed]
        print(f"{name} int{nbit} M={M}", flush=True)
        rc, _, _ = T.call(sym, *tens)
        assert rc == 0, (name, lib.wq_last_error())
        u.assert_close(u.host(out), oracle.intb_linear(x, A, s, nbit, nthreads=4, **kw), f"{name} int{nbit} M={M}")
        # one argument short is refused
        rc, _, _ = T.call(sym, *tens[:-1])
        assert rc == -1, name


@pytest.mark.parametrize("nbit", [8, 4])
def test_decode_matmul_preprocess_and_full_bias(env, oracle, nbit):
    lib, u, T, torch = env
    M, N, K = 48, 128, 256
    x, A, s = oracle.make_intb_inputs(M, N, K, nbit, seed=nbit)
    rng = np.random.default_rng(2)
    dA = u.dev(A)
    # weight reordering through the DPS PackedFunc on device tensors
    P = torch.empty_like(dA)
    tA, _ = T.from_torch(dA)
    tP, _ = T.from_torch(P)
    rc, _, _ = T.call(lib.relax_amd_ft_preprocess_weight_dps, tA, 80, int(nbit == 4), tP)
    assert rc == 0, lib.wq_last_error()
    assert np.array_equal(u.host(P), oracle.ft_preprocess(A, nbit == 4, 80))
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    dx, ds = u.dev(x), u.dev(s.reshape(1, N))
    tx, _ = T.from_torch(dx)
    ts, _ = T.from_torch(ds)
    to, _ = T.from_torch(out)
    # a bias that varies along M selects bias_stride = N (python/tvm/contrib/cutlass/build.py:728-734)
    bias2 = rng.standard_normal((M, N)).astype(np.float16)
    db2 = u.dev(bias2)
    tb2, _ = T.from_torch(db2)
    rc, _, _ = T.call(lib.relax_amd_decode_matmul_bias, tx, tP, ts, tb2, to)
    assert rc == 0
    u.assert_close(u.host(out), oracle.intb_linear(x, A, s, nbit, bias=bias2, bias_stride=N, nthreads=4), "full bias")


def test_autogptq_family(env, oracle):
    """decode, prepare (returns whether a row order is needed) and matmul + add over an act-order layer,
    with g_idx typed uint32 as in the reference's PrimFunc (tests/python/dlight/test_gpu_gemv.py:639)."""
    lib, u, T, torch = env
    M, N, K, gs = 2, 136, 512, 128
    G = K // gs
    x, qw, qz, s, g_idx = oracle.make_gptq_inputs(M, N, K, gs, seed=21, act_order=True)
    res = np.random.default_rng(4).standard_normal((M, N)).astype(np.float16)
    d = {k: u.dev(v) for k, v in dict(qw=qw, qz=qz, s=s, g=g_idx, x=x.reshape(M, 1, K), r=res.reshape(M, 1, N)).items()}
    tqw, _ = T.from_torch(d["qw"], "uint32")
    tqz, _ = T.from_torch(d["qz"], "uint32")
    ts, _ = T.from_torch(d["s"])
    tg, _ = T.from_torch(d["g"], "uint32")
    tx, _ = T.from_torch(d["x"])
    tr, _ = T.from_torch(d["r"])
    B = torch.empty((K, N), dtype=torch.float16, device="cuda")
    tB, _ = T.from_torch(B)
    rc, _, _ = T.call(lib.relax_amd_autogptq_decode, tqw, tqz, ts, tg, tB)
    assert rc == 0, lib.wq_last_error()
    Bref = oracle.gptq_dequant(qw, qz, s, g_idx)
    assert np.array_equal(u.host(B).view(np.uint16), Bref.view(np.uint16))

    W = torch.empty((N, K // 8), dtype=torch.int32, device="cuda")
    SZ = torch.empty((N, G, 2), dtype=torch.float16, device="cuda")
    perm = torch.empty((K,), dtype=torch.int32, device="cuda")
    scratch = torch.empty((1,), dtype=torch.int32, device="cuda")
    tW, _ = T.from_torch(W, "uint32")
    tSZ, _ = T.from_torch(SZ)
    tp, _ = T.from_torch(perm)
    tsc, _ = T.from_torch(scratch)
    rc, rv, rcode = T.call(lib.relax_amd_autogptq_prepare, tqw, tqz, ts, tg, tW, tSZ, tp, tsc)
    assert rc == 0, lib.wq_last_error()
    assert rcode == T.kTVMArgInt and rv.v_int64 == 1
    assert np.array_equal(u.host(perm), np.argsort(g_idx, kind="stable").astype(np.int32))

    y = torch.empty((M, 1, N), dtype=torch.float16, device="cuda")
    ty, _ = T.from_torch(y)
    ws = torch.empty((40 * K * 2,), dtype=torch.uint8, device="cuda")  # gathered activations, up to M = 40
    tws, _ = T.from_torch(ws)
    rc, _, _ = T.call(lib.relax_amd_autogptq_matmul, tW, tSZ, tp, tx, tr, ty, tws)
    assert rc == 0, lib.wq_last_error()
    want = oracle.nt_matmul_f32acc(np.ascontiguousarray(Bref.T), x, None, res)
    u.assert_close(u.host(y).reshape(M, N), want, "packed autogptq matmul + add")
    rc, _, _ = T.call(lib.relax_amd_autogptq_matmul, tW, tSZ, tp, tx, None, ty, tws)
    assert rc == 0, lib.wq_last_error()
    u.assert_close(u.host(y).reshape(M, N), oracle.nt_matmul_f32acc(np.ascontiguousarray(Bref.T), x), "no residual")

    # a row order needs the workspace for the gathered activations
    M2 = 40
    x2 = np.random.default_rng(5).standard_normal((M2, K)).astype(np.float16)
    dx2 = u.dev(x2)
    y2 = torch.empty((M2, N), dtype=torch.float16, device="cuda")
    tx2, _ = T.from_torch(dx2)
    ty2, _ = T.from_torch(y2)
    rc, _, _ = T.call(lib.relax_amd_autogptq_matmul, tW, tSZ, tp, tx2, None, ty2)
    assert rc == -1 and b"workspace" in lib.wq_last_error()
    rc, _, _ = T.call(lib.relax_amd_autogptq_matmul, tW, tSZ, tp, tx2, None, ty2, tws)
    assert rc == 0, lib.wq_last_error()
    u.assert_close(u.host(y2), oracle.nt_matmul_f32acc(np.ascontiguousarray(Bref.T), x2, nthreads=4), "prefill")

    # without act-order the preparation reports that no row order is needed
    _, qw3, qz3, s3, g3 = oracle.make_gptq_inputs(1, N, K, gs, seed=22)
    e = [u.dev(v) for v in (qw3, qz3, s3, g3)]
    t3 = [T.from_torch(e[0], "uint32")[0], T.from_torch(e[1], "uint32")[0], T.from_torch(e[2])[0], T.from_torch(e[3])[0]]
    rc, rv, rcode = T.call(lib.relax_amd_autogptq_prepare, *t3, tW, tSZ, tp, tsc)
    assert rc == 0 and rv.v_int64 == 0
    rc, _, _ = T.call(lib.relax_amd_autogptq_matmul, tW, tSZ, None, tx, None, ty)
    assert rc == 0, lib.wq_last_error()
    u.assert_close(u.host(y).reshape(M, N), oracle.gptq_linear(qw3, qz3, s3, g3, x), "identity order")
    # wrong arity / shapes
    rc, _, _ = T.call(lib.relax_amd_autogptq_decode, tqw, tqz, ts, tB)
    assert rc == -1
    rc, _, _ = T.call(lib.relax_amd_autogptq_matmul, tW, tSZ, tp, tx2, tr, ty2, tws)
    assert rc == -1 and b"inconsistent" in lib.wq_last_error()


def test_q4f16_1_kn_matmul(env, oracle):
    """relax_amd.q4f16_1_kn_matmul: the K-major layout of tests/python/dlight/test_gpu_reduction.py:102-120 in place."""
    lib, u, T, torch = env
    M, N, K = 3, 520, 4096
    rng = np.random.default_rng(40)
    W_kn = rng.integers(0, 2**32, size=(K // 8, N), dtype=np.uint64).astype(np.uint32)
    S_kn = rng.uniform(0.005, 0.02, size=(K // 32, N)).astype(np.float16)
    x = rng.standard_normal((M, 1, K)).astype(np.float16)
    dW, dS, dx = u.dev(W_kn), u.dev(S_kn), u.dev(x)
    y = torch.empty((M, 1, N), dtype=torch.float16, device="cuda")
    ws = torch.empty((int(lib.wq_q4g32_kn_gemv_workspace_bytes(M, N, K)),), dtype=torch.uint8, device="cuda")
    assert ws.numel() > 0
    tW, _ = T.from_torch(dW, "uint32")
    tS, _ = T.from_torch(dS)
    tx, _ = T.from_torch(dx)
    ty, _ = T.from_torch(y)
    tws, _ = T.from_torch(ws)
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_kn_matmul, tW, tS, tx, ty, tws)
    assert rc == 0, lib.wq_last_error()
    B = oracle.q4g32_kn_dequant(W_kn, S_kn)
    u.assert_close(u.host(y).reshape(M, N), oracle.nt_matmul_f32acc(np.ascontiguousarray(B.T), x.reshape(M, K)), "kn matmul")
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_kn_matmul, tW, tS, tx, ty)   # K is sliced here: the workspace is needed
    assert rc == -1 and b"workspace" in lib.wq_last_error()
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_kn_matmul, tS, tS, tx, ty, tws)
    assert rc == -1


def test_q4f16_1_matmul_f16acc(env, oracle):
    """relax_amd.q4f16_1_matmul_f16acc: the fp16-accumulate mode of the decode fixtures with a small dynamic batch;
    the same bits as the C entry point, and within the fp16 accumulation bound of the fp32-accumulate result."""
    lib, u, T, torch = env
    from relax_amd import ops

    M, N, K = 5, 264, 2048
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=60)
    dW, dS, dx = u.dev(W), u.dev(S), u.dev(x.reshape(M, 1, K))
    y = torch.empty((M, 1, N), dtype=torch.float16, device="cuda")
    tW, _ = T.from_torch(dW, "uint32")
    tS, _ = T.from_torch(dS)
    tx, _ = T.from_torch(dx)
    ty, _ = T.from_torch(y)
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_matmul_f16acc, tW, tS, tx, ty)
    assert rc == 0, lib.wq_last_error()
    direct = ops.q4g32_gemv_f16acc(dW, dS, u.dev(x))
    assert torch.equal(y.reshape(M, N), direct)
    ref = oracle.q4g32_linear(W, S, x).astype(np.float64)
    mag = np.abs(x).astype(np.float64) @ np.abs(oracle.q4g32_dequant(W, S)).astype(np.float64).T
    assert np.all(np.abs(u.host(y).reshape(M, N) - ref) <= 1.1 * (16 + 8 + 2) * 2.0**-11 * mag + 1e-6)
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_matmul_f16acc, tW, tS, tx)
    assert rc == -1
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_matmul_f16acc, tW, tW, tx, ty)
    assert rc == -1


def test_q4f16_1_ngroup_pair(env, oracle):
    """relax_amd.q4f16_1_ngroup_prepare / _matmul_bias_residual: the operands and the buffer order of
    tests/python/dlight/test_gpu_matmul.py:352-401 (codes packed along N; dynamic n rows of x)."""
    lib, u, T, torch = env
    n, N, K = 70, 416, 256
    _, W, S = oracle.make_q4g32_inputs(1, K, N, seed=50)  # W [K, N/8], S [K, N/32]
    rng = np.random.default_rng(51)
    x = rng.standard_normal((1, n, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((1, n, N)).astype(np.float16)
    dW, dS = u.dev(W), u.dev(S)
    W_nk = torch.empty((N, K // 8), dtype=torch.int32, device="cuda")
    ST = torch.empty((N // 32, K), dtype=torch.float16, device="cuda")
    y = torch.empty((1, n, N), dtype=torch.float16, device="cuda")
    tW, _ = T.from_torch(dW, "uint32")
    tS, _ = T.from_torch(dS)
    tWn, _ = T.from_torch(W_nk, "uint32")
    tST, _ = T.from_torch(ST)
    tx, _ = T.from_torch(u.dev(x))
    tb, _ = T.from_torch(u.dev(bias))
    tr, _ = T.from_torch(u.dev(res))
    ty, _ = T.from_torch(y)
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_ngroup_prepare, tW, tS, tWn, tST)
    assert rc == 0, lib.wq_last_error()
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_ngroup_matmul_bias_residual, tWn, tST, tx, tb, tr, ty)
    assert rc == 0, lib.wq_last_error()
    Bt = np.ascontiguousarray(oracle.q4g32_dequant(W, S).T)  # [N, K]: the fixture's decode, transposed
    want = oracle.nt_matmul_f32acc(Bt, x.reshape(n, K), bias, res.reshape(n, N))
    u.assert_close(u.host(y).reshape(n, N), want, "packed ngroup matmul + bias + residual")
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_ngroup_matmul_bias_residual, tWn, tST, tx, None, None, ty)
    assert rc == 0, lib.wq_last_error()
    u.assert_close(u.host(y).reshape(n, N), oracle.nt_matmul_f32acc(Bt, x.reshape(n, K)), "packed ngroup matmul")
    # the unprepared operands are refused by their shapes; wrong arity
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_ngroup_matmul_bias_residual, tW, tS, tx, None, None, ty)
    assert rc == -1 and b"inconsistent" in lib.wq_last_error()
    rc, _, _ = T.call(lib.relax_amd_q4f16_1_ngroup_prepare, tW, tS, tWn)
    assert rc == -1


@pytest.mark.parametrize("M", [1, 3, 40])
def test_autogptq_padded_pair(env, oracle, M):
    """relax_amd.autogptq_prepare_padded / autogptq_matmul_padded: a g_idx whose groups differ in size
    (tests/python/dlight/test_gpu_gemv.py:645-648 index scales[g_idx[k], n] without restriction)."""
    lib, u, T, torch = env
    N, K, G = 136, 1024, 8
    x, qw, qz, s, _ = oracle.make_gptq_inputs(M, N, K, K // G, seed=30 + M)
    g_idx = np.random.default_rng(31).integers(0, G, size=K).astype(np.int32)
    assert len(set(np.bincount(g_idx, minlength=G).tolist())) > 1
    res = np.random.default_rng(32).standard_normal((M, N)).astype(np.float16)
    d = {k: u.dev(v) for k, v in dict(qw=qw, qz=qz, s=s, g=g_idx, x=x, r=res).items()}
    tqw, _ = T.from_torch(d["qw"], "uint32")
    tqz, _ = T.from_torch(d["qz"], "uint32")
    ts, _ = T.from_torch(d["s"])
    tg, _ = T.from_torch(d["g"])
    tx, _ = T.from_torch(d["x"])
    tr, _ = T.from_torch(d["r"])
    cap = int(lib.wq_gptq_padded_k_bound(K, G))
    assert cap >= K and cap % 32 == 0
    W = torch.empty((N * cap // 8,), dtype=torch.int32, device="cuda")
    SZ = torch.empty((N * cap // 32 * 2,), dtype=torch.float16, device="cuda")
    perm = torch.empty((cap,), dtype=torch.int32, device="cuda")
    tW, _ = T.from_torch(W, "uint32")
    tSZ, _ = T.from_torch(SZ)
    tp, _ = T.from_torch(perm)
    rc, rv, rcode = T.call(lib.relax_amd_autogptq_prepare_padded, tqw, tqz, ts, tg, tW, tSZ, tp)
    assert rc == 0, lib.wq_last_error()
    kp = rv.v_int64
    assert rcode == T.kTVMArgInt and K <= kp <= cap and kp % 32 == 0
    order = u.host(perm)[:kp]
    assert np.array_equal(order[order >= 0], np.argsort(g_idx, kind="stable"))
    y = torch.empty((M, N), dtype=torch.float16, device="cuda")
    ty, _ = T.from_torch(y)
    ws = torch.empty((int(lib.wq_gptq_padded_workspace_bytes(M, kp)),), dtype=torch.uint8, device="cuda")
    tws, _ = T.from_torch(ws)
    Bref = oracle.gptq_dequant(qw, qz, s, g_idx)
    rc, _, _ = T.call(lib.relax_amd_autogptq_matmul_padded, tW, tSZ, tp, int(kp), tx, tr, ty, tws)
    assert rc == 0, lib.wq_last_error()
    u.assert_close(u.host(y), oracle.nt_matmul_f32acc(np.ascontiguousarray(Bref.T), x, None, res), "padded matmul + add")
    rc, _, _ = T.call(lib.relax_amd_autogptq_matmul_padded, tW, tSZ, tp, int(kp), tx, None, ty, tws)
    assert rc == 0, lib.wq_last_error()
    u.assert_close(u.host(y), oracle.nt_matmul_f32acc(np.ascontiguousarray(Bref.T), x), "padded matmul")
    # errors: a K_padded that the buffers cannot hold; too few arguments
    rc, _, _ = T.call(lib.relax_amd_autogptq_matmul_padded, tW, tSZ, tp, cap + 32, tx, None, ty, tws)
    assert rc == -1 and b"inconsistent" in lib.wq_last_error()
    rc, _, _ = T.call(lib.relax_amd_autogptq_prepare_padded, tqw, tqz, ts, tg, tW, tSZ)
    assert rc == -1


@pytest.mark.parametrize("case,nbit,group,M", [("int8_percol", 8, -1, 40), ("int8_nobias", 8, -1, 1),
                                               ("int8_percol", 8, -1, 300), ("int4_fine", 4, 64, 24),
                                               ("int4_fine", 4, 64, 260)])
def test_emitted_host_code_runs_on_device(env, oracle, tmp_path, case, nbit, group, M):
    """tests/cpp/ft_api_device.cc calls fastertransformer::gemm_fp16_int_bias_act<uint8_t, PER_COLUMN_SCALE_ONLY>
    and ..._residual<cutlass::uint4b_t, FINEGRAINED_SCALE_ONLY> on device buffers with the argument lists the
    reference emits (python/tvm/contrib/cutlass/gemm_operation.py:441-458), as its own process."""
    import subprocess

    from relax_amd import ops

    lib, u, T, torch = env
    N, K = 192, 512
    x, A, s = oracle.make_intb_inputs(M, N, K, nbit, seed=M + nbit, group_size=group)
    rng = np.random.default_rng(M)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    P = u.host(ops.ft_preprocess_weight(u.dev(A), 80, nbit == 4))
    x.tofile(tmp_path / "A.bin")
    P.tofile(tmp_path / "B.bin")
    s.tofile(tmp_path / "scales.bin")
    kw = {}
    if case != "int8_nobias":
        bias.tofile(tmp_path / "bias.bin")
        kw["bias"] = bias
    if case == "int8_percol":
        kw["activation"] = "gelu"
    if case == "int4_fine":
        res.tofile(tmp_path / "residual.bin")
        kw.update(residual=res, binary_op="plus", unary_op="relu", group_size=64)
    exe = u.build_cpp_program("ft_api_device")
    print(f"ft_api_device {case} M={M}", flush=True)
    r = subprocess.run([exe, case, str(tmp_path), str(M), str(N), str(K)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(tmp_path / "C.bin", np.float16).reshape(M, N)
    u.assert_close(got, oracle.intb_linear(x, A, s, nbit, nthreads=4, **kw), f"emitted host code {case} M={M}")
