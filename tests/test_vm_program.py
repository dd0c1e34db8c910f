"""The instruction-list executor (include/relax_amd_vm.h): planning and error paths on the CPU,
execution, memory reuse and HIP-graph replay against the oracle on the GPU."""
import ctypes

import numpy as np
import pytest


def _lib():
    from relax_amd import _lib

    return _lib.lib()


def _shape(*dims):
    return (ctypes.c_int64 * max(1, len(dims)))(*dims)


def _call(l, p, name, regs):
    n = len(regs)
    vals = (ctypes.c_int64 * n)(*regs)
    kinds = (ctypes.c_int * n)(*([1] * n))
    return l.wq_program_add_call(p, name.encode(), n, vals, kinds)


def test_plan_reuses_storage_of_dead_tensors():
    l = _lib()
    p = l.wq_program_create()
    try:
        w = l.wq_program_add_external(p, 1, 32, 2, _shape(64, 8), 0x1000, 10)
        s = l.wq_program_add_external(p, 2, 16, 2, _shape(64, 2), 0x2000, 10)
        x = l.wq_program_add_external(p, 2, 16, 2, _shape(4, 64), 0x3000, 10)
        # chain x -> t0 -> t1 -> t2 -> t3: t_i is dead once t_{i+1} is written
        t = [l.wq_program_add_planned(p, 2, 16, 2, _shape(4, 64)) for _ in range(4)]
        big = l.wq_program_add_planned(p, 2, 16, 2, _shape(4, 6400))  # never used: costs nothing
        assert min(t) >= 0 and big >= 0
        prev = x
        for r in t:
            assert _call(l, p, "relax_amd.q4f16_1_matmul", [w, s, prev, r]) == 0
            prev = r
        assert l.wq_program_num_instructions(p) == 4
        need = l.wq_program_plan(p)
        # an instruction's input and output are live together, so two blocks of 512 bytes, not four
        assert need == 2 * 512
        assert l.wq_program_unplanned_bytes(p) == 4 * 512
        # running without storage is refused
        assert l.wq_program_run(p, None) != 0
        assert b"no storage" in l.wq_last_error()
        assert l.wq_program_set_workspace(p, 0x10000, 100) != 0 and b"needed" in l.wq_last_error()
        assert l.wq_program_set_workspace(p, 0x10010, 4096) != 0 and b"aligned" in l.wq_last_error()
    finally:
        l.wq_program_destroy(p)


def test_plan_keeps_overlapping_tensors_apart_and_fits_sizes():
    l = _lib()
    p = l.wq_program_create()
    try:
        w = l.wq_program_add_external(p, 1, 32, 2, _shape(64, 8), 0x1000, 10)
        s = l.wq_program_add_external(p, 2, 16, 2, _shape(64, 2), 0x2000, 10)
        x = l.wq_program_add_external(p, 2, 16, 2, _shape(4, 64), 0x3000, 10)
        a = l.wq_program_add_planned(p, 2, 16, 2, _shape(4, 64))      # 512 B, live 0..3
        b = l.wq_program_add_planned(p, 2, 16, 2, _shape(40, 64))     # 5120 B, live 1..1
        c = l.wq_program_add_planned(p, 2, 16, 2, _shape(8, 64))      # 1024 B, live 2..3: fits b's block
        d = l.wq_program_add_planned(p, 2, 16, 2, _shape(400, 64))    # 51200 B, live 3..3: fits nothing
        for regs in ([w, s, x, a], [w, s, x, b], [w, s, x, c], [w, s, a, d], ):
            assert _call(l, p, "relax_amd_q4f16_1_matmul", regs) == 0  # C symbol name works too
        assert _call(l, p, "relax_amd_q4f16_1_matmul", [w, s, c, d]) == 0
        assert l.wq_program_plan(p) == 512 + 5120 + 51200
    finally:
        l.wq_program_destroy(p)


def test_program_argument_errors():
    l = _lib()
    p = l.wq_program_create()
    try:
        assert _call(l, p, "no.such.function", []) != 0 and b"no PackedFunc" in l.wq_last_error()
        assert l.wq_program_add_planned(p, 2, 12, 1, _shape(4)) < 0
        assert l.wq_program_add_planned(p, 2, 16, 1, _shape(-4)) < 0
        r = l.wq_program_add_planned(p, 2, 16, 1, _shape(4))
        assert r == 0
        assert _call(l, p, "relax_amd.q4f16_1_matmul", [0, 7]) != 0 and b"does not exist" in l.wq_last_error()
        assert l.wq_program_rebind(p, r, 0x1000) != 0  # planned storage cannot be rebound
        assert l.wq_program_replay(p, None) != 0 and b"nothing captured" in l.wq_last_error()
        assert l.wq_program_set_workspace(p, 0x1000, 1 << 20) != 0  # not planned yet
    finally:
        l.wq_program_destroy(p)


def test_fused_group_order_keeps_dependences_and_separates_producers_from_consumers():
    """Planning alone (no GPU): a stack of decode linears (one row of x) becomes one fused run whose
    order is a permutation that keeps every true / anti / output dependence and puts other linears
    between a producer and its consumer."""
    l = _lib()
    p = l.wq_program_create()
    try:
        L = 6
        dims = {"q": (384, 128), "o": (128, 128), "g": (512, 128), "d": (128, 256)}
        addr = [0x100000]

        def ext(code, bits, *shape):
            addr[0] += 0x100000
            return l.wq_program_add_external(p, code, bits, len(shape), _shape(*shape), addr[0], 10)

        hidden, attn, act = ext(2, 16, 1, 128), ext(2, 16, 1, 128), ext(2, 16, 1, 256)
        reads, writes = [], []
        h = hidden
        for layer in range(L):
            w = {k: (ext(1, 32, n, kk // 8), ext(2, 16, n, kk // 32)) for k, (n, kk) in dims.items()}
            t = {k: l.wq_program_add_planned(p, 2, 16, 2, _shape(1, n)) for k, (n, _) in dims.items()}
            for k, x in (("q", h), ("o", attn), ("g", t["o"]), ("d", act)):
                assert _call(l, p, "relax_amd.q4f16_1_matmul", [w[k][0], w[k][1], x, t[k]]) == 0
                reads.append({w[k][0], w[k][1], x})
                writes.append(t[k])
            h = t["d"]
        n = 4 * L
        need = l.wq_program_plan(p)
        # nothing is shared inside the run, and the run's descriptor table is part of the workspace
        assert need >= l.wq_program_unplanned_bytes(p) + l.wq_q4g32_gemv_list_workspace_bytes(n)
        buf = (ctypes.c_int * n)()
        assert l.wq_program_fused_order(p, 0, buf, n) == n
        order = list(buf)
        assert sorted(order) == list(range(n))
        pos = {ins: k for k, ins in enumerate(order)}
        gaps = []
        for i in range(n):
            for j in range(i):
                raw = writes[j] in reads[i]
                if raw or writes[i] == writes[j] or writes[i] in reads[j]:
                    assert pos[j] < pos[i], (j, i)
                if raw:
                    gaps.append(pos[i] - pos[j])
        # at the end of the run nothing independent is left to put between the last producers and
        # consumers; everywhere else at least three linears lie between
        assert len(gaps) == 2 * L - 1 and min(gaps[:-2]) >= 4 and min(gaps) >= 2, gaps
        # switched off: the instructions keep their order and storage is shared again
        assert l.wq_program_set_option(p, b"fuse_decode", 0) == 0
        assert l.wq_program_plan(p) < l.wq_program_unplanned_bytes(p)
        assert l.wq_program_fused_order(p, 0, buf, n) < 0
        assert l.wq_program_set_option(p, b"no_such_option", 1) != 0
    finally:
        l.wq_program_destroy(p)


@pytest.mark.parametrize("M,n,fused", [(1, 2, 1), (4, 2, 1), (4, 1, 0), (8, 3, 0), (8, 4, 1), (16, 8, 0), (16, 16, 1),
                                       (32, 8, 0), (32, 12, 1)])
def test_short_runs_of_batched_linears_are_not_fused(M, n, fused):
    """Planning alone (no GPU): with several rows of x a run only becomes one launch of the list kernel from the
    length at which that launch is faster than the calls one by one."""
    l = _lib()
    p = l.wq_program_create()
    try:
        addr = [0x100000]

        def ext(code, bits, *shape):
            addr[0] += 0x100000
            return l.wq_program_add_external(p, code, bits, len(shape), _shape(*shape), addr[0], 10)

        x = ext(2, 16, M, 256)
        for _ in range(n):
            W, S, y = ext(1, 32, 64, 32), ext(2, 16, 64, 8), ext(2, 16, M, 64)
            assert _call(l, p, "relax_amd.q4f16_1_matmul", [W, S, x, y]) == 0
        assert l.wq_program_plan(p) >= 0
        buf = (ctypes.c_int * n)()
        got = l.wq_program_fused_order(p, 0, buf, n)  # the first run, if there is one
        assert (got == n) if fused else (got < 0), got
    finally:
        l.wq_program_destroy(p)


def test_a_residual_from_the_run_ends_the_fused_run():
    """Planning alone: the list kernel orders a linear behind one earlier linear through its x only, so an
    instruction whose residual (or bias) is the output of an earlier linear of the run starts a new run instead
    of making the whole run fall back to one launch per instruction."""
    l = _lib()
    p = l.wq_program_create()
    try:
        addr = [0x100000]

        def ext(code, bits, *shape):
            addr[0] += 0x100000
            return l.wq_program_add_external(p, code, bits, len(shape), _shape(*shape), addr[0], 10)

        x = ext(2, 16, 1, 256)
        bias = ext(2, 16, 64)
        ys = []
        for i in range(5):
            W, S, y = ext(1, 32, 64, 32), ext(2, 16, 64, 8), ext(2, 16, 1, 64)
            if i == 3:  # the residual stream: the output of linear 1 is added to linear 3
                assert _call(l, p, "relax_amd.q4f16_1_matmul_bias_residual", [W, S, x, bias, ys[1], y]) == 0
            else:
                assert _call(l, p, "relax_amd.q4f16_1_matmul", [W, S, x, y]) == 0
            ys.append(y)
        assert l.wq_program_plan(p) > 0  # the descriptor tables of the runs
        buf = (ctypes.c_int * 8)()
        assert l.wq_program_fused_order(p, 0, buf, 8) == 3 and sorted(buf[:3]) == [0, 1, 2]
        assert l.wq_program_fused_order(p, 1, buf, 8) == 2 and sorted(buf[:2]) == [3, 4]
        assert l.wq_program_unfused_reason(p, 0) == b""
    finally:
        l.wq_program_destroy(p)


def test_runs_of_autogptq_decode_linears_are_fused_apart_from_q4f16_1_runs():
    """Planning alone: relax_amd.autogptq_matmul with one row of x and a group size of 32 << t joins a run of its
    own kind (with or without a row order, with or without the gather workspace argument); a q4f16_1 linear, a
    group size of 96 or a second row of x ends the run."""
    l = _lib()
    p = l.wq_program_create()
    try:
        addr = [0x100000]

        def ext(code, bits, *shape):
            addr[0] += 0x100000
            return l.wq_program_add_external(p, code, bits, len(shape), _shape(*shape), addr[0], 10)

        def call(name, args):  # None: a null handle
            n = len(args)
            vals = (ctypes.c_int64 * n)(*[0 if a is None else a for a in args])
            kinds = (ctypes.c_int * n)(*[2 if a is None else 1 for a in args])
            return l.wq_program_add_call(p, name.encode(), n, vals, kinds)

        K, N = 768, 64
        x, x2, ws = ext(2, 16, 1, K), ext(2, 16, 2, K), ext(1, 8, 2 * K)
        perm = ext(0, 32, K)

        def gptq(G, xr=None, with_perm=False, with_ws=False, rows=1):
            W, SZ, y = ext(1, 32, N, K // 8), ext(2, 16, N, G, 2), ext(2, 16, rows, N)
            args = [W, SZ, perm if with_perm else None, x if xr is None else xr, None, y] + ([ws] if with_ws else [])
            assert call("relax_amd.autogptq_matmul", args) == 0

        gptq(6)                                   # 0: group size 128
        gptq(24, with_perm=True, with_ws=True)    # 1: group size 32, a row order
        gptq(3, with_ws=True)                     # 2: group size 256
        W, S, y = ext(1, 32, N, K // 8), ext(2, 16, N, K // 32), ext(2, 16, 1, N)
        assert call("relax_amd.q4f16_1_matmul", [W, S, x, y]) == 0   # 3
        W, S, y = ext(1, 32, N, K // 8), ext(2, 16, N, K // 32), ext(2, 16, 1, N)
        assert call("relax_amd.q4f16_1_matmul", [W, S, x, y]) == 0   # 4
        gptq(6)                                   # 5
        gptq(8)                                   # 6: group size 96: call by call
        gptq(6)                                   # 7
        gptq(6, xr=x2, rows=2)                    # 8: two rows: call by call
        gptq(6)                                   # 9 (a run of one is not fused)
        assert l.wq_program_plan(p) > 0
        buf = (ctypes.c_int * 8)()
        assert l.wq_program_fused_order(p, 0, buf, 8) == 3 and sorted(buf[:3]) == [0, 1, 2]
        assert l.wq_program_fused_order(p, 1, buf, 8) == 2 and sorted(buf[:2]) == [3, 4]
        assert l.wq_program_fused_order(p, 2, buf, 8) < 0  # no third run
    finally:
        l.wq_program_destroy(p)


def test_autogptq_list_workspace_size():
    """wq_gptq_gemv_list_workspace_bytes: the plain size, plus (only if some layer has a row order) a table of jobs
    and 2 K bytes per such layer, each rounded up to 256."""
    import ctypes as C

    class Desc(C.Structure):
        _fields_ = [(n, C.c_void_p) for n in ("W_nk", "SZ", "perm", "x", "bias", "residual", "y")] + \
                   [(n, C.c_int64) for n in ("N", "K", "G")]

    l = _lib()
    arr = (Desc * 3)()
    for i, (K, has) in enumerate(((4096, False), (1000 * 32, True), (96, True))):
        arr[i] = Desc(None, None, 0x1000 if has else None, None, None, None, None, 64, K, K // 32)
    plain = l.wq_q4g32_gemv_list_workspace_bytes(3)
    assert l.wq_gptq_gemv_list_workspace_bytes(arr, 3) == plain + 256 + 64000 + 256
    arr[1].perm = None
    arr[2].perm = None
    assert l.wq_gptq_gemv_list_workspace_bytes(arr, 3) == plain
    assert l.wq_gptq_gemv_list_workspace_bytes(None, 3) == 0


def test_options_and_a_program_of_external_tensors_only_needs_its_workspace():
    l = _lib()
    p = l.wq_program_create()
    try:
        assert l.wq_program_set_option(p, b"spin_limit_us", 50) == 0
        assert l.wq_program_set_option(p, b"spin_limit_us", -1) != 0 and b"negative" in l.wq_last_error()
        assert l.wq_program_set_option(p, b"no_such_option", 1) != 0 and b"unknown option" in l.wq_last_error()
        # nothing fused yet: nothing to poll
        assert l.wq_program_poll(p, None, 0, None) == 0
        addr = [0x100000]

        def ext(code, bits, *shape):
            addr[0] += 0x100000
            return l.wq_program_add_external(p, code, bits, len(shape), _shape(*shape), addr[0], 10)

        x = ext(2, 16, 1, 256)
        for _ in range(2):
            assert _call(l, p, "relax_amd.q4f16_1_matmul", [ext(1, 32, 64, 32), ext(2, 16, 64, 8), x, ext(2, 16, 1, 64)]) == 0
        # every tensor is external, yet the fused run keeps its descriptor table and counters in the workspace
        assert l.wq_program_plan(p) > 0
        assert l.wq_program_run(p, None) != 0 and b"set the workspace" in l.wq_last_error()
        assert l.wq_program_capture(p, 1) != 0 and b"set the workspace" in l.wq_last_error()
    finally:
        l.wq_program_destroy(p)


SMALL_LINEARS = (("qkv_proj", 384, 128), ("o_proj", 128, 128), ("gate_up_proj", 512, 128), ("down_proj", 128, 256))


@pytest.mark.gpu
@pytest.mark.parametrize("M", [1, 8, 32])
def test_linear_stack_program_matches_oracle_eager_and_replayed(oracle, M):
    import torch

    from relax_amd import vm
    from tests import gpu_util as u

    L = 3
    rng = np.random.default_rng(M)
    host_w, dev_w = [], []
    for l in range(L):
        hw, dw = {}, {}
        for name, N, K in SMALL_LINEARS:
            _, W, S = oracle.make_q4g32_inputs(1, N, K, seed=100 * l + N + K)
            hw[name] = (W, S)
            dw[name] = (u.dev(W), u.dev(S))
        host_w.append(hw)
        dev_w.append(dw)
    hidden = rng.standard_normal((M, 128)).astype(np.float16)
    attn = rng.standard_normal((M, 128)).astype(np.float16)
    act = (rng.standard_normal((M, 256)) * 0.5).astype(np.float16)
    out = torch.zeros((M, 128), dtype=torch.float16, device="cuda")
    d_hidden = u.dev(hidden)
    prog = vm.llama_linear_stack(dev_w, M, d_hidden, u.dev(attn), u.dev(act), out, linears=SMALL_LINEARS)
    assert prog.num_instructions == 4 * L
    if M == 1:
        # the decode step runs as one fused launch: its tensors do not share storage, and the
        # workspace also holds the descriptor table and the counters of the run
        need = prog.plan()
        assert need >= prog.unplanned_bytes
        unfused = vm.llama_linear_stack(dev_w, M, d_hidden, u.dev(attn), u.dev(act), out, linears=SMALL_LINEARS)
        unfused.set_option("fuse_decode", 0)
        assert 0 < unfused.plan() < unfused.unplanned_bytes
    else:
        need = prog.plan()
        # per layer qkv, o, gate_up and the hidden state: storage is reused across layers
        assert 0 < need < prog.unplanned_bytes
        assert need <= 2 * M * (384 + 128 + 512 + 128) * 2 + 8 * 256

    # the last down_proj only depends on mlp_act; check it and, through a second program, the o -> gate_up chain
    want = oracle.q4g32_linear(*host_w[-1]["down_proj"], act, nthreads=4)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        prog.run(stream)
    stream.synchronize()
    eager = u.host(out).copy()
    u.assert_close(eager, want, "stack eager")
    assert prog.num_fused_groups == (1 if M == 1 else 0)
    prog.status(stream)

    prog.capture(stream)
    for rep in range(3):
        out.zero_()                       # eager work between replays
        torch.cuda.synchronize()
        prog.replay(stream)
        stream.synchronize()
        assert np.array_equal(u.host(out).view(np.uint16), eager.view(np.uint16)), rep

    if M == 1:
        # the non-blocking check of the fused run's error word, and a wait that is made to run out from the host:
        # with a spin limit of 0 the gate_up linears give up on their producers at once; every launch still ends
        from relax_amd._lib import WqError

        words = torch.full((4,), -1, dtype=torch.int32).pin_memory()
        assert prog.poll(words, stream) == 1
        stream.synchronize()
        assert words[0].item() == 0
        prog.set_option("spin_limit_us", 0)
        prog.run(stream)
        assert prog.poll(words, stream) == 1
        stream.synchronize()
        if words[0].item() != 0:  # (a 3-layer stack this small may finish its producers before anyone looks)
            with pytest.raises(WqError, match="timed out"):
                prog.status(stream)
        prog.set_option("spin_limit_us", 2_000_000)
        prog.run(stream)
        prog.status(stream)
        assert np.array_equal(u.host(out).view(np.uint16), eager.view(np.uint16))

    # chain through planned storage: y = gate_up(o_proj(attn)) with both intermediates planned
    p2 = vm.DpsProgram()
    wq, sq = dev_w[0]["o_proj"]
    wg, sg = dev_w[0]["gate_up_proj"]
    y = torch.zeros((M, 512), dtype=torch.float16, device="cuda")
    t = p2.planned((M, 128))
    p2.call("relax_amd.q4f16_1_matmul", p2.external(wq, as_uint32=True), p2.external(sq), p2.external(u.dev(attn)), t)
    p2.call("relax_amd.q4f16_1_matmul", p2.external(wg, as_uint32=True), p2.external(sg), t, p2.external(y))
    p2.plan()
    p2.run()
    torch.cuda.synchronize()
    o_ref = oracle.q4g32_linear(*host_w[0]["o_proj"], attn, nthreads=4)
    y_ref = oracle.q4g32_linear(*host_w[0]["gate_up_proj"], o_ref, nthreads=4)
    u.assert_close(u.host(y), y_ref, "planned chain")


@pytest.mark.gpu
def test_llama7b_stack_full_size_matches_oracle(oracle):
    """The real 32-layer program (128 instructions, 3.6 GB of codes and scales) at M = 1, 8, 16, 32, eager and
    replayed.  Checked against the oracle: `out` (the last down_proj, which depends only on mlp_act), and
    two taps in the middle of the stack that each sit behind a dependency through planned storage:
    gate_up_proj of layer 15 (reads that layer's o_proj result) and qkv_proj of layer 16 (reads the hidden
    state written by layer 15's down_proj)."""
    import torch

    from relax_amd import vm
    from tests import gpu_util as u

    L = 32
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    weights = []
    for _ in range(L):
        layer = {}
        for name, N, K in vm.LLAMA7B_LINEARS:
            W = torch.randint(-2**31, 2**31 - 1, (N, K // 8), dtype=torch.int32, device="cuda", generator=g)
            S = (torch.rand((N, K // 32), device="cuda", generator=g) * 0.015 + 0.005).to(torch.float16)
            layer[name] = (W, S)
        weights.append(layer)

    def host_ws(l, name):
        W, S = weights[l][name]
        return u.host(W).view(np.uint32), u.host(S)

    stream = torch.cuda.Stream()
    for M in (1, 8, 16, 32):
        print(f"llama stack M={M}", flush=True)
        rng = np.random.default_rng(40 + M)
        hidden = rng.standard_normal((M, 4096)).astype(np.float16)
        attn = rng.standard_normal((M, 4096)).astype(np.float16)
        act = (rng.standard_normal((M, 11008)) * 0.5).astype(np.float16)
        out = torch.zeros((M, 4096), dtype=torch.float16, device="cuda")
        tap_gu = torch.zeros((M, 22016), dtype=torch.float16, device="cuda")
        tap_qkv = torch.zeros((M, 12288), dtype=torch.float16, device="cuda")
        prog = vm.llama_linear_stack(weights, M, u.dev(hidden), u.dev(attn), u.dev(act), out,
                                     taps={(15, "gate_up_proj"): tap_gu, (16, "qkv_proj"): tap_qkv})
        assert prog.num_instructions == 4 * L
        prog.plan()
        want_out = oracle.q4g32_linear(*host_ws(L - 1, "down_proj"), act, nthreads=8)
        o15 = oracle.q4g32_linear(*host_ws(15, "o_proj"), attn, nthreads=8)
        want_gu = oracle.q4g32_linear(*host_ws(15, "gate_up_proj"), o15, nthreads=8)
        h16 = oracle.q4g32_linear(*host_ws(15, "down_proj"), act, nthreads=8)
        want_qkv = oracle.q4g32_linear(*host_ws(16, "qkv_proj"), h16, nthreads=8)

        def check(what):
            u.assert_close(u.host(out), want_out, f"stack M={M} {what}: out")
            u.assert_close(u.host(tap_gu), want_gu, f"stack M={M} {what}: gate_up of layer 15")
            u.assert_close(u.host(tap_qkv), want_qkv, f"stack M={M} {what}: qkv of layer 16")

        prog.run(stream)
        stream.synchronize()
        prog.status(stream)
        assert prog.num_fused_groups == 1  # one launch for the whole stack
        check("eager")
        eager = [t.clone() for t in (out, tap_gu, tap_qkv)]
        prog.capture(stream)
        for rep in range(2):
            for t in (out, tap_gu, tap_qkv):
                t.zero_()
            torch.cuda.synchronize()
            prog.replay(stream)
            stream.synchronize()
            check(f"replay {rep}")
            for t, e in zip((out, tap_gu, tap_qkv), eager):
                assert torch.equal(t, e), (M, rep)
        del prog


@pytest.mark.gpu
def test_rebind_drops_the_captured_graph(oracle):
    """After a rebind the captured graph would still address the old tensor: replay is refused until the
    program is captured again, and the new capture reads the new tensor."""
    import torch

    from relax_amd import vm
    from relax_amd._lib import WqError
    from tests import gpu_util as u

    M, N, K = 2, 64, 128
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=4)
    x2 = (x * 0.5).astype(np.float16)
    p = vm.DpsProgram()
    X = p.external(u.dev(x))
    y = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    p.call("relax_amd.q4f16_1_matmul", p.external(u.dev(W), as_uint32=True), p.external(u.dev(S)), X, p.external(y))
    p.plan()
    stream = torch.cuda.Stream()
    p.capture(stream)
    p.replay(stream)
    stream.synchronize()
    u.assert_close(u.host(y), oracle.q4g32_linear(W, S, x), "first binding")
    p.rebind(X, u.dev(x2))
    with pytest.raises(WqError, match="nothing captured"):
        p.replay(stream)
    p.capture(stream)
    p.replay(stream)
    stream.synchronize()
    u.assert_close(u.host(y), oracle.q4g32_linear(W, S, x2), "second binding")
    assert len(p._keep) == 4  # one tensor per external register: the first x was released


@pytest.mark.gpu
def test_program_reports_callee_errors():
    import torch

    from relax_amd import vm
    from relax_amd._lib import WqError

    p = vm.DpsProgram()
    w = p.external(torch.zeros((8, 8), dtype=torch.int32, device="cuda"), as_uint32=True)
    s = p.external(torch.zeros((8, 2), dtype=torch.float16, device="cuda"))
    x = p.external(torch.zeros((1, 32), dtype=torch.float16, device="cuda"))  # K mismatch: W says 64
    y = p.planned((1, 8))
    p.call("relax_amd.q4f16_1_matmul", w, s, x, y)
    p.plan()
    with pytest.raises(WqError, match="instruction 0"):
        p.run()


@pytest.mark.gpu
def test_weight_preparation_program(oracle):
    """fp16 weights -> quantize -> (reorder) -> linear, every step a PackedFunc of the instruction list:
    q4f16_1 (encode, and a K-major checkpoint through kn_to_nk) and fpA_intB int8 (encode, ft_preprocess DPS,
    decode_matmul_bias)."""
    import torch

    from relax_amd import vm
    from tests import gpu_util as u

    rng = np.random.default_rng(21)
    M, N, K = 5, 128, 256
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    p = vm.DpsProgram()
    A = p.external(u.dev(w))
    X = p.external(u.dev(x))
    # format A
    Wq = p.external(torch.zeros((N, K // 8), dtype=torch.int32, device="cuda"), as_uint32=True)
    Sq = p.external(torch.zeros((N, K // 32), dtype=torch.float16, device="cuda"))
    ya = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    p.call("relax_amd.q4f16_1_encode", A, Wq, Sq)
    p.call("relax_amd.q4f16_1_matmul", Wq, Sq, X, p.external(ya))
    # the same weights arriving K-major
    W_ref, S_ref = oracle.q4g32_encode(w)
    Wkn = p.external(u.dev(np.ascontiguousarray(W_ref.T)), as_uint32=True)
    Skn = p.external(u.dev(np.ascontiguousarray(S_ref.T)))
    Wt = p.planned((N, K // 8), torch.int32, as_uint32=True)
    St = p.planned((N, K // 32))
    yk = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    p.call("relax_amd.q4f16_1_kn_to_nk", Wkn, Skn, Wt, St)
    p.call("relax_amd.q4f16_1_matmul", Wt, St, X, p.external(yk))
    # format B int8
    q8 = p.planned((K, N), torch.int8)
    sc = p.external(torch.zeros((N,), dtype=torch.float16, device="cuda"))
    tmp = p.planned((N,), torch.float32)
    pre = p.planned((K, N), torch.int8)
    yb = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    p.call("relax_amd.fpA_intB_encode", A, q8, sc, tmp)
    p.call("relax_amd.ft_preprocess_weight_dps", q8, 80, 0, pre)
    p.call("relax_amd.decode_matmul_bias", X, pre, sc, p.external(u.dev(bias)), p.external(yb))
    p.plan()
    p.run()
    torch.cuda.synchronize()
    u.assert_close(u.host(ya), oracle.q4g32_linear(W_ref, S_ref, x), "encoded q4f16_1")
    assert torch.equal(ya, yk)
    q_ref, s_ref = oracle.intb_encode(w, 8)
    u.assert_close(u.host(yb), oracle.intb_linear(x, q_ref, s_ref, 8, bias=bias), "encoded int8")


@pytest.mark.gpu
def test_autogptq_layer_in_a_program(oracle):
    """An act-order AutoGPTQ layer run by the instruction list: the load-time preparation eagerly (it
    synchronises), then matmul + add with the gather workspace as a planned tensor, eager and replayed."""
    import torch

    from relax_amd import ops, vm
    from tests import gpu_util as u

    M, N, K, gs = 4, 264, 512, 128
    x, qw, qz, s, g_idx = oracle.make_gptq_inputs(M, N, K, gs, seed=31, act_order=True)
    res = np.random.default_rng(2).standard_normal((M, N)).astype(np.float16)
    w = ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
    p = vm.DpsProgram()
    W, SZ, perm = p.external(w.W_nk, as_uint32=True), p.external(w.SZ), p.external(w.perm)
    X, R = p.external(u.dev(x)), p.external(u.dev(res))
    y1 = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    y2 = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    ws = p.planned((ops.gptq_workspace_bytes(M, K, True),), torch.uint8)
    h = p.planned((M, N))
    p.call("relax_amd.autogptq_matmul", W, SZ, perm, X, None, h, ws)          # no residual: a null handle
    p.call("relax_amd.autogptq_matmul", W, SZ, perm, X, R, p.external(y1), ws)
    ws2 = p.planned((ops.gptq_workspace_bytes(M, K, True),), torch.uint8)
    p.call("relax_amd.autogptq_matmul", W, SZ, perm, X, h, p.external(y2), ws2)  # residual = the first result
    assert p.plan() >= M * K * 2 + M * N * 2
    p.run()
    torch.cuda.synchronize()
    B = np.ascontiguousarray(oracle.gptq_dequant(qw, qz, s, g_idx).T)
    plain = oracle.nt_matmul_f32acc(B, x)
    u.assert_close(u.host(y1), oracle.nt_matmul_f32acc(B, x, None, res), "autogptq + residual")
    u.assert_close(u.host(y2), oracle.nt_matmul_f32acc(B, x, None, plain), "autogptq chained")
    keep = y2.clone()
    stream = torch.cuda.Stream()
    p.capture(stream)
    for _ in range(2):
        y2.zero_()
        torch.cuda.synchronize()
        p.replay(stream)
        torch.cuda.synchronize()
        assert torch.equal(y2, keep)


@pytest.mark.gpu
@pytest.mark.parametrize("act_order", [False, True])
def test_autogptq_decoder_layer_is_one_launch(oracle, act_order):
    """The four linears of a decoder layer as AutoGPTQ layers at M = 1 (o and down add the residual stream, which
    comes from outside the run): the program runs them as ONE launch of the list kernel, with the same results as
    the calls one by one, eager and replayed; the gather workspaces of the calls are simply not used."""
    import torch

    from relax_amd import ops, vm
    from tests import gpu_util as u

    shapes = [(1536, 512), (512, 512), (2752, 512), (512, 1376 + 32)]  # (N, K); the last K: a partial chunk
    gs = 32
    rng = np.random.default_rng(9)
    layers = []
    for i, (N, K) in enumerate(shapes):
        _, qw, qz, s, g_idx = oracle.make_gptq_inputs(1, N, K, gs, seed=40 + i, act_order=act_order)
        s = (s.astype(np.float32) * 0.2).astype(np.float16)
        w = ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
        layers.append((w, np.ascontiguousarray(oracle.gptq_dequant(qw, qz, s, g_idx).T)))
    x0 = rng.standard_normal((1, 512)).astype(np.float16)
    res = rng.standard_normal((1, 512)).astype(np.float16)
    attn = rng.standard_normal((1, 512)).astype(np.float16)
    act = rng.standard_normal((1, 1408)).astype(np.float16)

    def build(fuse):
        p = vm.DpsProgram()
        p.set_option("fuse_decode", fuse)
        regs = []
        for w, _ in layers:
            regs.append((p.external(w.W_nk, as_uint32=True), p.external(w.SZ),
                         p.external(w.perm) if w.perm is not None else None))
        X0, R, A, C = p.external(u.dev(x0)), p.external(u.dev(res)), p.external(u.dev(attn)), p.external(u.dev(act))
        outs = [torch.zeros((1, n), dtype=torch.float16, device="cuda") for n, _ in shapes]
        O = [p.external(o) for o in outs]
        ws = [p.planned((max(16, ops.gptq_workspace_bytes(1, k, True)),), torch.uint8) for _, k in shapes]
        p.call("relax_amd.autogptq_matmul", *regs[0], X0, None, O[0], ws[0])   # qkv
        p.call("relax_amd.autogptq_matmul", *regs[1], A, R, O[1], ws[1])       # o + residual
        p.call("relax_amd.autogptq_matmul", *regs[2], O[1], None, O[2], ws[2])  # gate/up, fed by o
        p.call("relax_amd.autogptq_matmul", *regs[3], C, R, O[3], ws[3])       # down + residual
        p.plan()
        return p, outs

    fused, got = build(1)
    assert sorted(fused.fused_order(0)) == [0, 1, 2, 3]
    plain, want = build(0)
    print("autogptq decoder layer as one launch", flush=True)
    fused.run()
    plain.run()
    torch.cuda.synchronize()
    assert fused.num_fused_groups == 1 and plain.num_fused_groups == 0  # (lists are built by the first run)
    fused.status()
    r1 = oracle.nt_matmul_f32acc(layers[1][1], attn, None, res)
    refs = [oracle.nt_matmul_f32acc(layers[0][1], x0), r1, oracle.nt_matmul_f32acc(layers[2][1], r1),
            oracle.nt_matmul_f32acc(layers[3][1], act, None, res)]
    for g, w, r, name in zip(got, want, refs, ("qkv", "o", "gate_up", "down")):
        u.assert_close(u.host(g), r, f"fused autogptq {name}")
        u.assert_close(u.host(g), u.host(w), f"fused against call by call, {name}")
    keep = [g.clone() for g in got]
    stream = torch.cuda.Stream()
    fused.capture(stream)
    for _ in range(3):
        for g in got:
            g.zero_()
        torch.cuda.synchronize()
        fused.replay(stream)
        torch.cuda.synchronize()
        for g, k in zip(got, keep):
            assert torch.equal(g, k)
    fused.status()


@pytest.mark.gpu
def test_autogptq_stack_program_fused_against_call_by_call(oracle):
    """vm.llama_autogptq_stack on a small stack (3 layers, every other layer with a row order): the fused program
    (one launch) against the same program run call by call, and its last output against the oracle."""
    import torch

    from relax_amd import ops, vm
    from tests import gpu_util as u

    linears = (("qkv_proj", 384, 128), ("o_proj", 128, 128), ("gate_up_proj", 704, 128), ("down_proj", 128, 352))
    rng = np.random.default_rng(3)
    weights, dense = [], []
    for l in range(3):
        layer, dl = {}, {}
        for name, N, K in linears:
            _, qw, qz, s, g_idx = oracle.make_gptq_inputs(1, N, K, 32, seed=60 + 7 * l + len(name), act_order=(l % 2 == 1))
            s = (s.astype(np.float32) * 0.3).astype(np.float16)
            layer[name] = ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
            dl[name] = np.ascontiguousarray(oracle.gptq_dequant(qw, qz, s, g_idx).T)
        weights.append(layer)
        dense.append(dl)
    hidden = rng.standard_normal((1, 128)).astype(np.float16)
    attn = rng.standard_normal((1, 128)).astype(np.float16)
    act = rng.standard_normal((1, 352)).astype(np.float16)
    outs = []
    for fuse in (1, 0):
        out = torch.zeros((1, 128), dtype=torch.float16, device="cuda")
        p = vm.llama_autogptq_stack(weights, u.dev(hidden), u.dev(attn), u.dev(act), out, linears=linears)
        p.set_option("fuse_decode", fuse)
        p.plan()
        p.run()
        torch.cuda.synchronize()
        p.status()
        assert p.num_fused_groups == (1 if fuse else 0)
        outs.append(u.host(out))
    # only down_proj of the last layer reaches `out`, and its input is the stand-in activation
    want = oracle.nt_matmul_f32acc(dense[-1]["down_proj"], act)
    u.assert_close(outs[0], want, "autogptq stack, fused")
    u.assert_close(outs[1], want, "autogptq stack, call by call")
