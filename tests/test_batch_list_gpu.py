"""wq_q4g32_gemv_list_create_batched: a list of linears with 2 .. 32 rows of activations in one launch (matrix
cores; up to 16 rows: tiles split along K among the wavefronts; more: wavefronts that own rows of W and keep their
sums in registers), against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch

    assert torch.cuda.is_available(), "these tests need a GPU"
    from relax_amd import ops
    from tests import gpu_util

    return ops, gpu_util, torch


def _linear(oracle, u, N, K, M, seed):
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed)
    return dict(W=W, S=S, x=x, dW=u.dev(W), dS=u.dev(S), N=N, K=K)


# K = 256: one short panel; 4096: exactly one panel at M <= 8, two at M > 8; 11008: three panels, the last one short;
# N = 1, 7, 130: fewer rows than a tile / a partial last tile; 40000: ten tiles per workgroup
SHAPES = [(4096, 4096), (12288, 4096), (22016, 4096), (4096, 11008), (1, 256), (7, 512), (130, 11008), (1001, 2304),
          (40000, 256), (48, 16384), (600, 28672), (70, 32768)]


@pytest.mark.parametrize("M", [2, 5, 8, 9, 16, 17, 32])
def test_independent_linears_match_oracle(env, oracle, M):
    ops, u, torch = env
    lins = []
    for i, (N, K) in enumerate(SHAPES):
        l = _linear(oracle, u, N, K, M, seed=200 + i)
        l["dx"] = u.dev(l["x"])
        l["y"] = torch.zeros((M, N), dtype=torch.float16, device="cuda")
        lins.append(l)
    gl = ops.Q4G32GemvList([(l["dW"], l["dS"], l["dx"], l["y"]) for l in lins], M=M)
    assert gl.info()[0] == 0
    print(f"batch list: independent linears, M = {M}", flush=True)
    gl.run()
    gl.status()
    first = [l["y"].clone() for l in lins]
    for l in lins:
        u.assert_close(u.host(l["y"]), oracle.q4g32_linear(l["W"], l["S"], l["x"], nthreads=8), f"batch list M={M} {l['N']}x{l['K']}")
    # launches repeat bit for bit: the partial sums are added in a fixed order
    for rep in range(2):
        for l in lins:
            l["y"].zero_()
        gl.run()
        gl.status()
        for l, f in zip(lins, first):
            assert torch.equal(l["y"], f), (rep, l["N"], l["K"], float((l["y"].float() - f.float()).abs().max()),
                                            int((l["y"] != f).sum()))


@pytest.mark.parametrize("M", [2, 8, 9, 16, 17, 32])
def test_every_nibble_position_carries_its_scale(env, oracle, M):
    """All codes 8 (weight = scale), a different power-of-two-free scale per (row, group), activations that pick
    ONE of the 8 nibble positions of every word: y[m, n] = sum over groups of scale[n, g] * (sum of the x at that
    position), exactly representable.  Catches a scale applied to some positions only (one-hot activations and
    uniform scales both hide that), on a single tile and on a matrix of several panels."""
    ops, u, torch = env
    for N, K in [(16, 256), (48, 4096)]:
        G = K // 32
        W = np.full((N, K // 8), 0x88888888, dtype=np.uint32)
        S = (1.0 + (np.arange(N)[:, None] * 7 + np.arange(G)[None, :] * 3) % 29).astype(np.float16)
        dW, dS = u.dev(W), u.dev(S)
        for p in range(8):
            x = np.zeros((M, K), np.float16)
            x[:, p::8] = (1 + np.arange(M)[:, None] % 3).astype(np.float16)      # 4 weights per group and row of x
            y = torch.zeros((M, N), dtype=torch.float16, device="cuda")
            gl = ops.Q4G32GemvList([(dW, dS, u.dev(x), y)], M=M)
            gl.run()
            gl.status()
            want = (4.0 * (1 + np.arange(M) % 3))[:, None] * S.astype(np.float64).sum(axis=1)[None, :]
            assert want.max() < 65504
            got = u.host(y).astype(np.float64)
            assert np.array_equal(got, want.astype(np.float16).astype(np.float64)), (M, N, K, p, np.abs(got - want).max())


# N = 520 with aligned operands: the four outputs of a lane go out as one 8-byte store; N = 522 / 1001 or a bias that
# starts 2 bytes past an 8-byte boundary: one 2-byte store per output
@pytest.mark.parametrize("M,N,shift", [(6, 520, 0), (20, 520, 0), (6, 522, 0), (20, 1001, 0), (6, 520, 1), (32, 520, 1)])
def test_epilogue_and_one_hot(env, oracle, M, N, shift):
    ops, u, torch = env
    K = 1024
    x, W, S = oracle.make_q4g32_inputs(M, N, K, seed=7)
    rng = np.random.default_rng(3)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    # (shift = 1: y, like the bias below, starts 2 bytes past an 8-byte boundary)
    y = torch.zeros((M * N + shift,), dtype=torch.float16, device="cuda")[shift:].view(M, N)
    assert y.data_ptr() % 8 == 2 * shift
    y2 = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    xh = np.zeros((M, K), np.float16)
    cols = ([0, 37, 260, 511, 777, 1023] * 6)[:M]
    for m, c in enumerate(cols):
        xh[m, c] = 1
    dW, dS = u.dev(W), u.dev(S)
    dbias = u.dev(np.concatenate([np.zeros(shift, np.float16), bias]))[shift:]
    assert dbias.data_ptr() % 8 == 2 * shift
    gl = ops.Q4G32GemvList([(dW, dS, u.dev(x), y, dbias, u.dev(res)), (dW, dS, u.dev(xh), y2)], M=M)
    gl.run()
    gl.status()
    u.assert_close(u.host(y), oracle.q4g32_linear(W, S, x, bias=bias, residual=res), "batch list epilogue")
    # a one-hot row of x selects a dequantized column exactly (every position of the 8-weight unpack is hit)
    B = oracle.q4g32_dequant(W, S)
    got = u.host(y2)
    for m, c in enumerate(cols):
        assert np.array_equal(got[m].view(np.uint16), B[:, c].view(np.uint16)), (m, c)


def test_many_passes_with_a_ragged_end(env, oracle):
    """One long linear at M = 20 (the kernel whose wavefronts own rows of W): every workgroup makes several passes
    over its rows, the last one short (fewer row tiles per wavefront, some wavefronts without any).  N is odd
    (2-byte stores) and ends 7 rows into a row tile."""
    ops, u, torch = env
    M, N, K = 20, 150007, 2048
    l = _linear(oracle, u, N, K, M, seed=77)
    rng = np.random.default_rng(5)
    bias = rng.standard_normal(N).astype(np.float16)
    y = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    gl = ops.Q4G32GemvList([(l["dW"], l["dS"], u.dev(l["x"]), y, u.dev(bias))], M=M)
    print("batch list: many passes", flush=True)
    gl.run()
    gl.status()
    u.assert_close(u.host(y), oracle.q4g32_linear(l["W"], l["S"], l["x"], bias=bias, nthreads=8), "batch list, many passes")


@pytest.mark.parametrize("M,N,K", [(19, 16 * 37 + 5, 512), (32, 8 * 64 * 3 + 16 * 11, 768), (25, 33, 256), (17, 4096, 11008)])
def test_short_passes_of_the_row_owner_kernel(env, oracle, M, N, K):
    """M > 16, a list of ONE linear (every workgroup takes part): N chosen so that workgroups hold a few row tiles
    only (one per wavefront, some wavefronts idle), a last row tile that ends past N, and K of 1, 1.5, 0.5 and 21.5
    panels of activations (an odd number of 256-k pairs ends a panel after one pair); with bias and residual."""
    ops, u, torch = env
    l = _linear(oracle, u, N, K, M, seed=N + K)
    rng = np.random.default_rng(N)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((M, N)).astype(np.float16)
    y = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    gl = ops.Q4G32GemvList([(l["dW"], l["dS"], u.dev(l["x"]), y, u.dev(bias), u.dev(res))], M=M)
    print(f"batch list: short passes M={M} N={N} K={K}", flush=True)
    for _ in range(2):
        y.zero_()
        gl.run()
        gl.status()
        u.assert_close(u.host(y), oracle.q4g32_linear(l["W"], l["S"], l["x"], bias=bias, residual=res, nthreads=8),
                       f"batch list short passes {M}x{N}x{K}")


@pytest.mark.parametrize("M", [8, 16, 20])
def test_a_short_list_shares_the_xcds_by_cost(env, oracle, M):
    """Four linears of a decoder layer's proportions (rows 3 : 1 : 5.4 : 1 with a long K for the last), the last
    one reading what the third wrote: up to 16 rows the planner gives every linear a SET of XCDs (reported as 0 equal
    groups) instead of equal groups, two dependency levels; results against the oracle, twice."""
    ops, u, torch = env
    from relax_amd import _lib

    shapes = [(1536, 1024), (512, 1024), (2816, 1024), (512, 2816)]
    lins = [_linear(oracle, u, N, K, M, seed=300 + i) for i, (N, K) in enumerate(shapes)]
    ys = [torch.zeros((M, N), dtype=torch.float16, device="cuda") for N, _ in shapes]
    xs = [u.dev(l["x"]) for l in lins]
    entries = [(l["dW"], l["dS"], x, y) for l, x, y in zip(lins, xs, ys)]
    entries[3] = (lins[3]["dW"], lins[3]["dS"], ys[2], ys[3])  # the last linear reads what the third wrote
    gl = ops.Q4G32GemvList(entries, M=M)
    assert gl.info()[0] == 1
    if M <= 16:  # (beyond, a pass costs the same however few rows it holds, and equal groups do as well)
        assert _lib.lib().wq_debug_gemv_list_groups(gl._h) == 0, "expected sets of XCDs for a list of four linears"
    print(f"batch list: short list, M = {M}", flush=True)
    for _ in range(2):
        for y in ys:
            y.zero_()
        gl.run()
        gl.status()
        for i in range(3):
            u.assert_close(u.host(ys[i]), oracle.q4g32_linear(lins[i]["W"], lins[i]["S"], lins[i]["x"], nthreads=8), f"short list {i}")
        # the consumer against the oracle on the producer's DEVICE output (its actual input)
        u.assert_close(u.host(ys[3]), oracle.q4g32_linear(lins[3]["W"], lins[3]["S"], u.host(ys[2]), nthreads=8), "short list consumer")


@pytest.mark.parametrize("M", [4, 12, 27])
def test_dependent_chain_matches_oracle(env, oracle, M):
    """x of a linear is the y of an earlier one: directly in front, one apart, two consumers of one producer; a
    producer with several panels (K = 11008)."""
    ops, u, torch = env
    rng = np.random.default_rng(11)
    a = _linear(oracle, u, 4096, 4096, M, seed=1)    # 0: x0 -> t0
    b = _linear(oracle, u, 11008, 4096, M, seed=2)   # 1: t0 -> t1   (directly behind its producer)
    c = _linear(oracle, u, 4096, 11008, M, seed=3)   # 2: t1 -> t2   (again directly behind, three panels)
    d = _linear(oracle, u, 12288, 4096, M, seed=4)   # 3: t0 -> t3   (second consumer of t0)
    e = _linear(oracle, u, 1024, 4096, M, seed=5)    # 4: t2 -> t4   (producer two in front)
    x0 = rng.standard_normal((M, 4096)).astype(np.float16)
    t = [torch.zeros((M, n), dtype=torch.float16, device="cuda") for n in (4096, 11008, 4096, 12288, 1024)]
    gl = ops.Q4G32GemvList([(a["dW"], a["dS"], u.dev(x0), t[0]), (b["dW"], b["dS"], t[0], t[1]),
                            (c["dW"], c["dS"], t[1], t[2]), (d["dW"], d["dS"], t[0], t[3]),
                            (e["dW"], e["dS"], t[2], t[4])], M=M)
    assert gl.info()[0] == 4  # dependent linears
    print(f"batch list: dependent chain, M = {M}", flush=True)
    r0 = oracle.q4g32_linear(a["W"], a["S"], x0, nthreads=8)
    r1 = oracle.q4g32_linear(b["W"], b["S"], r0, nthreads=8)
    r2 = oracle.q4g32_linear(c["W"], c["S"], r1, nthreads=8)
    r3 = oracle.q4g32_linear(d["W"], d["S"], r0, nthreads=8)
    r4 = oracle.q4g32_linear(e["W"], e["S"], r2, nthreads=8)
    for rep in range(3):
        for y in t:
            y.zero_()
        gl.run()
        gl.status()
        for got, ref, name in zip(t, (r0, r1, r2, r3, r4), "abcde"):
            u.assert_close(u.host(got), ref, f"batch chain {name} rep {rep}")
    # the same list inside a HIP graph, replayed with eager work in between
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        gl.run()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            gl.run()
    keep = [y.clone() for y in t]
    for rep in range(3):
        for y in t:
            y.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for y, k in zip(t, keep):
            assert torch.equal(y, k), rep
    gl.status()


@pytest.mark.parametrize("M", [3, 16, 32])
def test_a_long_row_behind_its_producer(env, oracle, M):
    """The longest rows (K = 28672: seven or fourteen panels, 56 of the row-owner kernel) fed by a linear of the same
    list, beside a second long linear."""
    ops, u, torch = env
    rng = np.random.default_rng(5)
    up = _linear(oracle, u, 28672, 256, M, seed=21)     # 0: x0 -> t0 [M, 28672]
    down = _linear(oracle, u, 300, 28672, M, seed=22)   # 1: t0 -> t1
    other = _linear(oracle, u, 64, 32768, M, seed=23)   # 2: independent
    x0 = rng.standard_normal((M, 256)).astype(np.float16)
    t = [torch.zeros((M, n), dtype=torch.float16, device="cuda") for n in (28672, 300, 64)]
    gl = ops.Q4G32GemvList([(up["dW"], up["dS"], u.dev(x0), t[0]), (down["dW"], down["dS"], t[0], t[1]),
                            (other["dW"], other["dS"], u.dev(other["x"]), t[2])], M=M)
    print(f"batch list: long rows, M = {M}", flush=True)
    r0 = oracle.q4g32_linear(up["W"], up["S"], x0, nthreads=8)
    refs = (r0, oracle.q4g32_linear(down["W"], down["S"], r0, nthreads=8),
            oracle.q4g32_linear(other["W"], other["S"], other["x"], nthreads=8))
    for rep in range(2):
        for y in t:
            y.zero_()
        gl.run()
        gl.status()
        for got, ref, name in zip(t, refs, ("up", "down", "other")):
            u.assert_close(u.host(got), ref, f"batch long rows M={M} {name} rep {rep}")


def test_argument_errors(env, oracle):
    ops, u, torch = env
    from relax_amd._lib import WqError

    a = _linear(oracle, u, 64, 128, 4, seed=1)
    y = torch.zeros((4, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(WqError, match="multiple of 256"):
        ops.Q4G32GemvList([(a["dW"], a["dS"], u.dev(a["x"]), y)], M=4)
    b = _linear(oracle, u, 64, 256, 33, seed=1)
    with pytest.raises(WqError, match="rows of activations"):
        ops.Q4G32GemvList([(b["dW"], b["dS"], u.dev(b["x"]), torch.zeros((33, 64), dtype=torch.float16, device="cuda"))], M=33)
    c = _linear(oracle, u, 64, 256, 4, seed=1)
    with pytest.raises(ValueError):
        ops.Q4G32GemvList([(c["dW"], c["dS"], u.dev(c["x"])[:2], y)], M=4)
    with pytest.raises(WqError, match="more than one linear"):
        # an x that two earlier linears of the list write: the consumer could only wait for one of them
        d = _linear(oracle, u, 256, 256, 4, seed=2)
        xd = u.dev(d["x"])
        h = torch.zeros((4 * 256,), dtype=torch.float16, device="cuda")   # [4, 256], written in two pieces
        ops.Q4G32GemvList([(d["dW"][:128], d["dS"][:128], xd, h[:512]), (d["dW"][:128], d["dS"][:128], xd, h[512:]),
                           (d["dW"], d["dS"], h, torch.zeros((4, 256), dtype=torch.float16, device="cuda"))], M=4)


def test_a_wait_that_runs_out_is_reported_and_every_wavefront_exits(env, oracle):
    """Spin limit 0: the consumer's first look at the producer's counters comes before the producer's group has
    finished, so the wait gives up at once; the launch still ends, status() reports it, and the next launch
    with the normal limit is correct."""
    ops, u, torch = env
    M = 6
    a = _linear(oracle, u, 22016, 4096, M, seed=21)
    b = _linear(oracle, u, 512, 4096, M, seed=22)
    t0 = torch.zeros((M, 22016), dtype=torch.float16, device="cuda")
    t1 = torch.zeros((M, 512), dtype=torch.float16, device="cuda")
    mid = torch.zeros((M, 4096), dtype=torch.float16, device="cuda")
    c = _linear(oracle, u, 4096, 4096, M, seed=23)
    # c writes `mid`, which b reads: b waits for c; a keeps the other workgroups busy
    gl = ops.Q4G32GemvList([(a["dW"], a["dS"], u.dev(a["x"]), t0), (c["dW"], c["dS"], u.dev(c["x"]), mid),
                            (b["dW"], b["dS"], mid, t1)], M=M)
    assert gl.info()[0] == 1
    from relax_amd._lib import WqError

    gl.set_spin_limit(0)
    print("batch list: spin limit 0", flush=True)
    gl.run()
    with pytest.raises(WqError, match="timed out"):
        gl.status()
    gl.set_spin_limit(200_000_000)
    gl.run()
    gl.status()
    r_mid = oracle.q4g32_linear(c["W"], c["S"], c["x"], nthreads=8)
    u.assert_close(u.host(t0), oracle.q4g32_linear(a["W"], a["S"], a["x"], nthreads=8), "bystander after a reported time-out")
    u.assert_close(u.host(mid), r_mid, "producer after a reported time-out")
    u.assert_close(u.host(t1), oracle.q4g32_linear(b["W"], b["S"], r_mid, nthreads=8), "consumer after a reported time-out")
