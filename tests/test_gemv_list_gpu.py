"""wq_q4g32_gemv_list_*: a list of decode linears in one launch, against the CPU oracle, through the C ABI."""
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


def _linear(oracle, u, torch, N, K, seed, x=None):
    xh, W, S = oracle.make_q4g32_inputs(1, N, K, seed)
    return dict(W=W, S=S, x=xh if x is None else x, dW=u.dev(W), dS=u.dev(S), N=N, K=K)


# ragged shapes: one group, one group more than a chunk of 64, a partial last chunk (K = 11008: 344 groups),
# fewer rows than wavefronts, more rows than one turn of the grid
SHAPES = [(4096, 4096), (12288, 4096), (22016, 4096), (4096, 11008), (1, 32), (7, 64), (1001, 2080), (130, 11008),
          (5000, 8192), (40000, 256), (64, 16384), (600, 28672), (9, 32736), (70, 32768)]


def test_independent_linears_match_oracle(env, oracle):
    ops, u, torch = env
    lins, outs = [], []
    for i, (N, K) in enumerate(SHAPES):
        l = _linear(oracle, u, torch, N, K, seed=100 + i)
        l["dx"] = u.dev(l["x"])
        l["y"] = torch.zeros((1, N), dtype=torch.float16, device="cuda")
        lins.append(l)
    gl = ops.Q4G32GemvList([(l["dW"], l["dS"], l["dx"], l["y"]) for l in lins])
    assert gl.info() == (0, 0)
    print("gemv list: independent linears", flush=True)
    gl.run()
    gl.status()
    first = [l["y"].clone() for l in lins]
    for l in lins:
        u.assert_close(u.host(l["y"]), oracle.q4g32_linear(l["W"], l["S"], l["x"], nthreads=8), f"list {l['N']}x{l['K']}")
    # launches repeat: the counters clear themselves
    for rep in range(3):
        for l in lins:
            l["y"].zero_()
        gl.run()
        gl.status()
        for l, f in zip(lins, first):
            assert torch.equal(l["y"], f), (rep, l["N"], l["K"])


def test_epilogue_and_one_hot(env, oracle):
    ops, u, torch = env
    N, K = 520, 1024
    x, W, S = oracle.make_q4g32_inputs(1, N, K, seed=7)
    rng = np.random.default_rng(3)
    bias = rng.standard_normal(N).astype(np.float16)
    res = rng.standard_normal((1, N)).astype(np.float16)
    y = torch.zeros((1, N), dtype=torch.float16, device="cuda")
    y2 = torch.zeros((1, N), dtype=torch.float16, device="cuda")
    xh = np.zeros((1, K), np.float16)
    xh[0, 37] = 1
    dW, dS = u.dev(W), u.dev(S)
    gl = ops.Q4G32GemvList([(dW, dS, u.dev(x), y, u.dev(bias), u.dev(res)), (dW, dS, u.dev(xh), y2)])
    gl.run()
    gl.status()
    u.assert_close(u.host(y), oracle.q4g32_linear(W, S, x, bias=bias, residual=res), "list epilogue")
    # a one-hot x selects a dequantized column exactly
    B = oracle.q4g32_dequant(W, S)
    assert np.array_equal(u.host(y2)[0].view(np.uint16), B[:, 37].view(np.uint16))


def test_dependent_chain_matches_oracle(env, oracle):
    """x of a linear is the y of an earlier one: directly in front (two barriers, no overlap) and one apart
    (staged while the linear in between streams); also two consumers of one producer."""
    ops, u, torch = env
    rng = np.random.default_rng(11)
    a = _linear(oracle, u, torch, 4096, 4096, seed=1)     # 0: x0 -> t0
    b = _linear(oracle, u, torch, 22016, 4096, seed=2)    # 1: t0 -> t1   (directly behind its producer)
    c = _linear(oracle, u, torch, 4096, 11008, seed=3)    # 2: independent input -> t2
    d = _linear(oracle, u, torch, 12288, 4096, seed=4)    # 3: t0 -> t3   (second consumer of t0, two apart... three)
    e = _linear(oracle, u, torch, 1024, 4096, seed=5)     # 4: t2 -> t4   (producer two in front)
    x0 = rng.standard_normal((1, 4096)).astype(np.float16)
    xc = (rng.standard_normal((1, 11008)) * 0.5).astype(np.float16)
    t = [torch.zeros((1, n), dtype=torch.float16, device="cuda") for n in (4096, 22016, 4096, 12288, 1024)]
    gl = ops.Q4G32GemvList([(a["dW"], a["dS"], u.dev(x0), t[0]), (b["dW"], b["dS"], t[0], t[1]),
                            (c["dW"], c["dS"], u.dev(xc), t[2]), (d["dW"], d["dS"], t[0], t[3]),
                            (e["dW"], e["dS"], t[2], t[4])])
    assert gl.info() == (3, 1)  # three waits, one of them for the linear directly in front
    print("gemv list: dependent chain", flush=True)
    r0 = oracle.q4g32_linear(a["W"], a["S"], x0, nthreads=8)
    r1 = oracle.q4g32_linear(b["W"], b["S"], r0, nthreads=8)
    r2 = oracle.q4g32_linear(c["W"], c["S"], xc, nthreads=8)
    r3 = oracle.q4g32_linear(d["W"], d["S"], r0, nthreads=8)
    r4 = oracle.q4g32_linear(e["W"], e["S"], r2, nthreads=8)
    for rep in range(3):
        for y in t:
            y.zero_()
        gl.run()
        gl.status()
        for got, ref, name in zip(t, (r0, r1, r2, r3, r4), "abcde"):
            u.assert_close(u.host(got), ref, f"chain {name} rep {rep}")
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


def test_a_long_row_behind_its_producer(env, oracle):
    """The longest rows (K = 28672: 72 KB of staged activations) fed by a linear of the same list, next to a
    second long linear whose activations share the LDS ring with them."""
    ops, u, torch = env
    rng = np.random.default_rng(5)
    up = _linear(oracle, u, torch, 28672, 256, seed=21)     # 0: x0 -> t0 [28672]
    down = _linear(oracle, u, torch, 300, 28672, seed=22)   # 1: t0 -> t1
    other = _linear(oracle, u, torch, 64, 32768, seed=23)   # 2: independent
    x0 = rng.standard_normal((1, 256)).astype(np.float16)
    t = [torch.zeros((1, n), dtype=torch.float16, device="cuda") for n in (28672, 300, 64)]
    gl = ops.Q4G32GemvList([(up["dW"], up["dS"], u.dev(x0), t[0]), (down["dW"], down["dS"], t[0], t[1]),
                            (other["dW"], other["dS"], u.dev(other["x"]), t[2])])
    print("gemv list: long rows", flush=True)
    r0 = oracle.q4g32_linear(up["W"], up["S"], x0, nthreads=8)
    refs = (r0, oracle.q4g32_linear(down["W"], down["S"], r0, nthreads=8),
            oracle.q4g32_linear(other["W"], other["S"], other["x"], nthreads=8))
    for rep in range(2):
        for y in t:
            y.zero_()
        gl.run()
        gl.status()
        for got, ref, name in zip(t, refs, ("up", "down", "other")):
            u.assert_close(u.host(got), ref, f"long rows {name} rep {rep}")


def test_a_linear_without_rows_in_a_workgroup_does_not_disturb_the_ring(env, oracle):
    """A narrow linear (most workgroups hold no row of it) that waits for a large producer, followed by enough long
    linears that the last one is given the narrow one's part of the LDS ring: a workgroup without rows of the narrow
    linear must leave that part alone (it used to stage the narrow linear's activations there late, over the
    activations of the last one)."""
    ops, u, torch = env
    rng = np.random.default_rng(9)
    prod = _linear(oracle, u, torch, 16384, 4096, seed=31)    # 0: x0 -> t0 [16384]
    narrow = _linear(oracle, u, torch, 5, 16384, seed=32)     # 1: t0 -> t1, five rows
    fill = [_linear(oracle, u, torch, 4096, 16384, seed=33 + i) for i in range(4)]  # 2 .. 5: independent
    x0 = rng.standard_normal((1, 4096)).astype(np.float16)
    t = [torch.zeros((1, n), dtype=torch.float16, device="cuda") for n in (16384, 5, 4096, 4096, 4096, 4096)]
    ent = [(prod["dW"], prod["dS"], u.dev(x0), t[0]), (narrow["dW"], narrow["dS"], t[0], t[1])]
    ent += [(f["dW"], f["dS"], u.dev(f["x"]), t[2 + i]) for i, f in enumerate(fill)]
    gl = ops.Q4G32GemvList(ent)
    print("gemv list: a narrow dependent linear in front of long ones", flush=True)
    r0 = oracle.q4g32_linear(prod["W"], prod["S"], x0, nthreads=8)
    refs = [r0, oracle.q4g32_linear(narrow["W"], narrow["S"], r0, nthreads=8)]
    refs += [oracle.q4g32_linear(f["W"], f["S"], f["x"], nthreads=8) for f in fill]
    for rep in range(6):
        for y in t:
            y.zero_()
        gl.run()
        gl.status()
        for i, (got, ref) in enumerate(zip(t, refs)):
            u.assert_close(u.host(got), ref, f"narrow dependent linear: linear {i} rep {rep}")


def test_a_wait_that_runs_out_is_reported_and_every_wavefront_exits(env, oracle):
    """Spin limit 0: the consumer's first look at the producer's counters comes before every workgroup has
    finished the producer, so the wait gives up at once; the launch still ends, status() reports it, and
    the next launch with the normal limit is correct."""
    ops, u, torch = env
    a = _linear(oracle, u, torch, 22016, 4096, seed=21)
    b = _linear(oracle, u, torch, 512, 4096, seed=22)
    x0 = np.random.default_rng(5).standard_normal((1, 4096)).astype(np.float16)
    t0 = torch.zeros((1, 22016), dtype=torch.float16, device="cuda")
    # the consumer reads the first 4096 values of the producer's output
    t1 = torch.zeros((1, 512), dtype=torch.float16, device="cuda")
    gl = ops.Q4G32GemvList([(a["dW"], a["dS"], u.dev(x0), t0), (b["dW"], b["dS"], t0[:, :4096], t1)])
    assert gl.info() == (1, 1)
    from relax_amd._lib import WqError

    gl.set_spin_limit(0)
    print("gemv list: spin limit 0", flush=True)
    gl.run()
    # the non-blocking check: the word lands in pinned host memory behind the launch, nothing synchronises
    word = torch.zeros(1, dtype=torch.int32).pin_memory()
    gl.poll(word)
    torch.cuda.current_stream().synchronize()
    assert word.item() != 0
    with pytest.raises(WqError, match="timed out"):
        gl.status()
    gl.set_spin_limit(200_000_000)
    gl.run()
    gl.poll(word)
    gl.status()
    assert word.item() == 0
    r0 = oracle.q4g32_linear(a["W"], a["S"], x0, nthreads=8)
    u.assert_close(u.host(t0), r0, "producer after a reported time-out")
    u.assert_close(u.host(t1), oracle.q4g32_linear(b["W"], b["S"], r0[:, :4096], nthreads=8), "consumer after a reported time-out")


def test_argument_errors(env, oracle):
    ops, u, torch = env
    from relax_amd._lib import WqError

    a = _linear(oracle, u, torch, 64, 128, seed=1)
    x = u.dev(a["x"])
    y = torch.zeros((1, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(WqError, match="overlaps an operand"):
        ops.Q4G32GemvList([(a["dW"], a["dS"], x, y), (a["dW"], a["dS"], x, y)])  # two linears write one y
    big = torch.zeros((1, 128), dtype=torch.float16, device="cuda")
    with pytest.raises(WqError, match="overlaps an operand"):
        # the second linear overwrites the first one's input
        ops.Q4G32GemvList([(a["dW"], a["dS"], big, y), (a["dW"], a["dS"], x, big[:, :64])])
    with pytest.raises(WqError, match="bias or residual"):
        y2 = torch.zeros((1, 64), dtype=torch.float16, device="cuda")
        ops.Q4G32GemvList([(a["dW"], a["dS"], x, y), (a["dW"], a["dS"], x, y2, None, y)])
    with pytest.raises(WqError, match="more than one linear"):
        # q / k written side by side by two linears and read as one [1, 128] tensor by a third: the
        # consumer could only wait for one of the producers
        qk = torch.zeros((1, 128), dtype=torch.float16, device="cuda")
        y3 = torch.zeros((1, 64), dtype=torch.float16, device="cuda")
        ops.Q4G32GemvList([(a["dW"], a["dS"], x, qk[:, :64]), (a["dW"], a["dS"], x, qk[:, 64:]), (a["dW"], a["dS"], qk, y3)])
    with pytest.raises(ValueError):
        ops.Q4G32GemvList([(a["dW"], a["dS"], x[:, :64], y)])
