"""wq_gptq_gemv_list_create: a list of prepared AutoGPTQ layers at M = 1 in one launch, against the CPU oracle
(the fp32-accumulated matmul over the bit-exact dequantized weight) and against wq_gptq_linear, through the C ABI."""
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


def _layer(oracle, ops, u, N, K, gs, seed, shrink=1.0, act_order=False):
    x, qw, qz, s, g_idx = oracle.make_gptq_inputs(1, N, K, gs, seed=seed, act_order=act_order)
    s = (s.astype(np.float32) * shrink).astype(np.float16)
    w = ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
    assert (w.perm is not None) == act_order
    B = oracle.gptq_dequant(qw, qz, s, g_idx)  # fp16 [K, N]
    return dict(w=w, x=x, Bt=np.ascontiguousarray(B.T), N=N, K=K, gs=gs)


def _ref(oracle, l, x, bias=None, residual=None):
    return oracle.nt_matmul_f32acc(l["Bt"], x, bias, residual, nthreads=8)


# (N, K, group size): the usual 128, every supported size from 32 to 2048, one group per row, a partial last chunk
# of 64 x 32 columns (K = 11008, 4224), fewer rows than wavefronts, more rows than one turn of the grid, N % 8 == 0
SHAPES = [(4096, 4096, 128), (12288, 4096, 128), (4096, 11008, 128), (8, 32, 32), (72, 64, 32), (1000, 2112, 64),
          (136, 11008, 64), (5000, 8192, 256), (40000, 256, 128), (64, 16384, 512), (328, 8192, 1024),
          (520, 4096, 2048), (96, 2048, 2048), (600, 28672, 128), (16, 32768, 32), (200, 4224, 128), (88, 1024, 1024)]


@pytest.mark.parametrize("act_order,gather_in_front", [(False, True), (True, True), (True, False)])
def test_independent_layers_match_oracle_and_call_by_call(env, oracle, act_order, gather_in_front):
    """With ``act_order`` every layer but each third has a row order (a random assignment of the rows to the groups,
    what AutoGPTQ's desc_act leaves): its activations are gathered by a kernel in front of the list, or, in a
    workspace of the plain size (``gather_in_front=False``), inside the list kernel while they are staged."""
    ops, u, torch = env
    lins = []
    for i, (N, K, gs) in enumerate(SHAPES):
        l = _layer(oracle, ops, u, N, K, gs, seed=300 + i, act_order=act_order and i % 3 != 2 and K > gs)
        l["dx"] = u.dev(l["x"])
        l["y"] = torch.zeros((1, N), dtype=torch.float16, device="cuda")
        lins.append(l)
    gl = ops.GptqGemvList([(l["w"], l["dx"], l["y"]) for l in lins], gather_in_front=gather_in_front)
    assert gl.info() == (0, 0)
    print("gptq list: independent layers", flush=True)
    gl.run()
    gl.status()
    first = [l["y"].clone() for l in lins]
    for l in lins:
        name = f"gptq list {l['N']}x{l['K']} g{l['gs']}"
        u.assert_close(u.host(l["y"]), _ref(oracle, l, l["x"]), name)
        u.assert_close(u.host(l["y"]), u.host(ops.gptq_linear(l["w"], l["dx"])), name + " against wq_gptq_linear")
    for rep in range(3):  # launches repeat: the counters clear themselves
        for l in lins:
            l["y"].zero_()
        gl.run()
        gl.status()
        for l, f in zip(lins, first):
            assert torch.equal(l["y"], f), (rep, l["N"], l["K"])


def test_epilogue_and_one_hot(env, oracle):
    ops, u, torch = env
    rng = np.random.default_rng(3)
    for N, K, gs, act, front in [(520, 1024, 128, False, True), (264, 4224, 64, False, True), (264, 4224, 64, True, True),
                                 (264, 4224, 64, True, False), (72, 2048, 32, True, False)]:
        l = _layer(oracle, ops, u, N, K, gs, seed=7, act_order=act)
        bias = rng.standard_normal(N).astype(np.float16)
        res = rng.standard_normal((1, N)).astype(np.float16)
        y = torch.zeros((1, N), dtype=torch.float16, device="cuda")
        hot = []
        for k in (0, 37, gs - 1, gs, K - 1):
            xh = np.zeros((1, K), np.float16)
            xh[0, k] = 1
            hot.append((k, u.dev(xh), torch.zeros((1, N), dtype=torch.float16, device="cuda")))
        gl = ops.GptqGemvList([(l["w"], u.dev(l["x"]), y, u.dev(bias), u.dev(res))] + [(l["w"], dx, yh) for _, dx, yh in hot],
                              gather_in_front=front)
        gl.run()
        gl.status()
        u.assert_close(u.host(y), _ref(oracle, l, l["x"], bias, res), "gptq list epilogue")
        # a one-hot x selects a dequantized row of the [K, N] weight exactly
        for k, _, yh in hot:
            assert np.array_equal(u.host(yh)[0].view(np.uint16), l["Bt"][:, k].view(np.uint16)), (N, K, gs, act, k)


@pytest.mark.parametrize("act_order", [False, True])
def test_decoder_layer_chain(env, oracle, act_order):
    """The four linears of a Llama-2-7B decoder layer at group size 128, each fed by the one in front (qkv -> o
    takes the first 4096 of qkv's outputs, gate/up -> down the first 11008), eager and as a replayed HIP graph.
    (Scales a twentieth of the generator's: its weights have mean -scale, which a chain of four would amplify
    beyond fp16.)  With ``act_order`` the consumers gather what their producers wrote."""
    ops, u, torch = env
    rng = np.random.default_rng(11)
    qkv = _layer(oracle, ops, u, 12288, 4096, 128, seed=1, shrink=0.05, act_order=act_order)
    o = _layer(oracle, ops, u, 4096, 4096, 128, seed=2, shrink=0.05, act_order=act_order)
    gu = _layer(oracle, ops, u, 22016, 4096, 128, seed=3, shrink=0.05, act_order=act_order)
    down = _layer(oracle, ops, u, 4096, 11008, 128, seed=4, shrink=0.05, act_order=act_order)
    x0 = rng.standard_normal((1, 4096)).astype(np.float16)
    res = rng.standard_normal((1, 4096)).astype(np.float16)
    t = [torch.zeros((1, n), dtype=torch.float16, device="cuda") for n in (12288, 4096, 22016, 4096)]
    dres = u.dev(res)
    gl = ops.GptqGemvList([(qkv["w"], u.dev(x0), t[0]), (o["w"], t[0][:, :4096], t[1], None, dres),
                           (gu["w"], t[1], t[2]), (down["w"], t[2][:, :11008], t[3], None, dres)])
    assert gl.info() == (3, 3)
    print("gptq list: decoder layer", flush=True)
    r0 = _ref(oracle, qkv, x0)
    r1 = _ref(oracle, o, np.ascontiguousarray(r0[:, :4096]), None, res)
    r2 = _ref(oracle, gu, r1)
    r3 = _ref(oracle, down, np.ascontiguousarray(r2[:, :11008]), None, res)
    for rep in range(3):
        for y in t:
            y.zero_()
        gl.run()
        gl.status()
        for got, ref, name in zip(t, (r0, r1, r2, r3), ("qkv", "o", "gate_up", "down")):
            u.assert_close(u.host(got), ref, f"gptq chain {name} rep {rep}")
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


def test_what_the_list_refuses(env, oracle):
    ops, u, torch = env
    from relax_amd import _lib

    x, qw, qz, s, g_idx = oracle.make_gptq_inputs(1, 64, 192, 96, seed=5)  # group size 96: not 32 << t
    w = ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
    y = torch.zeros((1, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.WqError, match="group size"):
        ops.GptqGemvList([(w, u.dev(x), y)])
    # an error found by the code shared with the q4f16_1 lists names the entry point that was called
    x2, qw2, qz2, s2, g2 = oracle.make_gptq_inputs(1, 64, 64, 32, seed=8)
    w2 = ops.gptq_prepare(u.dev(qw2), u.dev(qz2), u.dev(s2), u.dev(g2))
    with pytest.raises(_lib.WqError, match="wq_gptq_gemv_list_create: linear 0: y overlaps x"):
        ops.GptqGemvList([(w2, y, y)])
    g_idx = np.random.default_rng(1).integers(0, 2, size=192).astype(np.int32)  # groups of unequal size
    w = ops.gptq_prepare_padded(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
    with pytest.raises(ValueError, match="padded"):
        ops.GptqGemvList([(w, u.dev(x), y)])


def test_the_gathered_copy_follows_the_input_between_launches(env, oracle):
    """A layer with a row order fed from outside the list: the gather in front of the list kernel runs at every launch,
    so new contents of x are seen (eager and in a replayed graph)."""
    ops, u, torch = env
    l = _layer(oracle, ops, u, 136, 1024, 128, seed=12, act_order=True)
    dx = torch.zeros((1, 1024), dtype=torch.float16, device="cuda")
    y = torch.zeros((1, 136), dtype=torch.float16, device="cuda")
    gl = ops.GptqGemvList([(l["w"], dx, y)])
    rng = np.random.default_rng(13)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        gl.run()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            gl.run()
    for rep in range(4):
        x = rng.standard_normal((1, 1024)).astype(np.float16)
        dx.copy_(u.dev(x))
        torch.cuda.synchronize()
        if rep % 2:
            graph.replay()
        else:
            gl.run()
        torch.cuda.synchronize()
        u.assert_close(u.host(y), _ref(oracle, l, x), f"new x, launch {rep}")
    gl.status()
