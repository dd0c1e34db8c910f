"""Every compute entry point is capturable into a HIP graph (no allocation, no synchronisation inside),
which is what RewriteCUDAGraph relies on for regions that contain these calls
(tests/python/relax/test_codegen_cutlass.py:88-107).  The graph is replayed several times with eager
work in between and every replay is compared with the eager result."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_all_entry_points_in_one_graph(oracle):
    import torch

    from relax_amd import ops
    from tests import gpu_util as u

    rng = np.random.default_rng(3)
    N, K = 256, 512
    _, W, S = oracle.make_q4g32_inputs(1, N, K, seed=1)
    dW, dS = u.dev(W), u.dev(S)
    xs = {M: u.dev(rng.standard_normal((M, K)).astype(np.float16)) for M in (1, 2, 8, 40, 100, 300)}
    wf = u.dev((rng.standard_normal((N, K)) * 0.05).astype(np.float16))
    q8 = u.dev(rng.integers(-127, 128, size=(K, N)).astype(np.int8))
    sc = u.dev(rng.uniform(0.001, 0.01, size=(N,)).astype(np.float16))
    bias = u.dev(rng.standard_normal(N).astype(np.float16))
    _, qw, qz, gsc, g_idx = oracle.make_gptq_inputs(1, N, K, 128, seed=2, act_order=True)
    gw = ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(gsc), u.dev(g_idx))   # load time: synchronises, not captured
    gws = torch.empty((300 * K * 2,), dtype=torch.uint8, device="cuda")     # gathered activations
    outs = {}

    def work():
        for M, x in xs.items():                       # GEMV, small batch, two-pass, GEMM (both tile families)
            outs[f"a{M}"] = ops.q4g32_linear(dW, dS, x, bias=bias, out=outs.get(f"a{M}"))
        outs["deq"] = ops.q4g32_dequantize(dW, dS) if "deq" not in outs else outs["deq"]
        P = ops.ft_preprocess_weight(q8, 80, False) if "P" not in outs else outs["P"]
        outs["P"] = P
        for M in (1, 8, 100, 300):                    # format B: GEMV, small batch, GEMMs
            outs[f"b{M}"] = ops.fpA_intB_gemm(xs[M], P, sc, bias, weight_nbit=8, activation="relu", out=outs.get(f"b{M}"))
        for M in (1, 8, 100, 300):                    # AutoGPTQ: gather + GEMV, small batch, GEMMs
            outs[f"c{M}"] = ops.gptq_linear(gw, xs[M], bias=bias, out=outs.get(f"c{M}"), workspace=gws)

    # first pass allocates every output (outside the capture) and sets one-time kernel attributes
    work()
    torch.cuda.synchronize()
    eager = {k: v.clone() for k, v in outs.items()}
    for v in outs.values():
        if v.dtype == torch.float16:
            v.zero_()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            work()
    for rep in range(3):
        for k in outs:
            if k[0] in "abc":
                outs[k].zero_()                       # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for k in outs:
            if k[0] in "abc":
                assert torch.equal(outs[k], eager[k]), (rep, k)
    # and the eager results are right
    u.assert_close(u.host(eager["a300"]), oracle.q4g32_linear(W, S, u.host(xs[300]), bias=u.host(bias), nthreads=4), "a300")
    u.assert_close(u.host(eager["b100"]),
                   oracle.intb_linear(u.host(xs[100]), u.host(q8), u.host(sc), 8, bias=u.host(bias), activation="relu"), "b100")
    B = oracle.gptq_dequant(qw, qz, gsc, g_idx)
    u.assert_close(u.host(eager["c8"]), oracle.nt_matmul_f32acc(np.ascontiguousarray(B.T), u.host(xs[8]), u.host(bias)), "c8")
