"""wq_gptq_linear_noalloc (the entry point that allocates nothing: gathered activations in a buffer built
into the library) against wq_gptq_linear with a caller workspace, through the C ABI, bit for bit, and
against the oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _call(lib, name, w, x, y, res, M, ws=None):
    import torch

    from relax_amd._lib import check

    s = torch.cuda.current_stream().cuda_stream
    p = lambda t: 0 if t is None else t.data_ptr()
    if name == "wq_gptq_linear":
        check(lib.wq_gptq_linear(p(w.W_nk), p(w.SZ), p(w.perm), p(x), 0, p(res), p(y), M, w.N, w.K, w.G, p(ws),
                                 0 if ws is None else ws.numel(), s), name)
    else:
        check(lib.wq_gptq_linear_noalloc(p(w.W_nk), p(w.SZ), p(w.perm), p(x), 0, p(res), p(y), M, w.N, w.K, w.G, s),
              name)


def test_no_alloc_entry_matches_the_workspace_entry(oracle):
    import torch

    from relax_amd import _lib, ops
    from tests import gpu_util as u

    lib = _lib.lib()
    N, K, gs = 264, 1024, 128
    # two calls in a row on the shared buffer, the second with a smaller input: M = 40 (MFMA path behind the
    # gather), then M = 3 (small batch), then M = 1 (streaming kernel)
    _, qw, qz, s, g_idx = oracle.make_gptq_inputs(1, N, K, gs, seed=51, act_order=True)
    w = ops.gptq_prepare(u.dev(qw), u.dev(qz), u.dev(s), u.dev(g_idx))
    assert w.perm is not None
    B = np.ascontiguousarray(oracle.gptq_dequant(qw, qz, s, g_idx).T)
    for M in (40, 3, 1):
        rng = np.random.default_rng(M)
        x = rng.standard_normal((M, K)).astype(np.float16)
        res = rng.standard_normal((M, N)).astype(np.float16)
        dx, dr = u.dev(x), u.dev(res)
        y_ws = torch.zeros((M, N), dtype=torch.float16, device="cuda")
        y_na = torch.zeros((M, N), dtype=torch.float16, device="cuda")
        ws = torch.empty((M * K * 2,), dtype=torch.uint8, device="cuda")
        print(f"no-alloc M={M}", flush=True)
        _call(lib, "wq_gptq_linear", w, dx, y_ws, dr, M, ws)
        _call(lib, "wq_gptq_linear_noalloc", w, dx, y_na, dr, M)
        torch.cuda.synchronize()
        assert torch.equal(y_ws, y_na), M
        u.assert_close(u.host(y_na), oracle.nt_matmul_f32acc(B, x, None, res, nthreads=4), f"no-alloc M={M}")

    # under stream capture (the address was looked up by the calls above): replays against the eager result
    M = 3
    x = np.random.default_rng(33).standard_normal((M, K)).astype(np.float16)
    dx = u.dev(x)
    y_eager = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    y_graph = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    _call(lib, "wq_gptq_linear_noalloc", w, dx, y_eager, None, M)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            _call(lib, "wq_gptq_linear_noalloc", w, dx, y_graph, None, M)
    for rep in range(3):
        y_graph.zero_()  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_graph, y_eager), rep

    # without a row order nothing is gathered and the buffer is not used
    _, qw2, qz2, s2, g2 = oracle.make_gptq_inputs(1, N, K, gs, seed=52)
    w2 = ops.gptq_prepare(u.dev(qw2), u.dev(qz2), u.dev(s2), u.dev(g2))
    assert w2.perm is None
    x = np.random.default_rng(9).standard_normal((2, K)).astype(np.float16)
    y = torch.zeros((2, N), dtype=torch.float16, device="cuda")
    _call(lib, "wq_gptq_linear_noalloc", w2, u.dev(x), y, None, 2)
    torch.cuda.synchronize()
    u.assert_close(u.host(y), oracle.gptq_linear(qw2, qz2, s2, g2, x), "no-alloc, identity order")

    # beyond the built-in buffer: refused with a clear message, nothing launched
    big_M = (1 << 20) // (K * 2) + 1
    rc = lib.wq_gptq_linear_noalloc(w.W_nk.data_ptr(), w.SZ.data_ptr(), w.perm.data_ptr(), w.W_nk.data_ptr(), 0, 0,
                                    w.W_nk.data_ptr(), big_M, N, K, w.G, 0)
    assert rc != 0 and b"built-in scratch" in lib.wq_last_error()
