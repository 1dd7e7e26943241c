"""The matmul entry points inside a captured HIP graph: no allocation, no synchronisation and no
memset node in any of them, so a model step can be replayed as one graph.  Each replay is checked
against the eagerly computed result for the inputs of that replay, with eager work and
synchronisations between the replays."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from oracle import cpu_oracle as orc  # noqa: E402  (checker only)
from test_gpu_parity import make_inputs  # noqa: E402


def test_graph_replays_match_eager():
    from candle_amd import qhip
    L = qhip.load()
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(21)
    # one call per kernel family: one-launch decode, decode with a fused rms_norm, split-K MFMA (4 rows),
    # dot-product kernel (2 rows of Q8_0), tile kernel with split K (zero fill + atomic adds), grouped experts,
    # two weights in one decode launch
    # (three rows of short weight rows take the one-launch kernel again: "rows")
    cases = [("decode", orc.Q4K, 1, 4096, 512), ("rms", orc.Q6K, 1, 2048, 256), ("rows", orc.Q4K, 3, 1024, 64),
             ("skinny", orc.Q4K, 6, 1024, 64), ("batched", orc.Q8_0, 2, 8192, 40), ("gemm", orc.Q6K, 40, 2048, 64)]
    weights, xs, ys, wss = {}, {}, {}, {}
    for name, dt, m, k, n in cases:
        w, _ = make_inputs(len(name) + k, m, k, n)
        weights[name] = qhip.QWeight.from_ggml(dt, orc.quantize(dt, w), n, k)
        xs[name] = torch.empty((m, k), dtype=torch.float32, device=dev)
        ys[name] = torch.empty((m, n), dtype=torch.float32, device=dev)
        wss[name] = torch.empty(max(weights[name].workspace_bytes(m), 256), dtype=torch.uint8, device=dev)
    alpha = torch.from_numpy((1 + 0.1 * rng.standard_normal(2048)).astype(np.float32)).to(dev)
    n_e, gk, gn = 3, 512, 64
    experts = [qhip.QWeight.from_ggml(orc.Q4K, orc.quantize(orc.Q4K, (rng.standard_normal((gn, gk)) * 0.05).astype(np.float32)),
                                      gn, gk) for _ in range(n_e)]
    offsets = np.array([0, 9, 9, 30], dtype=np.int32)
    gx = torch.empty((30, gk), dtype=torch.float32, device=dev)
    gy = torch.empty((30, gn), dtype=torch.float32, device=dev)
    arr = (C.c_void_p * n_e)(*[e.handle.value for e in experts])
    gws = torch.empty(L.cq_grouped_workspace_bytes(arr, n_e, 30, 0), dtype=torch.uint8, device=dev)

    # two weights on the decode case's input in one launch
    pair = [weights["decode"], qhip.QWeight.from_ggml(orc.Q4K, orc.quantize(orc.Q4K, make_inputs(77, 1, 4096, 128)[0]), 128, 4096)]
    pair_y = [torch.empty((1, 512), dtype=torch.float32, device=dev), torch.empty((1, 128), dtype=torch.float32, device=dev)]
    pair_w = (C.c_void_p * 2)(*[w.handle for w in pair])
    pair_o = (C.c_void_p * 2)(*[t.data_ptr() for t in pair_y])

    def step():
        s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        qhip.check(L.cq_qmatmul_multi(pair_w, 2, qhip.PRE_NONE, C.c_void_p(xs["decode"].data_ptr()), None, 0.0, 1, pair_o, 0,
                                      C.c_void_p(wss["decode"].data_ptr()), wss["decode"].numel(), s))
        for name, dt, m, k, n in cases:
            args = (C.c_void_p(xs[name].data_ptr()), m, C.c_void_p(ys[name].data_ptr()), 0,
                    C.c_void_p(wss[name].data_ptr()), wss[name].numel(), s)
            if name == "rms":
                qhip.check(L.cq_qmatmul_fused(weights[name].handle, qhip.PRE_RMS_NORM, args[0], C.c_void_p(alpha.data_ptr()),
                                              1e-5, *args[1:]))
            else:
                qhip.check(L.cq_qmatmul(weights[name].handle, *args))
        qhip.check(L.cq_qmatmul_grouped(arr, n_e, C.c_void_p(gx.data_ptr()), None, offsets.ctypes.data_as(C.POINTER(C.c_int32)),
                                        C.c_void_p(gy.data_ptr()), 0, C.c_void_p(gws.data_ptr()), gws.numel(), s))

    def fill(seed):
        g = torch.Generator(device=dev)
        g.manual_seed(seed)
        for t in list(xs.values()) + [gx]:
            t.copy_(torch.randn(t.shape, generator=g, device=dev))

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        fill(0)
        step()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step()
        for seed in (1, 2, 3, 4):
            fill(seed)
            step()                                   # eager, same inputs
            torch.cuda.synchronize()
            want = {k: v.clone() for k, v in ys.items()}
            want_g = gy.clone()
            want_p = [t.clone() for t in pair_y]
            for t in list(ys.values()) + [gy] + pair_y:
                t.fill_(float("nan"))                # eager work between the replays; also proves the replay writes
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for name, *_ in cases:
                if name == "gemm":   # split K adds its partial sums atomically: equal up to the order of the additions
                    assert torch.allclose(ys[name], want[name], rtol=1e-5, atol=1e-6), (seed, name)
                else:
                    assert torch.equal(ys[name], want[name]), (seed, name)
            assert torch.allclose(gy, want_g, rtol=1e-5, atol=1e-6), seed
            assert torch.equal(pair_y[0], want_p[0]) and torch.equal(pair_y[1], want_p[1]), seed
            assert torch.equal(pair_y[0], ys["decode"]), seed   # the same rows as the weight's own call
