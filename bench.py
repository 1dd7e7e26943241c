#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

Workload (BASELINE.json configs[1]): the Llama-2-7B-shaped decode QMatMul stack at batch 1 -
per layer q/k/v/o [4096x4096] Q4_K, gate/up [11008x4096] Q4_K, down [4096x11008] Q6_K, 32 layers,
plus an lm_head [32000x4096] Q6_K; activations f32 N(0,1) quantized to Q8_K.  A "step" is one
pass over all 225 QMatMul calls (4 122 255 360 bytes of GGML weights, all distinct, so every call
streams from HBM and not from the 256 MB Infinity Cache).  Weights are random N(0,0.02) drawn and
quantized on the device (bit-identical to the CPU quantizer, see tests).

Prints ONE JSON line.  `value` = GGML weight bytes per step / time per step (inputs resident in
HBM).  `roofline` covers the dominant kernel, the Q4_K decode matvec: algorithmic bytes per launch
divided by its average launch duration, measured here with HIP events recorded around each launch.
`cpu_baseline` times the restated candle CPU QMatMul (AVX2 + threads) on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak
# HBM bytes per Q4_K decode launch (mean over the step's 192 launches), from two rocprofv3 --pmc runs
# of this script (FETCH_SIZE, then WRITE_SIZE), each scaled by what the counter reads for a plain
# 256 MiB device copy (x2.000 and x1.000); see profiles/decode_stack_q4k_matvec_hbm_traffic.md.
Q4K_DECODE_TRAFFIC_BYTES_PER_LAUNCH = 15_400_448

LAYERS = 32
HIDDEN, FFN, VOCAB = 4096, 11008, 32000
# (name, dtype name, n, k, input id) per layer, in the order ModelWeights::forward issues them
# (candle-transformers/src/models/quantized_llama.rs:483-511)
LAYER_SHAPES = [
    ("attn_q", "q4k", HIDDEN, HIDDEN, "x_attn"), ("attn_k", "q4k", HIDDEN, HIDDEN, "x_attn"),
    ("attn_v", "q4k", HIDDEN, HIDDEN, "x_attn"), ("attn_o", "q4k", HIDDEN, HIDDEN, "x_o"),
    ("ffn_gate", "q4k", FFN, HIDDEN, "x_ffn"), ("ffn_up", "q4k", FFN, HIDDEN, "x_ffn"),
    ("ffn_down", "q6k", HIDDEN, FFN, "x_down"),
]


def ggml_bytes(dtype: str, n: int, k: int) -> int:
    blk, size = {"q4k": (256, 144), "q6k": (256, 210), "q4_0": (32, 18), "q8_0": (32, 34)}[dtype]
    return n * k // blk * size


def envelope() -> int:
    """What one launch can reach on this device: an empty kernel (the fixed cost of a launch) and a pure
    streaming read (16 bytes per lane and step, four steps in flight, nothing else) of the byte counts of the
    decode launches, back to back eagerly and as a chain of 225 graph nodes like the decode step.  Every
    launch of a chain reads a buffer of its own (4 GB in rotation: HBM, not the 256 MB Infinity Cache)."""
    import ctypes as C

    import torch

    from candle_amd import build as qbuild

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    P = C.CDLL(qbuild.PROBE_LIB_PATH)
    vp = C.c_void_p
    P.cqp_empty.argtypes = [C.c_int, C.c_int, C.c_int, vp, vp]
    P.cqp_stream_read.argtypes = [vp, C.c_size_t, C.c_int, C.c_int, C.c_int, vp, vp]
    P.cqp_stream_read_pol.argtypes = [vp, C.c_size_t, C.c_int, C.c_int, C.c_int, vp, vp]
    P.cqp_lds_read.argtypes = [vp, C.c_size_t, C.c_int, C.c_int, C.c_int, vp, vp]
    P.cqp_lds_read_rows.argtypes = [vp, C.c_size_t, C.c_int, C.c_int, vp, vp]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    pool = torch.full(((4 << 30) // 4,), 1, dtype=torch.int32, device=dev)
    NODES = 225

    def timed(launch, graph: bool):
        """µs per launch of NODES launches, eagerly or as one graph replay (median of 7)."""
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            s = vp(side.cuda_stream)
            for i in range(NODES):
                launch(i, s)
            torch.cuda.synchronize()
            g = None
            if graph:
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=side):
                    for i in range(NODES):
                        launch(i, s)
            times = []
            for _ in range(7):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                if g is not None:
                    g.replay()
                else:
                    for i in range(NODES):
                        launch(i, s)
                e1.record()
                torch.cuda.synchronize()
                times.append(e0.elapsed_time(e1) * 1e3 / NODES)
        return sorted(times)[len(times) // 2]

    out = {"nodes_per_chain": NODES, "empty_kernel_us": {}, "stream_read": {}}
    for grid, block, lds in ((256, 512, 0), (256, 512, 20480), (256, 256, 0), (256, 64, 0), (1, 64, 0), (2048, 256, 0)):
        def launch(i, s, grid=grid, block=block, lds=lds):
            P.cqp_empty(grid, block, lds, vp(sink.data_ptr()), s)
        out["empty_kernel_us"][f"grid{grid}_block{block}_lds{lds}"] = {
            "eager": round(timed(launch, False), 3), "graph": round(timed(launch, True), 3)}
    # the byte counts of the decode launches: Q4_K 4096x4096, Q4_K 11008x4096, Q6_K 4096x11008, Q6_K 32000x4096
    for name, nbytes in (("q4k_4096x4096", 9437184), ("q4k_11008x4096", 25362432), ("q6k_4096x11008", 36986880),
                         ("q6k_32000x4096", 107520000)):
        span = (nbytes + 4095) // 4096 * 4096
        slots = pool.numel() * 4 // span
        row = {"bytes": nbytes}
        for grid, block, unroll in ((2048, 256, 4), (1024, 512, 4), (256, 512, 8)):
            def launch(i, s, grid=grid, block=block, unroll=unroll):
                P.cqp_stream_read(vp(pool.data_ptr() + (i % slots) * span), nbytes, grid, block, unroll,
                                  vp(sink.data_ptr()), s)
            for mode, graph in (("eager", False), ("graph", True)):
                us = timed(launch, graph)
                row[f"grid{grid}_block{block}_u{unroll}_{mode}_us"] = round(us, 3)
                row[f"grid{grid}_block{block}_u{unroll}_{mode}_GBs"] = round(nbytes / us / 1e3, 1)
        # cache-policy bits on the loads (1 = sc0, 2 = nt, 16 = sc1), graph replay only
        for aux in (0, 1, 2, 3, 16, 17, 18, 19):
            def launch(i, s, aux=aux):
                rc = P.cqp_stream_read_pol(vp(pool.data_ptr() + (i % slots) * span), nbytes, 2048, 256, aux,
                                           vp(sink.data_ptr()), s)
                assert rc == 0, rc
            row[f"bufload_aux{aux}_graph_us"] = round(timed(launch, True), 3)
        # requests that land in LDS, a ring of 1-KiB slots per wave (8 waves per workgroup)
        for grid, ring, aux in ((256, 4, 0), (256, 8, 0), (256, 16, 0), (512, 8, 0), (512, 4, 0), (256, 16, 2), (256, 8, 2),
                                (256, 16, 16)):
            def launch(i, s, grid=grid, ring=ring, aux=aux):
                rc = P.cqp_lds_read(vp(pool.data_ptr() + (i % slots) * span), nbytes, grid, ring, aux,
                                    vp(sink.data_ptr()), s)
                assert rc == 0, rc
            row[f"lds_grid{grid}_ring{ring}_aux{aux}_graph_us"] = round(timed(launch, True), 3)
        # the same requests with a wave owning whole rows of P consecutive KiB (the decode kernels' ownership)
        for ppr in (1, 2, 3, 6, 9):
            def launch(i, s, ppr=ppr):
                rc = P.cqp_lds_read_rows(vp(pool.data_ptr() + (i % slots) * span), nbytes, 256, ppr, vp(sink.data_ptr()), s)
                assert rc == 0, rc
            row[f"lds_rows_of_{ppr}KiB_ring8_aux2_graph_us"] = round(timed(launch, True), 3)
        out["stream_read"][name] = row
    print(json.dumps(out), flush=True)
    return 0


def config3_activations(torch, gen, m, k, dev):
    """BASELINE configs[3]: f32 N(0,1) with 1 % of the positions at +-8 sigma (the time of an int8 MFMA depends on its
    operands' bits, so the prefill figures are timed on the configuration's own inputs)."""
    x = torch.randn((m, k), generator=gen, device=dev, dtype=torch.float32)
    pos = torch.rand((m, k), generator=gen, device=dev) < 0.01
    sign = torch.rand((m, k), generator=gen, device=dev) < 0.5
    return torch.where(pos, torch.where(sign, torch.full_like(x, 8.0), torch.full_like(x, -8.0)), x)


def mfma_clock_probe(torch):
    """Shader clock with every matrix pipe busy (ratio of the shader-clock counter to the constant 100 MHz counter inside a
    10 ms kernel of int8 MFMA chains, two waves per SIMD; the clock ramps up over the first milliseconds of load) and the
    time per 32x32x32 int8 MFMA and SIMD from the kernel's duration between two HIP events (probe library)."""
    import ctypes as C

    from candle_amd import build as qbuild
    try:
        P = C.CDLL(qbuild.PROBE_LIB_PATH)
        P.cqp_mfma_clock.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        out = torch.zeros(2, dtype=torch.int64, device="cuda")
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        iters = 16000
        rc = P.cqp_mfma_clock(iters, C.c_void_p(out.data_ptr()), C.c_void_p(sink.data_ptr()), s)
        assert rc == 0, rc
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        rc = P.cqp_mfma_clock(iters, C.c_void_p(out.data_ptr()), C.c_void_p(sink.data_ptr()), s)
        e1.record()
        assert rc == 0, rc
        torch.cuda.synchronize()
        cyc, ticks = (int(v) for v in out.cpu().tolist())
        ghz = cyc / (ticks * 10.0)          # ticks of 10 ns
        per_mfma_ns = e0.elapsed_time(e1) * 1e6 / (iters * 16 * 2)   # two waves per SIMD, sixteen MFMAs per iteration
        return {"shader_clock_ghz_all_matrix_pipes_busy": round(ghz, 3),
                "ns_per_32x32x32_i8_mfma_per_simd": round(per_mfma_ns, 2),
                "cycles_per_mfma": round(per_mfma_ns * ghz, 1),
                "int8_peak_at_that_clock_tops": round(5000.0 * ghz / 2.4, 0),
                "note": "the published 5000 TOP/s assume 2.4 GHz; pseudo-random operands"}
    except Exception as e:   # the probe library is an aid: the bench line stands without it
        return {"error": "%s: %s" % (type(e).__name__, e)}


def small_batch_probe(rounds: int, copy_probe: bool = False) -> int:
    """configs[2] alone, for a profiler run: whole cq_qmatmul calls with 2, 8 and 16 activation rows on Q4_K and
    Q8_0 weights of both decode shapes, launched eagerly `rounds` times over sixteen distinct weights per shape
    (each call streams its weights from HBM), and the same timed with HIP events.  One JSON line."""
    import ctypes as C

    import torch

    from candle_amd import qhip

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    L = qhip.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev)
    vp = C.c_void_p
    out = {"rounds": rounds, "weights_per_shape": 16, "whole_call_us": {}}
    if copy_probe:   # a kernel of known HBM traffic, to calibrate FETCH_SIZE / WRITE_SIZE
        src = torch.full((64 * 1024 * 1024,), 1.0, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for dtname, dt in (("q4k", qhip.Q4K), ("q8_0", qhip.Q8_0)):
        for n_out in (HIDDEN, FFN):
            weights = []
            for t in range(16):
                gen.manual_seed(70_000 + 100 * dt + n_out + t)
                w_ = torch.randn((n_out, HIDDEN), generator=gen, device=dev, dtype=torch.float32) * 0.02
                weights.append(qhip.QWeight.zeros(dt, n_out, HIDDEN).quantize_(w_))
                del w_
            for mb in (2, 8, 16):
                xb = torch.randn((mb, HIDDEN), generator=gen, device=dev, dtype=torch.float32)
                yb = torch.empty((mb, n_out), device=dev, dtype=torch.float32)
                wsb = torch.empty(max(weights[0].workspace_bytes(mb), 256), dtype=torch.uint8, device=dev)
                s = vp(torch.cuda.current_stream().cuda_stream)

                def sweep():
                    for qw in weights:
                        qhip.check(L.cq_qmatmul(qw.handle, vp(xb.data_ptr()), mb, vp(yb.data_ptr()), 0, vp(wsb.data_ptr()),
                                                wsb.numel(), s))
                sweep()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(rounds):
                    sweep()
                e1.record()
                torch.cuda.synchronize()
                out["whole_call_us"]["%s_%dx%d_m%d_eager" % (dtname, n_out, HIDDEN, mb)] = round(
                    e0.elapsed_time(e1) * 1e3 / (rounds * len(weights)), 2)
            del weights
    print(json.dumps(out), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    # (the part reaches its steady clocks some tens of milliseconds into a run: with 3 warm-up steps the first timed
    # region reads 2-4 % slower than the same steps timed a moment later)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--layers", type=int, default=LAYERS, help="(debug) fewer layers; the result is then not a bench line")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the figures reported beside the headline (fused neighbours, merged projections), "
                         "so that a profiler run sees the headline kernels only")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain device copy of 256 MiB three times (a kernel of known HBM traffic, to "
                         "calibrate FETCH_SIZE / WRITE_SIZE counters in a profiler run)")
    ap.add_argument("--envelope", action="store_true",
                    help="instead of the bench: time an empty kernel and a pure 16-byte-per-lane streaming read of the "
                         "decode launches' sizes, eagerly and as a 225-node graph chain (what a single launch can reach "
                         "on this device), and print that as one JSON line")
    ap.add_argument("--small-batch", type=int, default=0, metavar="ROUNDS",
                    help="instead of the bench: only the small-batch calls (2, 8, 16 rows; Q4_K and Q8_0; both decode "
                         "shapes), launched eagerly ROUNDS times, for a profiler run; prints one JSON line")
    args = ap.parse_args()
    if args.envelope:
        return envelope()
    if args.small_batch > 0:
        return small_batch_probe(args.small_batch, args.copy_probe)
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (one process, one MI355X); --gpus must be 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from candle_amd import qhip

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    L = qhip.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    DT = {"q4k": qhip.Q4K, "q6k": qhip.Q6K}

    # ---- synthetic weights, quantized on the device --------------------------------------
    t0 = time.time()
    gen = torch.Generator(device=dev)
    calls = []  # (QWeight, input name, dtype name, n, k)
    for layer in range(args.layers):
        for idx, (name, dt, n, k, xin) in enumerate(LAYER_SHAPES):
            gen.manual_seed(1000 * layer + idx)
            w = torch.randn((n, k), generator=gen, device=dev, dtype=torch.float32) * 0.02
            calls.append((qhip.QWeight.zeros(DT[dt], n, k).quantize_(w), xin, dt, n, k))
            del w
    gen.manual_seed(999_999)
    w = torch.randn((VOCAB, HIDDEN), generator=gen, device=dev, dtype=torch.float32) * 0.02
    calls.append((qhip.QWeight.zeros(qhip.Q6K, VOCAB, HIDDEN).quantize_(w), "x_head", "q6k", VOCAB, HIDDEN))
    del w
    torch.cuda.synchronize()
    t_setup = time.time() - t0

    gen.manual_seed(7)
    inputs = {name: torch.randn((1, k), generator=gen, device=dev, dtype=torch.float32)
              for name, k in (("x_attn", HIDDEN), ("x_o", HIDDEN), ("x_ffn", HIDDEN), ("x_down", FFN), ("x_head", HIDDEN))}
    outputs = [torch.empty((1, n), device=dev, dtype=torch.float32) for (_, _, _, n, _) in calls]
    ws_bytes = max(qw.workspace_bytes(1) for (qw, *_rest) in calls)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    bytes_per_step = sum(ggml_bytes(dt, n, k) for (_, _, dt, n, k) in calls)

    import ctypes as C

    def run_call(i, flags=0, stream=None):
        qw, xin, _, _, _ = calls[i]
        s = stream if stream is not None else C.c_void_p(torch.cuda.current_stream().cuda_stream)
        qhip.check(L.cq_qmatmul(qw.handle, C.c_void_p(inputs[xin].data_ptr()), 1, C.c_void_p(outputs[i].data_ptr()),
                                flags, C.c_void_p(ws.data_ptr()), ws.numel(), s))

    def step():
        s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        for i in range(len(calls)):
            run_call(i, 0, s)

    if args.copy_probe:
        src = torch.full((64 * 1024 * 1024,), 1.0, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- timed region ----------------------------------------------------------------------
    side = torch.cuda.Stream()
    graph = None
    with torch.cuda.stream(side):
        for _ in range(max(args.warmup, 1)):
            step()
        torch.cuda.synchronize()
        if not args.no_graph:
            try:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    step()
                graph.replay()
                torch.cuda.synchronize()
            except Exception as e:  # capture refused: fall back to eager launches and say so
                print(f"bench.py: graph capture failed ({e}); timing eager launches", file=sys.stderr)
                graph = None
        # The same K steps are timed as eager launches (what candle's own call sites do: one launch per
        # QMatMul::forward, the host running ahead of the device) and, unless --no-graph, as replays of the captured
        # graph; `value` is the faster of the two and `config.launch` names it.
        def time_steps(run):
            for _ in range(args.warmup):
                run()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(args.steps):
                run()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / args.steps

        ms_by_launch = {"eager": time_steps(step)}
        if graph is not None:
            ms_by_launch["hip graph replay"] = time_steps(graph.replay)
        launch_mode = min(ms_by_launch, key=ms_by_launch.get)
        ms_per_step = ms_by_launch[launch_mode]

        # ---- dominant kernel: the Q4_K decode matvec (activation quantizer fused in) ----------
        # Each Q4_K launch of the step is timed once per pass by a pair of HIP events that the
        # library records around that kernel on its stream, while the whole step runs eagerly
        # around it, so the kernel sees the same cache and clock state as in the timed region.
        q4k_calls = [i for i, c in enumerate(calls) if c[2] == "q4k"]
        durs, alg_bytes = [], []
        s_here = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        for rep in range(2):
            for target in q4k_calls:
                for i in range(len(calls)):
                    if i == target:
                        us = qhip.timed_kernel_us(lambda: run_call(i, 0, s_here))
                    else:
                        run_call(i, 0, s_here)
                if rep == 0:
                    continue  # first pass warms the instrumented path
                _, _, dt, n, k = calls[target]
                durs.append(us * 1e-6)
                # weights + f32 activations read + f32 outputs written
                alg_bytes.append(ggml_bytes(dt, n, k) + 4 * k + 4 * n)
            torch.cuda.synchronize()
        eager_avg_dur = sum(durs) / len(durs)
        # The same launches back to back, as in the timed region: a HIP graph of the Q4_K calls
        # alone, replayed between two events on this stream; time / launches bounds the kernel's
        # average duration from above (it includes the dispatch gaps between kernels).
        avg_dur = eager_avg_dur
        if graph is not None:
            g4 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g4, stream=side):
                s_cap = C.c_void_p(torch.cuda.current_stream().cuda_stream)
                for i in q4k_calls:
                    run_call(i, 0, s_cap)
            for _ in range(3):
                g4.replay()
            torch.cuda.synchronize()
            f0, f1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            f0.record()
            for _ in range(args.steps):
                g4.replay()
            f1.record()
            torch.cuda.synchronize()
            avg_dur = f0.elapsed_time(f1) * 1e-3 / (args.steps * len(q4k_calls))
    avg_bytes = sum(alg_bytes) / len(alg_bytes)
    achieved = avg_bytes / avg_dur / 1e9
    # headline shape alone (gate/up, 11008x4096)
    big = [(d, b) for d, b in zip(durs, alg_bytes) if b > 20_000_000]
    big_gbs = (sum(b for _, b in big) / sum(d for d, _ in big) / 1e9) if big else None
    small = [(d, b) for d, b in zip(durs, alg_bytes) if b <= 20_000_000]
    small_gbs = (sum(b for _, b in small) / sum(d for d, _ in small) / 1e9) if small else None

    # ---- the other half of the metric: Q4_K prefill GEMM, M = 512 on the Mistral FFN shape ----
    # (BASELINE.json configs[3]; reported beside the headline, not as `value`)
    gm, gk, gn = 512, 4096, 14336
    gen.manual_seed(4242)
    gw = torch.randn((gn, gk), generator=gen, device=dev, dtype=torch.float32) * 0.02
    gq = qhip.QWeight.zeros(qhip.Q4K, gn, gk).quantize_(gw)
    del gw
    gx = config3_activations(torch, gen, gm, gk, dev)
    gy = torch.empty((gm, gn), device=dev, dtype=torch.float32)
    gws = torch.empty(gq.workspace_bytes(gm), dtype=torch.uint8, device=dev)

    def gemm_call(flags):
        qhip.check(L.cq_qmatmul(gq.handle, C.c_void_p(gx.data_ptr()), gm, C.c_void_p(gy.data_ptr()), flags,
                                C.c_void_p(gws.data_ptr()), gws.numel(),
                                C.c_void_p(torch.cuda.current_stream().cuda_stream)))

    # (thirty calls ahead of every timed one: reading a time synchronises, the part idles and drops its clocks, and a
    # few calls are not enough to bring them back - four calls ahead read 82 us where back-to-back calls take 74)
    gemm_us = []
    for rep in range(12):
        for _ in range(30):
            gemm_call(0)
        us = qhip.timed_kernel_us(lambda: gemm_call(0))
        if rep >= 2:
            gemm_us.append(us)
    gemm_avg_us = sum(gemm_us) / len(gemm_us)
    gemm_tops = 2.0 * gm * gk * gn / (gemm_avg_us * 1e-6) / 1e12
    del gq, gx, gy, gws

    # whole calls (activation quantizer + GEMM) on both shapes of configs[3] and on the attention shape
    whole_calls = {}
    gemm_cases = {}
    if not args.no_extras:
        for name, dt, (wn, wk) in (("q4k_14336x4096", qhip.Q4K, (14336, 4096)), ("q4k_4096x14336", qhip.Q4K, (4096, 14336)),
                                   ("q6k_14336x4096", qhip.Q6K, (14336, 4096)), ("q6k_4096x14336", qhip.Q6K, (4096, 14336)),
                                   ("q4k_4096x4096", qhip.Q4K, (4096, 4096))):
            ww = torch.randn((wn, wk), generator=gen, device=dev, dtype=torch.float32) * 0.02
            wq = qhip.QWeight.zeros(dt, wn, wk).quantize_(ww)
            del ww
            wx = config3_activations(torch, gen, gm, wk, dev)
            wy = torch.empty((gm, wn), device=dev, dtype=torch.float32)
            wws = torch.empty(wq.workspace_bytes(gm), dtype=torch.uint8, device=dev)

            def whole():
                qhip.check(L.cq_qmatmul(wq.handle, C.c_void_p(wx.data_ptr()), gm, C.c_void_p(wy.data_ptr()), 0,
                                        C.c_void_p(wws.data_ptr()), wws.numel(),
                                        C.c_void_p(torch.cuda.current_stream().cuda_stream)))
            for _ in range(5):
                whole()
            w0, w1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            w0.record()
            for _ in range(40):
                whole()
            w1.record()
            torch.cuda.synchronize()
            whole_calls[name] = round(w0.elapsed_time(w1) * 1e3 / 40, 1)
            if name != "q4k_4096x4096":
                # the matmul kernel alone (library event pair), as TOPS and as a fraction of the int8 MFMA peak
                def warm_timed():
                    for _ in range(20):   # (see the note at gemm_us above)
                        whole()
                    return qhip.timed_kernel_us(whole)
                k_us = sorted(warm_timed() for _ in range(5))[2]
                case = {"kernel_us": round(k_us, 2), "tops": round(2.0 * gm * wk * wn / (k_us * 1e-6) / 1e12, 1)}
                case["frac_of_int8_mfma_peak"] = round(case["tops"] / 5000.0, 4)
                # the same product with the activations quantized to Q8_1 (the reference's CUDA formulation): its cost and
                # its distance from the CPU formulation's result
                q81_ws = torch.empty(L.cq_workspace_bytes(wq.handle, gm, qhip.FLAG_ACT_Q8_1), dtype=torch.uint8, device=dev)
                y81 = torch.empty_like(wy)

                def whole81():
                    qhip.check(L.cq_qmatmul(wq.handle, C.c_void_p(wx.data_ptr()), gm, C.c_void_p(y81.data_ptr()),
                                            qhip.FLAG_ACT_Q8_1, C.c_void_p(q81_ws.data_ptr()), q81_ws.numel(),
                                            C.c_void_p(torch.cuda.current_stream().cuda_stream)))
                whole81()
                w0.record()
                for _ in range(3):
                    whole81()
                w1.record()
                torch.cuda.synchronize()
                case["q8_1_variant_us"] = round(w0.elapsed_time(w1) * 1e3 / 3, 1)
                case["q8_1_variant_rel_l2_vs_q8k"] = float(f"{float((y81 - wy).norm() / wy.norm()):.3e}")
                gemm_cases[name] = case
                del q81_ws, y81
            del wq, wx, wy, wws

    # ---- the same step with the model's neighbours of each matmul (reported beside the headline) ----
    # Per layer rms_norm -> q, k, v; o; rms_norm -> gate, up; silu(gate) * up -> down; final rms_norm
    # -> lm_head (quantized_llama.rs:453-511 without attention and residuals).  "separate": one more
    # launch per rms_norm (torch's kernel) and per silu * mul (cq_silu_mul); "fused": those steps inside
    # the matmul launches (cq_qmatmul_fused).  Same weights as the headline step, HIP graph replay.
    neighbours = None
    try:
        if args.no_extras or args.no_graph:   # both extras are graph replays
            raise RuntimeError("skipped by --no-extras / --no-graph")
        alpha = torch.ones(HIDDEN, device=dev, dtype=torch.float32)
        h_buf = torch.empty((1, FFN), device=dev, dtype=torch.float32)
        eps = 1e-5

        def fused_call(i, pre, x, aux, s):
            qhip.check(L.cq_qmatmul_fused(calls[i][0].handle, pre, C.c_void_p(x.data_ptr()), C.c_void_p(aux.data_ptr()),
                                          eps, 1, C.c_void_p(outputs[i].data_ptr()), 0, C.c_void_p(ws.data_ptr()),
                                          ws.numel(), s))

        def plain_call(i, x, s):
            qhip.check(L.cq_qmatmul(calls[i][0].handle, C.c_void_p(x.data_ptr()), 1, C.c_void_p(outputs[i].data_ptr()),
                                    0, C.c_void_p(ws.data_ptr()), ws.numel(), s))

        def multi_call(first, count, x, s):   # rms_norm -> `count` projections, one launch
            hs = (C.c_void_p * count)(*[calls[first + t][0].handle for t in range(count)])
            ys = (C.c_void_p * count)(*[outputs[first + t].data_ptr() for t in range(count)])
            qhip.check(L.cq_qmatmul_multi(hs, count, qhip.PRE_RMS_NORM, C.c_void_p(x.data_ptr()), C.c_void_p(alpha.data_ptr()),
                                          eps, 1, ys, 0, C.c_void_p(ws.data_ptr()), ws.numel(), s))

        def chain(fused):
            s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
            norm = lambda x: torch.nn.functional.rms_norm(x, (HIDDEN,), alpha, eps)
            for layer in range(args.layers):
                b = layer * len(LAYER_SHAPES)
                if fused == "shared":
                    multi_call(b, 3, inputs["x_attn"], s)
                    plain_call(b + 3, inputs["x_o"], s)
                    multi_call(b + 4, 2, outputs[b + 3], s)
                    fused_call(b + 6, qhip.PRE_SILU_MUL, outputs[b + 4], outputs[b + 5], s)
                elif fused:
                    for j in range(3):
                        fused_call(b + j, qhip.PRE_RMS_NORM, inputs["x_attn"], alpha, s)
                    plain_call(b + 3, inputs["x_o"], s)
                    for j in (4, 5):
                        fused_call(b + j, qhip.PRE_RMS_NORM, outputs[b + 3], alpha, s)
                    fused_call(b + 6, qhip.PRE_SILU_MUL, outputs[b + 4], outputs[b + 5], s)
                else:
                    xn = norm(inputs["x_attn"])
                    for j in range(3):
                        plain_call(b + j, xn, s)
                    plain_call(b + 3, inputs["x_o"], s)
                    xn = norm(outputs[b + 3])
                    for j in (4, 5):
                        plain_call(b + j, xn, s)
                    qhip.check(L.cq_silu_mul(0, C.c_void_p(outputs[b + 4].data_ptr()), C.c_void_p(outputs[b + 5].data_ptr()),
                                             C.c_void_p(h_buf.data_ptr()), FFN, s))
                    plain_call(b + 6, h_buf, s)
            last = len(calls) - 1
            if fused:
                fused_call(last, qhip.PRE_RMS_NORM, inputs["x_head"], alpha, s)
            else:
                plain_call(last, norm(inputs["x_head"]), s)

        times = {}
        with torch.cuda.stream(side):
            for name, fused in (("separate", False), ("fused", True), ("shared", "shared")):
                chain(fused)
                torch.cuda.synchronize()
                gn_ = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gn_, stream=side):
                    chain(fused)
                for _ in range(3):
                    gn_.replay()
                torch.cuda.synchronize()
                n0, n1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                n0.record()
                for _ in range(args.steps):
                    gn_.replay()
                n1.record()
                torch.cuda.synchronize()
                times[name] = n0.elapsed_time(n1) / args.steps
        neighbours = {
            "workload": "the headline step plus per layer 2 x rms_norm and silu * mul, and the final rms_norm",
            "matmuls_only_ms": round(ms_by_launch.get("hip graph replay", ms_per_step), 4),   # graph replay like the others here
            "separate_launches_ms": round(times["separate"], 4),
            "fused_ms": round(times["fused"], 4),
            "fused_shared_input_ms": round(times["shared"], 4),   # q, k, v and gate, up each in one cq_qmatmul_multi launch
        }
    except Exception as e:  # reported beside the headline only: never fails the bench line
        if not (args.no_extras or args.no_graph):
            print(f"bench.py: neighbour chain not measured ({e})", file=sys.stderr)

    # ---- the same bytes in fewer, larger calls (reported beside the headline) -----------------------
    # A model that keeps q|k|v and gate|up as one quantized tensor each (rows of GGML blocks simply
    # concatenated: [12288 x 4096] and [22016 x 4096]) issues 129 QMatMul calls per step instead of 225
    # over the same number of weight bytes.  Fresh random weights of those shapes, same kernels.
    merged = None
    try:
        if args.no_extras or args.no_graph:   # both extras are graph replays
            raise RuntimeError("skipped by --no-extras / --no-graph")
        m_calls = []
        for layer in range(args.layers):
            for idx, (dt, n, k, xin) in enumerate((("q4k", 3 * HIDDEN, HIDDEN, "x_attn"), ("q4k", HIDDEN, HIDDEN, "x_o"),
                                                   ("q4k", 2 * FFN, HIDDEN, "x_ffn"), ("q6k", HIDDEN, FFN, "x_down"))):
                gen.manual_seed(500_000 + 10 * layer + idx)
                w = torch.randn((n, k), generator=gen, device=dev, dtype=torch.float32) * 0.02
                m_calls.append((qhip.QWeight.zeros(DT[dt], n, k).quantize_(w), xin, dt, n, k))
                del w
        m_calls.append(calls[-1])
        m_out = [torch.empty((1, n), device=dev, dtype=torch.float32) for (_, _, _, n, _) in m_calls]
        m_bytes = sum(ggml_bytes(dt, n, k) for (_, _, dt, n, k) in m_calls)

        def m_step():
            s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
            for (qw, xin, _, _, _), out in zip(m_calls, m_out):
                qhip.check(L.cq_qmatmul(qw.handle, C.c_void_p(inputs[xin].data_ptr()), 1, C.c_void_p(out.data_ptr()), 0,
                                        C.c_void_p(ws.data_ptr()), ws.numel(), s))

        with torch.cuda.stream(side):
            m_step()
            torch.cuda.synchronize()
            gm_ = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gm_, stream=side):
                m_step()
            for _ in range(3):
                gm_.replay()
            torch.cuda.synchronize()
            m0, m1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            m0.record()
            for _ in range(args.steps):
                gm_.replay()
            m1.record()
            torch.cuda.synchronize()
            m_ms = m0.elapsed_time(m1) / args.steps
        merged = {
            "workload": "q|k|v and gate|up stored as one tensor each: %d calls per step" % len(m_calls),
            "weight_bytes_per_step": m_bytes,
            "ms_per_step": round(m_ms, 4),
            "GBs": round(m_bytes / (m_ms * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(m_bytes / (m_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        }
        del m_calls, m_out, gm_
    except Exception as e:  # reported beside the headline only: never fails the bench line
        if not (args.no_extras or args.no_graph):
            print(f"bench.py: merged-projection step not measured ({e})", file=sys.stderr)

    # ---- configs[2]-style small batches on the headline's weights (reported beside the headline) --------
    # Whole calls (quantizer launch included where there is one), graph replay over the 32 layers' attn_q
    # [4096 x 4096] and ffn_gate [11008 x 4096] weights, so every call streams its weights from HBM.
    small_batch = None
    try:
        if args.no_extras or args.no_graph or args.layers < 8:
            raise RuntimeError("skipped by --no-extras / --no-graph / --layers")
        small_batch = {}
        for label, idx in (("q4k_4096x4096", 0), ("q4k_11008x4096", 4)):
            picks = [calls[layer * len(LAYER_SHAPES) + idx] for layer in range(args.layers)]
            n_out = picks[0][3]
            for mb in (2, 4, 8, 16):
                xb = torch.randn((mb, HIDDEN), generator=gen, device=dev, dtype=torch.float32)
                yb = torch.empty((mb, n_out), device=dev, dtype=torch.float32)
                wsb = torch.empty(max(picks[0][0].workspace_bytes(mb), 256), dtype=torch.uint8, device=dev)

                def b_step():
                    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
                    for (qw, *_r) in picks:
                        qhip.check(L.cq_qmatmul(qw.handle, C.c_void_p(xb.data_ptr()), mb, C.c_void_p(yb.data_ptr()), 0,
                                                C.c_void_p(wsb.data_ptr()), wsb.numel(), s))

                with torch.cuda.stream(side):
                    b_step()
                    torch.cuda.synchronize()
                    gb_ = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(gb_, stream=side):
                        b_step()
                    gb_.replay()
                    torch.cuda.synchronize()
                    b0, b1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    b0.record()
                    for _ in range(10):
                        gb_.replay()
                    b1.record()
                    torch.cuda.synchronize()
                small_batch["%s_m%d_us" % (label, mb)] = round(b0.elapsed_time(b1) * 1e3 / (10 * len(picks)), 2)
                del gb_, xb, yb, wsb
    except Exception as e:  # reported beside the headline only: never fails the bench line
        small_batch = None
        if not (args.no_extras or args.no_graph):
            print(f"bench.py: small batches not measured ({e})", file=sys.stderr)

    # ---- the other configurations' shapes, whole calls in a graph replay (reported beside the headline) ------
    # configs[0]: one Q4_0 [4096 x 4096] matvec (Q8_0 activations); configs[2]'s Q8_0 half: 2-16 rows on
    # Q8_0 weights of both decode shapes; configs[4]: the Mixtral-shaped expert FFN (8 experts, 64 tokens,
    # top-2: two grouped launches on the routed rows, silu * mul on the way into the grouped w2 launch,
    # weighted scatter-add).  Sixteen distinct weights per shape take turns so that each call streams from HBM.
    other = None
    try:
        if args.no_extras or args.no_graph or args.layers < 8:
            raise RuntimeError("skipped by --no-extras / --no-graph / --layers")
        other = {}

        def replay_us(fn, calls_per_replay, reps=10):
            with torch.cuda.stream(side):
                fn()
                torch.cuda.synchronize()
                g_ = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g_, stream=side):
                    fn()
                g_.replay()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(reps):
                    g_.replay()
                e1.record()
                torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / (reps * calls_per_replay)
            del g_
            return us

        def make_weights(dt, n, k, count, seed0):
            out = []
            for t in range(count):
                gen.manual_seed(seed0 + t)
                w_ = torch.randn((n, k), generator=gen, device=dev, dtype=torch.float32) * 0.02
                out.append(qhip.QWeight.zeros(dt, n, k).quantize_(w_))
                del w_
            return out

        def calls_on(weights, xb, yb, wsb, mb):
            def fn():
                s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
                for qw in weights:
                    qhip.check(L.cq_qmatmul(qw.handle, C.c_void_p(xb.data_ptr()), mb, C.c_void_p(yb.data_ptr()), 0,
                                            C.c_void_p(wsb.data_ptr()), wsb.numel(), s))
            return fn

        for label, dt, dtname, n_out in (("q4_0_4096x4096", qhip.Q4_0, "q4_0", HIDDEN), ("q8_0_4096x4096", qhip.Q8_0, "q8_0", HIDDEN),
                                         ("q8_0_11008x4096", qhip.Q8_0, "q8_0", FFN)):
            weights = make_weights(dt, n_out, HIDDEN, 16, 50_000 + n_out + dt)
            for mb in ((1,) if dt == qhip.Q4_0 else (1, 2, 4, 8, 16)):
                xb = torch.randn((mb, HIDDEN), generator=gen, device=dev, dtype=torch.float32)
                yb = torch.empty((mb, n_out), device=dev, dtype=torch.float32)
                wsb = torch.empty(max(weights[0].workspace_bytes(mb), 256), dtype=torch.uint8, device=dev)
                us = replay_us(calls_on(weights, xb, yb, wsb, mb), len(weights))
                other["%s_m%d_us" % (label, mb)] = round(us, 2)
                if mb == 1:
                    other["%s_m1_GBs" % label] = round(ggml_bytes(dtname, n_out, HIDDEN) / us / 1e3, 1)
                del xb, yb, wsb
            del weights

        n_e, tokens, ffn_moe = 8, 64, 14336
        w1 = make_weights(qhip.Q4K, ffn_moe, HIDDEN, n_e, 60_000)
        w3 = make_weights(qhip.Q4K, ffn_moe, HIDDEN, n_e, 60_100)
        w2 = make_weights(qhip.Q6K, HIDDEN, ffn_moe, n_e, 60_200)
        gen.manual_seed(60_300)
        xs = torch.randn((tokens, HIDDEN), generator=gen, device=dev, dtype=torch.float32)
        probs = torch.softmax(torch.randn((tokens, n_e), generator=gen, device=dev, dtype=torch.float32), dim=-1).cpu().numpy()
        top = np.argsort(-probs, axis=1, kind="stable")[:, :2]
        topw = np.take_along_axis(probs, top, axis=1)
        topw = topw / topw.sum(axis=1, keepdims=True)
        rid, wts, offs = [], [], [0]
        for e in range(n_e):
            tok, slot = np.nonzero(top == e)
            rid.extend(tok.tolist())
            wts.extend(topw[tok, slot].tolist())
            offs.append(len(rid))
        rid_d = torch.tensor(rid, dtype=torch.int32, device=dev)
        wts_d = torch.tensor(wts, dtype=torch.float32, device=dev)
        offs = np.asarray(offs, dtype=np.int32)
        moe_ws = qhip.Workspace()

        def moe_ffn():
            h1 = qhip.qmatmul_grouped(w1, xs, rid_d, offs, workspace=moe_ws)
            h3 = qhip.qmatmul_grouped(w3, xs, rid_d, offs, flags=qhip.FLAG_REUSE_ACT, workspace=moe_ws)   # the rows quantized for w1
            y_ = qhip.qmatmul_grouped(w2, h1, None, offs, workspace=moe_ws, pre=qhip.PRE_SILU_MUL, aux=h3)
            return qhip.moe_scatter_add(y_, rid_d, wts_d, tokens)

        moe_us = replay_us(moe_ffn, 1, reps=20)
        moe_bytes = n_e * (2 * ggml_bytes("q4k", ffn_moe, HIDDEN) + ggml_bytes("q6k", HIDDEN, ffn_moe))
        other["moe_ffn"] = {
            "workload": "configs[4]: 8 experts (w1, w3 [14336x4096] Q4_K, w2 [4096x14336] Q6_K), 64 tokens, top-2: "
                        "3 grouped launches + quantizers + scatter-add, cold weights not forced (914 MB > caches)",
            "us_per_ffn": round(moe_us, 1),
            "weight_bytes": moe_bytes,
            "GBs": round(moe_bytes / moe_us / 1e3, 1),
            "frac_of_hbm_peak": round(moe_bytes / moe_us / 1e3 / 8000.0, 4),
            "rows_per_expert": [int(offs[e + 1] - offs[e]) for e in range(n_e)],
        }
        del w1, w2, w3
    except Exception as e:  # reported beside the headline only: never fails the bench line
        other = None
        if not (args.no_extras or args.no_graph):
            print(f"bench.py: other configurations not measured ({e})", file=sys.stderr)

    # ---- the headline's own weights, q/k/v and gate/up each through one cq_qmatmul_multi call ---------
    # (same weights, inputs and bytes as the headline step; 129 launches instead of 225)
    shared = None
    try:
        if args.no_extras or args.no_graph:
            raise RuntimeError("skipped by --no-extras / --no-graph")
        vp = C.c_void_p
        groups = []   # (handles array, outputs array, count, input) per launch
        i = 0
        while i < len(calls):
            j = i + 1
            while j < len(calls) and j - i < 3 and calls[j][1] == calls[i][1] and calls[j][2] == calls[i][2] \
                    and calls[j][4] == calls[i][4] and (j - 1) // len(LAYER_SHAPES) == i // len(LAYER_SHAPES):
                j += 1
            groups.append(((vp * (j - i))(*[calls[t][0].handle for t in range(i, j)]),
                           (vp * (j - i))(*[outputs[t].data_ptr() for t in range(i, j)]), j - i, calls[i][1]))
            i = j

        def s_step():
            s = vp(torch.cuda.current_stream().cuda_stream)
            for handles, ys, count, xin in groups:
                qhip.check(L.cq_qmatmul_multi(handles, count, qhip.PRE_NONE, vp(inputs[xin].data_ptr()), None, 0.0, 1, ys, 0,
                                              vp(ws.data_ptr()), ws.numel(), s))

        with torch.cuda.stream(side):
            s_step()
            torch.cuda.synchronize()
            gs_ = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gs_, stream=side):
                s_step()
            for _ in range(3):
                gs_.replay()
            torch.cuda.synchronize()
            s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s0.record()
            for _ in range(args.steps):
                gs_.replay()
            s1.record()
            torch.cuda.synchronize()
            s_ms = s0.elapsed_time(s1) / args.steps
        shared = {
            "workload": "the headline step with q, k, v and gate, up each as one cq_qmatmul_multi call: %d launches" % len(groups),
            "ms_per_step": round(s_ms, 4),
            "GBs": round(bytes_per_step / (s_ms * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(bytes_per_step / (s_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        }
        del gs_
    except Exception as e:  # reported beside the headline only: never fails the bench line
        if not (args.no_extras or args.no_graph):
            print(f"bench.py: shared-input step not measured ({e})", file=sys.stderr)

    value = bytes_per_step / (ms_per_step * 1e-3) / 1e9
    result = {
        "metric": "Q4_K matvec HBM GB/s (% of peak); Q4_K M=512 GEMM TOPS (% int8 MFMA peak)",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {
            "workload": "configs[1]: Llama-2-7B decode QMatMul stack, batch 1, %d layers + lm_head, %d calls/step, "
                        "Q4_K/Q6_K weights x Q8_K activations" % (args.layers, len(calls)),
            "weight_bytes_per_step": bytes_per_step,
            "launch": launch_mode,
            "ms_per_step_by_launch": {k: round(v, 4) for k, v in ms_by_launch.items()},
            "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
            "setup_s": round(t_setup, 1),
        },
        "roofline": {
            "kernel": "fused_kernel<Q4K> (decode matvec, all Q4_K launches of the step)",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": Q4K_DECODE_TRAFFIC_BYTES_PER_LAUNCH if args.layers == LAYERS else None,
            "traffic_source": "constant from a rocprofv3 --pmc run of this script (profiles/decode_stack_q4k_matvec_hbm_traffic.md), "
                              "not measured in this run",
            "avg_launch_us": round(avg_dur * 1e6, 3),
            "alg_bytes_per_launch": int(avg_bytes),
            "launches_timed": len(durs),
            "timing": "graph replay of the 192 Q4_K launches between two HIP events, time / launches"
                      if graph is not None else "per-kernel HIP event pairs, eager launches",
            "per_kernel_events_avg_launch_us": round(eager_avg_dur * 1e6, 3),
            "per_kernel_events_gate_up_11008x4096_GBs": round(big_gbs, 1) if big_gbs else None,
            "per_kernel_events_attn_4096x4096_GBs": round(small_gbs, 1) if small_gbs else None,
        },
        "prefill_gemm": {
            "workload": "configs[3]: Q4_K [14336x4096] x Q8_K activations, M=512 (Mistral-7B FFN up/gate), activations "
                        "N(0,1) with 1 % outliers at +-8 sigma",
            "kernel": "gemm_kernel<Q4K> (int8 MFMA, quantizer launch not included)",
            "bound": "int8 mfma",
            "achieved": round(gemm_tops, 1),
            "peak": 5000.0,
            "unit": "TOP/s",
            "frac": round(gemm_tops / 5000.0, 4),
            "ops_per_launch": 2 * gm * gk * gn,
            "avg_launch_us": round(gemm_avg_us, 2),
            "timing": "the library's HIP event pair around the kernel, mean of 10 launches",
            "clock": mfma_clock_probe(torch) if not args.no_extras else None,
            "tops": round(gemm_tops, 1),
            "peak_tops": 5000.0,
            "frac_of_int8_mfma_peak": round(gemm_tops / 5000.0, 4),
            "whole_call_us_m512": whole_calls or None,
            "configs3_cases": gemm_cases or None,
        },
    }

    if neighbours is not None:
        result["fused_neighbours"] = neighbours
    if merged is not None:
        result["merged_projections"] = merged
    if shared is not None:
        result["shared_input_launches"] = shared
    if small_batch is not None:
        result["small_batch"] = small_batch
    if other is not None:
        result["other_configs"] = other

    # ---- CPU baseline: restated candle CPU QMatMul (AVX2 + threads) on a bounded sample ----
    if not args.no_cpu:
        from oracle import cpu_oracle as orc
        threads = orc.baseline_lib().cpub_num_threads()
        sample_layers = min(8, args.layers)  # ~1 GB of weights: larger than the host's last-level cache
        host = []
        for i in range(sample_layers * len(LAYER_SHAPES)):
            qw, xin, dt, n, k = calls[i]
            host.append((DT[dt], qw.to_ggml(), inputs[xin].cpu().numpy(), n, np.empty((1, n), np.float32)))
        sample_bytes = sum(ggml_bytes(calls[i][2], calls[i][3], calls[i][4]) for i in range(len(host)))
        for (dt, blocks, x, n, out) in host:  # warm-up pass (page in, spin up the thread pool)
            orc.baseline_matmul(dt, x, blocks, n, out)
        reps, t_cpu = 0, 0.0
        t_start = time.perf_counter()
        while t_cpu < 10.0 and reps < 2000:
            for (dt, blocks, x, n, out) in host:
                orc.baseline_matmul(dt, x, blocks, n, out)
            reps += 1
            t_cpu = time.perf_counter() - t_start
        result["cpu_baseline"] = {
            "value": round(sample_bytes * reps / t_cpu / 1e9, 3),
            "unit": "GB/s",
            "cores": threads,
            "kind": "port",
            "sample": "%d of %d layers (%d QMatMul calls, %d weight bytes per pass), %d passes in %.1f s; "
                      "AVX2 restatement of k_quants::matmul + avx.rs, same weights and inputs as the GPU run"
                      % (sample_layers, args.layers, len(host), sample_bytes, reps, t_cpu),
        }
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
