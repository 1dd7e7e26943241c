#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

Workload (BASELINE.json configs[1]): the Llama-2-7B-shaped decode QMatMul stack at batch 1 -
per layer q/k/v/o [4096x4096] Q4_K, gate/up [11008x4096] Q4_K, down [4096x11008] Q6_K, 32 layers,
plus an lm_head [32000x4096] Q6_K; activations f32 N(0,1) quantized to Q8_K.  A "step" is one
pass over all 225 QMatMul calls (4 122 255 360 bytes of GGML weights, all distinct, so every call
streams from HBM and not from the 256 MB Infinity Cache).  Weights are random N(0,0.02) drawn and
quantized on the device (bit-identical to the CPU quantizer, see tests).

Prints ONE JSON line.  `value` = GGML weight bytes per step / time per step (inputs resident in
HBM).  `roofline` covers the dominant kernel, the Q4_K matvec: algorithmic bytes per launch
divided by its average launch duration, measured here with HIP events around single launches.
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
    return n * k // 256 * {"q4k": 144, "q6k": 210}[dtype]


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=LAYERS, help="(debug) fewer layers; the result is then not a bench line")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
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
        run = graph.replay if graph is not None else step
        for _ in range(args.warmup):
            run()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            run()
        e1.record()
        torch.cuda.synchronize()
        ms_per_step = e0.elapsed_time(e1) / args.steps

        # ---- dominant kernel: Q4_K matvec, one launch at a time between two events ---------
        q4k_calls = [i for i, c in enumerate(calls) if c[2] == "q4k"]
        durs, alg_bytes = [], []
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in q4k_calls]
        for rep in range(3):
            last_in = None
            for (a, b), i in zip(evs, q4k_calls):
                xin = calls[i][1]
                if xin != last_in:  # quantize this input into the workspace outside the event pair
                    run_call(i, 0)
                    last_in = xin
                a.record()
                run_call(i, qhip.FLAG_REUSE_ACT)
                b.record()
            torch.cuda.synchronize()
            if rep == 0:
                continue  # first pass warms the instrumented path
            for (a, b), i in zip(evs, q4k_calls):
                _, _, dt, n, k = calls[i]
                durs.append(a.elapsed_time(b) * 1e-3)
                # weights + quantized activations read (Q8K: k + k/256*(4+32) bytes) + f32 outputs written
                alg_bytes.append(ggml_bytes(dt, n, k) + k + k // 256 * 36 + 4 * n)
    avg_dur = sum(durs) / len(durs)
    avg_bytes = sum(alg_bytes) / len(alg_bytes)
    achieved = avg_bytes / avg_dur / 1e9
    # headline shape alone (gate/up, 11008x4096)
    big = [(d, b) for d, b in zip(durs, alg_bytes) if b > 20_000_000]
    big_gbs = (sum(b for _, b in big) / sum(d for d, _ in big) / 1e9) if big else None

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
            "launch": "hip graph replay" if graph is not None else "eager",
            "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
            "setup_s": round(t_setup, 1),
        },
        "roofline": {
            "kernel": "matvec_kernel<Q4K, 1>",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": None,
            "avg_launch_us": round(avg_dur * 1e6, 3),
            "alg_bytes_per_launch": int(avg_bytes),
            "launches_timed": len(durs),
            "gate_up_11008x4096_GBs": round(big_gbs, 1) if big_gbs else None,
        },
    }

    # ---- CPU baseline: restated candle CPU QMatMul (AVX2 + threads) on a bounded sample ----
    if not args.no_cpu:
        from oracle import cpu_oracle as orc
        threads = orc.baseline_lib().cpub_num_threads()
        sample_layers = min(2, args.layers)
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
