"""Builds libcandle_qhip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libcandle_qhip.so")
SOURCES = ["api.hip", "repack.hip", "quantize_act.hip", "quantize_weight.hip", "dequantize.hip", "matvec.hip",
           "gemm.hip", "gemm_blk32.hip", "skinny.hip", "moe.hip", "min_term.hip", "q8k_weight.hip", "no_alloc.hip"]
# -ffp-contract=off: quantizers must perform single IEEE operations in the reference's order.
# -packed-fp32-ops off: packed FP32 instructions are not to be generated on this hardware pool.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function"]
# gemm.hip: MFMA results are consumed by VALU code every block; keep the accumulators in ordinary
# VGPRs rather than AccVGPRs, which VALU instructions cannot read.
EXTRA_FLAGS = {"gemm.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"], "gemm_blk32.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
               "skinny.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _compile(src: str) -> str:
    obj = os.path.join(LIB_DIR, src.replace(".hip", ".o"))
    cmd = ["hipcc", *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


# Measurement aid (bench.py --envelope): empty and streaming-read reference kernels, a library of its own.
PROBE_SOURCE = "probe.hip"
PROBE_LIB_PATH = os.path.join(LIB_DIR, "libcandle_qhip_probe.so")


def build(verbose: bool = True) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES) + 1)) as ex:
        objs = list(ex.map(_compile, SOURCES + [PROBE_SOURCE]))
    probe_obj = objs.pop()
    subprocess.check_call(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs])
    subprocess.check_call(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", PROBE_LIB_PATH, probe_obj])
    if verbose:
        print("built", LIB_PATH)
        print("built", PROBE_LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build()
