"""ctypes front-end of the CPU oracle (test infrastructure only).

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the product (``candle_amd``) never does.
Everything here is a thin typed wrapper over ``libcandle_q_oracle.so``, the C
restatement of candle-core/src/quantized/k_quants.rs.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcandle_q_oracle.so")

# GgmlDType ids (candle-core/src/quantized/mod.rs:173-190)
Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1, Q2K, Q3K, Q4K, Q5K, Q6K, Q8K = 2, 3, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15
BLOCK_SIZE = {Q4_0: 32, Q4_1: 32, Q5_0: 32, Q5_1: 32, Q8_0: 32, Q8_1: 32, Q2K: 256, Q3K: 256, Q4K: 256, Q5K: 256, Q6K: 256, Q8K: 256}
TYPE_SIZE = {Q4_0: 18, Q4_1: 20, Q5_0: 22, Q5_1: 24, Q8_0: 34, Q8_1: 36, Q2K: 84, Q3K: 110, Q4K: 144, Q5K: 176, Q6K: 210, Q8K: 292}
# the reference's Q4_1 vectors also pin the `s` field of Q8_1 blocks
VEC_DOT_TYPE = {Q4_0: Q8_0, Q4_1: Q8_1, Q5_0: Q8_0, Q5_1: Q8_1, Q8_0: Q8_0, Q2K: Q8K, Q3K: Q8K, Q4K: Q8K, Q5K: Q8K, Q6K: Q8K, Q8K: Q8K}
NAMES = {Q4_0: "q4_0", Q4_1: "q4_1", Q5_0: "q5_0", Q5_1: "q5_1", Q8_0: "q8_0", Q8_1: "q8_1", Q2K: "q2k", Q3K: "q3k", Q4K: "q4k", Q5K: "q5k", Q6K: "q6k", Q8K: "q8k"}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc if the shared object is missing (or forced)."""
    src = os.path.join(_HERE, "candle_q_oracle.c")
    stale = (not os.path.exists(_LIB_PATH)) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src)
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "libcandle_q_oracle.so"] + (["-B"] if force else []))
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        f32p, vp, i64, i32p = C.POINTER(C.c_float), C.c_void_p, C.c_int64, C.POINTER(C.c_int32)
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_quantize.argtypes = [C.c_int, f32p, vp, i64]
        L.orc_dequantize.argtypes = [C.c_int, vp, f32p, i64]
        L.orc_vec_dot.argtypes = [C.c_int, i64, vp, vp, f32p]
        L.orc_matmul.argtypes = [C.c_int, i64, i64, i64, f32p, vp, f32p]
        L.orc_matmul_q8_1.argtypes = [C.c_int, i64, i64, i64, f32p, vp, f32p]
        L.orc_block_int_dots.argtypes = [C.c_int, i64, i64, i64, vp, vp, i32p, i32p]
        L.orc_softmax_last_dim.argtypes = [f32p, f32p, i64, i64]
        L.orc_softmax_last_dim.restype = None
        L.orc_moe_route.argtypes = [f32p, i64, C.c_int, C.c_int, i32p, i32p, f32p]
        L.orc_moe_ffn.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(vp), C.POINTER(vp), C.POINTER(vp),
                                  i64, i64, f32p, i64, i32p, i32p, f32p, f32p]
        L.orc_rms_norm.argtypes = [f32p, f32p, C.c_float, i64, i64, f32p]
        L.orc_rms_norm.restype = None
        L.orc_silu_mul.argtypes = [f32p, f32p, i64, f32p]
        L.orc_silu_mul.restype = None
        _lib = L
    return _lib


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(C.POINTER(C.c_float))


def _check(rc, what):
    if rc != 0:
        raise ValueError(f"oracle {what} failed with code {rc}")


def f16_to_f32(h: int) -> float:
    return float(lib().orc_f16_to_f32(int(h)))


def f32_to_f16(f: float) -> int:
    return int(lib().orc_f32_to_f16(float(f)))


def quantize(dtype: int, x) -> np.ndarray:
    """T::from_float: f32 array (any shape, last dim % block == 0) -> GGML bytes (uint8)."""
    x, xp = _f32(x)
    k = x.size
    if k % BLOCK_SIZE[dtype] != 0:
        raise ValueError(f"{k} is not divisible by {BLOCK_SIZE[dtype]}")
    out = np.zeros(k // BLOCK_SIZE[dtype] * TYPE_SIZE[dtype], dtype=np.uint8)
    _check(lib().orc_quantize(dtype, xp, out.ctypes.data, k), "quantize")
    return out


def dequantize(dtype: int, blocks: np.ndarray) -> np.ndarray:
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    nb = blocks.size // TYPE_SIZE[dtype]
    out = np.empty(nb * BLOCK_SIZE[dtype], dtype=np.float32)
    _check(lib().orc_dequantize(dtype, blocks.ctypes.data, out.ctypes.data_as(C.POINTER(C.c_float)), out.size),
           "dequantize")
    return out


def vec_dot(dtype: int, n: int, xs: np.ndarray, ys: np.ndarray) -> float:
    out = C.c_float(0)
    xs = np.ascontiguousarray(xs, dtype=np.uint8)
    ys = np.ascontiguousarray(ys, dtype=np.uint8)
    _check(lib().orc_vec_dot(dtype, n, xs.ctypes.data, ys.ctypes.data, C.byref(out)), "vec_dot")
    return float(np.float32(out.value))


def matmul(dtype: int, lhs, rhs_blocks: np.ndarray, n: int) -> np.ndarray:
    """k_quants::matmul((m,k,n), lhs, rhs_t, dst): lhs [m,k] f32, rhs GGML bytes of [n,k] -> [m,n]."""
    lhs, lp = _f32(lhs)
    m, k = lhs.shape
    rhs_blocks = np.ascontiguousarray(rhs_blocks, dtype=np.uint8)
    assert rhs_blocks.size == n * k // BLOCK_SIZE[dtype] * TYPE_SIZE[dtype], "rhs byte size mismatch"
    dst = np.empty((m, n), dtype=np.float32)
    _check(lib().orc_matmul(dtype, m, k, n, lp, rhs_blocks.ctypes.data, dst.ctypes.data_as(C.POINTER(C.c_float))),
           "matmul")
    return dst


def matmul_q8_1(dtype: int, lhs, rhs_blocks: np.ndarray, n: int) -> np.ndarray:
    lhs, lp = _f32(lhs)
    m, k = lhs.shape
    rhs_blocks = np.ascontiguousarray(rhs_blocks, dtype=np.uint8)
    dst = np.empty((m, n), dtype=np.float32)
    _check(lib().orc_matmul_q8_1(dtype, m, k, n, lp, rhs_blocks.ctypes.data,
                                 dst.ctypes.data_as(C.POINTER(C.c_float))), "matmul_q8_1")
    return dst


def block_int_dots(dtype: int, act_blocks: np.ndarray, m: int, rhs_blocks: np.ndarray, n: int, k: int):
    """Per-block integer dots I_b [m,n,kb] (and Mn_b for Q4K, else None)."""
    kb = k // BLOCK_SIZE[dtype]
    act_blocks = np.ascontiguousarray(act_blocks, dtype=np.uint8)
    rhs_blocks = np.ascontiguousarray(rhs_blocks, dtype=np.uint8)
    oi = np.zeros((m, n, kb), dtype=np.int32)
    om = np.zeros((m, n, kb), dtype=np.int32) if dtype in (Q2K, Q4K, Q5K) else None
    i32p = C.POINTER(C.c_int32)
    _check(lib().orc_block_int_dots(dtype, m, k, n, act_blocks.ctypes.data, rhs_blocks.ctypes.data,
                                    oi.ctypes.data_as(i32p),
                                    om.ctypes.data_as(i32p) if om is not None else None), "block_int_dots")
    return oi, om


def softmax_last_dim(x) -> np.ndarray:
    x, xp = _f32(x)
    out = np.empty_like(x)
    lib().orc_softmax_last_dim(xp, out.ctypes.data_as(C.POINTER(C.c_float)), x.size // x.shape[-1], x.shape[-1])
    return out


def rms_norm(x, alpha, eps: float) -> np.ndarray:
    """candle_nn::ops::rms_norm on f32 (candle-nn/src/ops.rs:482-495) over the last dimension."""
    x, xp = _f32(x)
    alpha, ap = _f32(alpha)
    assert alpha.ndim == 1 and alpha.shape[0] == x.shape[-1]
    out = np.empty_like(x)
    lib().orc_rms_norm(xp, ap, eps, x.size // x.shape[-1], x.shape[-1], out.ctypes.data_as(C.POINTER(C.c_float)))
    return out


def silu_mul(a, b) -> np.ndarray:
    """silu(a) * b as in Mlp::forward (quantized_llama.rs:60-62, op.rs:607-609)."""
    a, ap = _f32(a)
    b, bp = _f32(b)
    assert a.shape == b.shape
    out = np.empty_like(a)
    lib().orc_silu_mul(ap, bp, a.size, out.ctypes.data_as(C.POINTER(C.c_float)))
    return out


def moe_route(routing_weights, top_k: int):
    rw, rp = _f32(routing_weights)
    t, e = rw.shape
    offsets = np.zeros(e + 1, dtype=np.int32)
    row_ids = np.zeros(t * top_k, dtype=np.int32)
    weights = np.zeros(t * top_k, dtype=np.float32)
    i32p = C.POINTER(C.c_int32)
    _check(lib().orc_moe_route(rp, t, e, top_k, offsets.ctypes.data_as(i32p), row_ids.ctypes.data_as(i32p),
                               weights.ctypes.data_as(C.POINTER(C.c_float))), "moe_route")
    return offsets, row_ids, weights


def moe_ffn(dtype13: int, dtype2: int, w1, w2, w3, hidden: int, ffn: int, xs, offsets, row_ids, weights):
    """Sequential per-expert MoE FFN (quantized_llama.rs:116-135); w1/w2/w3 lists of GGML byte arrays."""
    xs, xp = _f32(xs)
    tokens = xs.shape[0]
    n_e = len(w1)
    keep = [np.ascontiguousarray(a, dtype=np.uint8) for a in list(w1) + list(w2) + list(w3)]
    arr = lambda lst: (C.c_void_p * n_e)(*[a.ctypes.data for a in lst])
    a1, a2, a3 = arr(keep[:n_e]), arr(keep[n_e:2 * n_e]), arr(keep[2 * n_e:])
    offsets = np.ascontiguousarray(offsets, dtype=np.int32)
    row_ids = np.ascontiguousarray(row_ids, dtype=np.int32)
    weights = np.ascontiguousarray(weights, dtype=np.float32)
    ys = np.empty((tokens, hidden), dtype=np.float32)
    i32p, f32p = C.POINTER(C.c_int32), C.POINTER(C.c_float)
    _check(lib().orc_moe_ffn(n_e, dtype13, dtype2, a1, a2, a3, hidden, ffn, xp, tokens,
                             offsets.ctypes.data_as(i32p), row_ids.ctypes.data_as(i32p),
                             weights.ctypes.data_as(f32p), ys.ctypes.data_as(f32p)), "moe_ffn")
    return ys


# ------------------------------------------------------------------ timed CPU baseline ----
_BASE_PATH = os.path.join(_HERE, "libcandle_q_cpu_baseline.so")
_base = None


def baseline_lib():
    """AVX2 + OpenMP restatement of the reference's CPU QMatMul (oracle/cpu_baseline.cpp)."""
    global _base
    if _base is None:
        src = os.path.join(_HERE, "cpu_baseline.cpp")
        if (not os.path.exists(_BASE_PATH)) or os.path.getmtime(_BASE_PATH) < os.path.getmtime(src):
            subprocess.check_call(["make", "-C", _HERE, "libcandle_q_cpu_baseline.so"])
        L = C.CDLL(_BASE_PATH)
        L.cpub_matmul.argtypes = [C.c_int, C.c_int64, C.c_int64, C.c_int64, C.POINTER(C.c_float), C.c_void_p,
                                  C.POINTER(C.c_float)]
        L.cpub_num_threads.restype = C.c_int
        L.cpub_set_num_threads.argtypes = [C.c_int]
        L.cpub_set_num_threads.restype = None
        _base = L
    return _base


def baseline_matmul(dtype: int, lhs, rhs_blocks: np.ndarray, n: int, out=None) -> np.ndarray:
    lhs, lp = _f32(lhs)
    m, k = lhs.shape
    rhs_blocks = np.ascontiguousarray(rhs_blocks, dtype=np.uint8)
    dst = out if out is not None else np.empty((m, n), dtype=np.float32)
    _check(baseline_lib().cpub_matmul(dtype, m, k, n, lp, rhs_blocks.ctypes.data,
                                      dst.ctypes.data_as(C.POINTER(C.c_float))), "baseline matmul")
    return dst
