"""ctypes binding of libcandle_qhip.so (the C ABI in include/candle_qhip.h).

torch is used for device memory and streams only.  There is no CPU fallback: if the
shared library is missing or no GPU is visible, calls raise.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("CQ_LIB_PATH", os.path.join(_HERE, "lib", "libcandle_qhip.so"))

# GgmlDType ids (candle-core/src/quantized/mod.rs:173-190)
Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1, Q2K, Q3K, Q4K, Q5K, Q6K, Q8K = 2, 3, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15
FLAG_AUTO, FLAG_FORCE_MATVEC, FLAG_FORCE_GEMM, FLAG_ACT_Q8_1, FLAG_REUSE_ACT, FLAG_STAGED_ACT = 0, 1, 2, 4, 8, 16
FLAG_FORCE_SKINNY = 32
FLAG_DETERMINISTIC = 64   # tile kernels never split K: the same bits on every run
PRE_NONE, PRE_RMS_NORM, PRE_SILU_MUL = 0, 1, 2

EXPORTS = [
    "cq_device_count", "cq_last_error", "cq_version", "cq_block_size", "cq_type_size", "cq_vec_dot_type",
    "cq_weight_create", "cq_weight_zeros", "cq_weight_quantize", "cq_weight_dequantize",
    "cq_weight_dequantize_f16", "cq_weight_to_ggml", "cq_weight_size_in_bytes", "cq_weight_dtype",
    "cq_weight_device", "cq_weight_shape", "cq_weight_destroy", "cq_act_bytes", "cq_quantize_act",
    "cq_workspace_bytes", "cq_qmatmul", "cq_qmatmul_int_dots", "cq_qmatmul_int_dots_mfma", "cq_grouped_workspace_bytes",
    "cq_qmatmul_grouped", "cq_silu_mul", "cq_moe_scatter_add", "cq_timing_arm", "cq_timing_elapsed_us",
    "cq_selfcheck_round", "cq_quantize_act_fused", "cq_qmatmul_fused", "cq_qmatmul_grouped_fused", "cq_qmatmul_multi",
    "cq_weight_zeros_flat", "cq_weight_create_flat", "cq_weight_elem_count", "cq_weight_set_shape",
    "cq_workspace_bytes_shaped", "cq_qmatmul_shaped", "cq_qmatmul_static",
]


class QHipError(RuntimeError):
    pass


_lib = None


def load():
    """Load the shared library; raises if it has not been built (python -m candle_amd.build)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise QHipError(f"{LIB_PATH} is missing: build it with `python -m candle_amd.build` (hipcc, gfx950)")
    L = C.CDLL(LIB_PATH)
    vp, i64, sz, ci = C.c_void_p, C.c_int64, C.c_size_t, C.c_int
    L.cq_device_count.restype = ci
    L.cq_last_error.restype = C.c_char_p
    L.cq_version.restype = C.c_char_p
    L.cq_block_size.restype = i64; L.cq_block_size.argtypes = [ci]
    L.cq_type_size.restype = i64; L.cq_type_size.argtypes = [ci]
    L.cq_vec_dot_type.restype = ci; L.cq_vec_dot_type.argtypes = [ci]
    L.cq_weight_create.argtypes = [ci, ci, vp, sz, i64, i64, C.POINTER(vp)]
    L.cq_weight_zeros.argtypes = [ci, ci, i64, i64, C.POINTER(vp)]
    L.cq_weight_quantize.argtypes = [vp, vp, vp]
    L.cq_weight_dequantize.argtypes = [vp, vp, vp]
    L.cq_weight_dequantize_f16.argtypes = [vp, vp, vp]
    L.cq_weight_to_ggml.argtypes = [vp, vp, sz]
    L.cq_weight_size_in_bytes.restype = sz; L.cq_weight_size_in_bytes.argtypes = [vp]
    L.cq_weight_dtype.argtypes = [vp]
    L.cq_weight_device.argtypes = [vp]
    L.cq_weight_shape.argtypes = [vp, C.POINTER(i64), C.POINTER(i64)]
    L.cq_weight_destroy.restype = None; L.cq_weight_destroy.argtypes = [vp]
    L.cq_act_bytes.restype = sz; L.cq_act_bytes.argtypes = [ci, i64, i64]
    L.cq_quantize_act.argtypes = [ci, ci, vp, i64, i64, vp, vp]
    L.cq_workspace_bytes.restype = sz; L.cq_workspace_bytes.argtypes = [vp, i64, ci]
    L.cq_qmatmul.argtypes = [vp, vp, i64, vp, ci, vp, sz, vp]
    L.cq_qmatmul_int_dots.argtypes = [vp, vp, i64, vp, vp, vp, sz, vp]
    L.cq_qmatmul_int_dots_mfma.argtypes = [vp, vp, i64, C.c_int, vp, vp, vp, sz, vp]
    L.cq_grouped_workspace_bytes.restype = sz
    L.cq_grouped_workspace_bytes.argtypes = [C.POINTER(vp), ci, i64, ci]
    L.cq_qmatmul_grouped.argtypes = [C.POINTER(vp), ci, vp, vp, C.POINTER(C.c_int32), vp, ci, vp, sz, vp]
    L.cq_silu_mul.argtypes = [ci, vp, vp, vp, i64, vp]
    L.cq_moe_scatter_add.argtypes = [ci, vp, vp, vp, i64, i64, vp, i64, vp]
    L.cq_timing_arm.argtypes = []
    L.cq_timing_elapsed_us.argtypes = [C.POINTER(C.c_double)]
    L.cq_selfcheck_round.argtypes = [ci, C.POINTER(C.c_uint64)]
    L.cq_quantize_act_fused.argtypes = [ci, ci, ci, vp, vp, C.c_float, i64, i64, vp, vp]
    L.cq_qmatmul_fused.argtypes = [vp, ci, vp, vp, C.c_float, i64, vp, ci, vp, sz, vp]
    L.cq_qmatmul_grouped_fused.argtypes = [C.POINTER(vp), ci, ci, vp, vp, C.c_float, vp, C.POINTER(C.c_int32), vp, ci,
                                           vp, sz, vp]
    L.cq_qmatmul_multi.argtypes = [C.POINTER(vp), ci, ci, vp, vp, C.c_float, i64, C.POINTER(vp), ci, vp, sz, vp]
    L.cq_weight_zeros_flat.argtypes = [ci, ci, i64, C.POINTER(vp)]
    L.cq_weight_create_flat.argtypes = [ci, ci, vp, sz, C.POINTER(vp)]
    L.cq_weight_elem_count.restype = i64; L.cq_weight_elem_count.argtypes = [vp]
    L.cq_weight_set_shape.argtypes = [vp, i64, i64]
    L.cq_workspace_bytes_shaped.restype = sz; L.cq_workspace_bytes_shaped.argtypes = [vp, i64, i64, i64, ci]
    L.cq_qmatmul_shaped.argtypes = [vp, i64, i64, vp, i64, vp, ci, vp, sz, vp]
    L.cq_qmatmul_static.argtypes = [vp, vp, i64, vp, ci, vp]
    _lib = L
    return L


def check(rc: int):
    if rc != 0:
        raise QHipError(f"[{rc}] {load().cq_last_error().decode()}")


def _torch():
    import torch
    return torch


def _stream_ptr():
    torch = _torch()
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _require_f32_cuda(x, name="x"):
    torch = _torch()
    if not x.is_cuda:
        raise QHipError(f"{name} must be a device tensor")
    if x.dtype != torch.float32:
        raise QHipError(f"{name} must be f32, got {x.dtype}")
    if not x.is_contiguous():
        # <QTensor as CustomOp1>::cpu_fwd, mod.rs:474-476 / cuda.rs:511-514 (RequiresContiguous)
        raise QHipError(f"input tensor is not contiguous ({name})")


class Workspace:
    """A growing device scratch buffer (the reference allocates its quantized-activation buffer
    per call, cuda.rs:249-252); one per stream of use."""

    def __init__(self):
        self.buf = None

    def get(self, nbytes: int, device):
        torch = _torch()
        if self.buf is None or self.buf.numel() < nbytes or self.buf.device != device:
            self.buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        return self.buf


_default_ws = Workspace()


class QWeight:
    """Owner of a `cq_weight` (device storage of one quantized [n, k] matrix)."""

    def __init__(self, handle, dev: int):
        self._h = C.c_void_p(handle)
        self.dev = dev

    # -- constructors
    @classmethod
    def from_ggml(cls, dtype: int, blocks: np.ndarray, n: int, k: int, dev: int = 0) -> "QWeight":
        L = load()
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        h = C.c_void_p()
        check(L.cq_weight_create(dev, dtype, blocks.ctypes.data, blocks.size, n, k, C.byref(h)))
        return cls(h.value, dev)

    @classmethod
    def zeros(cls, dtype: int, n: int, k: int, dev: int = 0) -> "QWeight":
        L = load()
        h = C.c_void_p()
        check(L.cq_weight_zeros(dev, dtype, n, k, C.byref(h)))
        return cls(h.value, dev)

    @classmethod
    def zeros_flat(cls, dtype: int, elem_count: int, dev: int = 0) -> "QWeight":
        """QCudaStorage::zeros(device, el_count, dtype) (cuda.rs:368-381): storage without a shape."""
        h = C.c_void_p()
        check(load().cq_weight_zeros_flat(dev, dtype, elem_count, C.byref(h)))
        return cls(h.value, dev)

    @classmethod
    def from_ggml_flat(cls, dtype: int, blocks: np.ndarray, dev: int = 0) -> "QWeight":
        """load_quantized(device, data) (cuda.rs:591-612): blocks only, the shape comes with the call."""
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        h = C.c_void_p()
        check(load().cq_weight_create_flat(dev, dtype, blocks.ctypes.data, blocks.size, C.byref(h)))
        return cls(h.value, dev)

    def set_shape(self, n: int, k: int) -> "QWeight":
        check(load().cq_weight_set_shape(self._h, n, k))
        return self

    @property
    def elem_count(self) -> int:
        return load().cq_weight_elem_count(self._h)

    def __del__(self):
        try:
            if self._h is not None and self._h.value:
                load().cq_weight_destroy(self._h)
                self._h = None
        except Exception:
            pass

    # -- properties
    @property
    def handle(self):
        return self._h

    @property
    def dtype(self) -> int:
        return load().cq_weight_dtype(self._h)

    @property
    def shape(self):
        n, k = C.c_int64(), C.c_int64()
        check(load().cq_weight_shape(self._h, C.byref(n), C.byref(k)))
        return (n.value, k.value)

    @property
    def size_in_bytes(self) -> int:
        return load().cq_weight_size_in_bytes(self._h)

    # -- operations
    def quantize_(self, src):
        _require_f32_cuda(src, "src")
        n, k = self.shape
        if src.numel() != n * k:
            raise QHipError(f"size mismatch {src.numel()} vs {n * k}")
        check(load().cq_weight_quantize(self._h, C.c_void_p(src.data_ptr()), _stream_ptr()))
        return self

    def dequantize(self):
        torch = _torch()
        n, k = self.shape
        out = torch.empty((n, k), dtype=torch.float32, device=f"cuda:{self.dev}")
        check(load().cq_weight_dequantize(self._h, C.c_void_p(out.data_ptr()), _stream_ptr()))
        return out

    def dequantize_f16(self):
        torch = _torch()
        n, k = self.shape
        out = torch.empty((n, k), dtype=torch.float16, device=f"cuda:{self.dev}")
        check(load().cq_weight_dequantize_f16(self._h, C.c_void_p(out.data_ptr()), _stream_ptr()))
        return out

    def to_ggml(self) -> np.ndarray:
        _torch().cuda.synchronize()
        out = np.empty(self.size_in_bytes, dtype=np.uint8)
        check(load().cq_weight_to_ggml(self._h, out.ctypes.data, out.size))
        return out

    def workspace_bytes(self, m: int, flags: int = 0) -> int:
        return load().cq_workspace_bytes(self._h, m, flags)


def _check_pre(pre: int, x, aux):
    """Shape rules of the fused steps: alpha [k] for rms_norm, a second operand shaped like x for
    silu * mul (rms_norm's own check: candle-nn/src/ops.rs:641-650)."""
    if pre == PRE_NONE:
        return
    _require_f32_cuda(aux, "aux")
    if pre == PRE_RMS_NORM:
        if aux.dim() != 1 or aux.shape[0] != x.shape[-1]:
            raise QHipError(f"shape mismatch in rms-norm {tuple(x.shape)} {tuple(aux.shape)}")
    elif pre == PRE_SILU_MUL:
        if tuple(aux.shape) != tuple(x.shape):
            raise QHipError(f"shape mismatch in silu-mul {tuple(x.shape)} {tuple(aux.shape)}")
    else:
        raise QHipError(f"unknown fused step {pre}")


def quantize_act(act_dtype: int, x, pre: int = PRE_NONE, aux=None, eps: float = 0.0):
    """T::VecDotType::from_float over the rows of x [m, k] (after the fused step `pre`, if any):
    returns a uint8 device tensor holding the GGML blocks."""
    torch = _torch()
    L = load()
    _require_f32_cuda(x)
    _check_pre(pre, x, aux)
    m, k = x.shape
    nbytes = L.cq_act_bytes(act_dtype, m, k)
    if nbytes == 0 and m * k != 0:
        raise QHipError(f"{k} is not divisible by the block size of dtype {act_dtype}")
    out = torch.zeros(max(nbytes, 4), dtype=torch.uint8, device=x.device)
    if pre == PRE_NONE:
        check(L.cq_quantize_act(x.device.index or 0, act_dtype, C.c_void_p(x.data_ptr()), m, k,
                                C.c_void_p(out.data_ptr()), _stream_ptr()))
    else:
        check(L.cq_quantize_act_fused(x.device.index or 0, act_dtype, pre, C.c_void_p(x.data_ptr()),
                                      C.c_void_p(aux.data_ptr()), eps, m, k, C.c_void_p(out.data_ptr()),
                                      _stream_ptr()))
    return out[:nbytes]


def qmatmul(w: QWeight, x, flags: int = 0, out=None, workspace: Workspace | None = None, pre: int = PRE_NONE,
            aux=None, eps: float = 0.0):
    """QMatMul::forward for a quantized weight: x [..., k] f32 contiguous -> [..., n].  With `pre`
    the model step in front of the matmul (rms_norm with alpha = aux, or silu(x) * aux) is computed
    inside the same launches."""
    torch = _torch()
    L = load()
    _require_f32_cuda(x)
    _check_pre(pre, x, aux)
    n, k = w.shape
    if x.dim() < 2:
        raise QHipError(f"input tensor has only one dimension {tuple(x.shape)}")   # mod.rs:480-482
    if x.shape[-1] != k:
        raise QHipError(f"input tensor {tuple(x.shape)} incompatible with {(n, k)}")  # mod.rs:485-487
    m = x.numel() // k if k else 0
    out_shape = tuple(x.shape[:-1]) + (n,)
    if out is None:
        out = torch.empty(out_shape, dtype=torch.float32, device=x.device)
    need = L.cq_workspace_bytes(w.handle, m, flags)
    ws = (workspace or _default_ws).get(need, x.device)
    if pre == PRE_NONE:
        check(L.cq_qmatmul(w.handle, C.c_void_p(x.data_ptr()), m, C.c_void_p(out.data_ptr()), flags,
                           C.c_void_p(ws.data_ptr()), ws.numel(), _stream_ptr()))
    else:
        check(L.cq_qmatmul_fused(w.handle, pre, C.c_void_p(x.data_ptr()), C.c_void_p(aux.data_ptr()), eps, m,
                                 C.c_void_p(out.data_ptr()), flags, C.c_void_p(ws.data_ptr()), ws.numel(),
                                 _stream_ptr()))
    return out


def qmatmul_shaped(w: QWeight, shape, x, flags: int = 0, out=None, workspace: Workspace | None = None):
    """QCudaStorage::fwd(&self, self_shape, x, layout) (cuda.rs:478-499): the weight's [n, k] arrives with the
    call; the storage only knows its element count."""
    torch = _torch()
    L = load()
    _require_f32_cuda(x)
    n, k = (int(v) for v in shape)
    if x.dim() < 2:
        raise QHipError(f"input tensor has only one dimension {tuple(x.shape)}")
    if x.shape[-1] != k:
        raise QHipError(f"input tensor {tuple(x.shape)} incompatible with {(n, k)}")
    m = x.numel() // k if k else 0
    if out is None:
        out = torch.empty(tuple(x.shape[:-1]) + (n,), dtype=torch.float32, device=x.device)
    need = L.cq_workspace_bytes_shaped(w.handle, n, k, m, flags)
    ws = (workspace or _default_ws).get(need, x.device)
    check(L.cq_qmatmul_shaped(w.handle, n, k, C.c_void_p(x.data_ptr()), m, C.c_void_p(out.data_ptr()), flags,
                              C.c_void_p(ws.data_ptr()), ws.numel(), _stream_ptr()))
    return out


def qmatmul_multi(ws, x, flags: int = 0, workspace: Workspace | None = None, pre: int = PRE_NONE, aux=None,
                  eps: float = 0.0):
    """[x . W^T for W in ws]: several weights (same dtype and row length) on the same activations, one
    launch for one activation row, rows quantized once otherwise (cq_qmatmul_multi)."""
    torch = _torch()
    L = load()
    _require_f32_cuda(x)
    _check_pre(pre, x, aux)
    ws = list(ws)
    if not ws:
        raise QHipError("no weights")
    k = ws[0].shape[1]
    if x.dim() < 2:
        raise QHipError(f"input tensor has only one dimension {tuple(x.shape)}")
    if x.shape[-1] != k:
        raise QHipError(f"input tensor {tuple(x.shape)} incompatible with {ws[0].shape}")
    m = x.numel() // k if k else 0
    outs = [torch.empty(tuple(x.shape[:-1]) + (w.shape[0],), dtype=torch.float32, device=x.device) for w in ws]
    need = max(L.cq_workspace_bytes(w.handle, m, flags) for w in ws)
    wsp = (workspace or _default_ws).get(need, x.device)
    vp = C.c_void_p
    handles = (vp * len(ws))(*[w.handle for w in ws])
    ys = (vp * len(ws))(*[o.data_ptr() for o in outs])
    check(L.cq_qmatmul_multi(handles, len(ws), pre, vp(x.data_ptr()), vp(aux.data_ptr()) if aux is not None else None,
                             eps, m, ys, flags, vp(wsp.data_ptr()), wsp.numel(), _stream_ptr()))
    return outs


def qmatmul_int_dots(w: QWeight, x):
    torch = _torch()
    L = load()
    _require_f32_cuda(x)
    n, k = w.shape
    m = x.shape[0]
    kb = k // L.cq_block_size(w.dtype)
    oi = torch.zeros((m, n, kb), dtype=torch.int32, device=x.device)
    om = torch.zeros((m, n, kb), dtype=torch.int32, device=x.device) if w.dtype in (Q4K, Q5K) else None
    need = L.cq_workspace_bytes(w.handle, m, 0)
    ws = _default_ws.get(need, x.device)
    check(L.cq_qmatmul_int_dots(w.handle, C.c_void_p(x.data_ptr()), m, C.c_void_p(oi.data_ptr()),
                                C.c_void_p(om.data_ptr()) if om is not None else None,
                                C.c_void_p(ws.data_ptr()), ws.numel(), _stream_ptr()))
    return oi, om


MFMA_SKINNY, MFMA_TILE = 1, 2
MFMA_INT_MIN = 16   # added to either: the min-term contraction delivers the integer Mn_b


def qmatmul_int_dots_mfma(w: QWeight, x, kernel: int):
    """The block integers out of the matrix-core kernels: (int32 [m, n, blocks], float32 min term or None)."""
    torch = _torch()
    L = load()
    _require_f32_cuda(x)
    n, k = w.shape
    m = x.shape[0]
    kb = k // L.cq_block_size(w.dtype)
    oi = torch.full((m, n, kb), -(2 ** 31), dtype=torch.int32, device=x.device)
    om = torch.full((m, n, kb), float("nan"), dtype=torch.float32, device=x.device) if w.dtype in (Q4K, Q5K) else None
    need = L.cq_workspace_bytes(w.handle, m, 0)
    ws = _default_ws.get(need, x.device)
    check(L.cq_qmatmul_int_dots_mfma(w.handle, C.c_void_p(x.data_ptr()), m, kernel, C.c_void_p(oi.data_ptr()),
                                     C.c_void_p(om.data_ptr()) if om is not None else None,
                                     C.c_void_p(ws.data_ptr()), ws.numel(), _stream_ptr()))
    return oi, om


def qmatmul_grouped(experts, x, row_ids, offsets, flags: int = 0, workspace: Workspace | None = None,
                    pre: int = PRE_NONE, aux=None, eps: float = 0.0):
    """y[p] = x[row_ids[p]] . W_e^T for p in [offsets[e], offsets[e+1]); offsets is a host int32 array.
    With `pre`, the gathered rows go through that step first (aux rows gathered like x rows)."""
    torch = _torch()
    L = load()
    _require_f32_cuda(x)
    _check_pre(pre, x, aux)
    n, k = experts[0].shape
    offsets = np.ascontiguousarray(offsets, dtype=np.int32)
    total = int(offsets[-1])
    arr = (C.c_void_p * len(experts))(*[e.handle.value for e in experts])
    y = torch.empty((total, n), dtype=torch.float32, device=x.device)
    need = L.cq_grouped_workspace_bytes(arr, len(experts), total, flags)
    ws = (workspace or _default_ws).get(need, x.device)
    rid = C.c_void_p(row_ids.data_ptr()) if row_ids is not None else None
    if pre == PRE_NONE:
        check(L.cq_qmatmul_grouped(arr, len(experts), C.c_void_p(x.data_ptr()), rid,
                                   offsets.ctypes.data_as(C.POINTER(C.c_int32)), C.c_void_p(y.data_ptr()), flags,
                                   C.c_void_p(ws.data_ptr()), ws.numel(), _stream_ptr()))
    else:
        check(L.cq_qmatmul_grouped_fused(arr, len(experts), pre, C.c_void_p(x.data_ptr()), C.c_void_p(aux.data_ptr()),
                                         eps, rid, offsets.ctypes.data_as(C.POINTER(C.c_int32)),
                                         C.c_void_p(y.data_ptr()), flags, C.c_void_p(ws.data_ptr()), ws.numel(),
                                         _stream_ptr()))
    return y


def silu_mul(a, b):
    torch = _torch()
    h = torch.empty_like(a)
    check(load().cq_silu_mul(a.device.index or 0, C.c_void_p(a.data_ptr()), C.c_void_p(b.data_ptr()),
                             C.c_void_p(h.data_ptr()), a.numel(), _stream_ptr()))
    return h


def moe_scatter_add(y, row_ids, weights, tokens: int):
    torch = _torch()
    total, hidden = y.shape
    ys = torch.zeros((tokens, hidden), dtype=torch.float32, device=y.device)
    check(load().cq_moe_scatter_add(y.device.index or 0, C.c_void_p(y.data_ptr()), C.c_void_p(row_ids.data_ptr()),
                                    C.c_void_p(weights.data_ptr()), total, hidden, C.c_void_p(ys.data_ptr()),
                                    tokens, _stream_ptr()))
    return ys


def timed_kernel_us(launch) -> float:
    """Runs `launch()` (which must call cq_qmatmul once on this thread) with the library's kernel
    timer armed and returns the duration of its matmul kernel in microseconds."""
    L = load()
    check(L.cq_timing_arm())
    launch()
    us = C.c_double()
    check(L.cq_timing_elapsed_us(C.byref(us)))
    return us.value
