"""The reference's quantized-tensor surface on top of libcandle_qhip.so.

Mirrors, name for name:
  * `GgmlDType` (candle-core/src/quantized/mod.rs:133-247): ids, `block_size`, `type_size`,
  * `QTensor` (mod.rs:35-38, 318-392): `quantize`, `dtype`, `shape`, `rank`, `dequantize`,
    `dequantize_f16`, `storage_size_in_bytes`,
  * `QMatMul` (mod.rs:394-462, 527-550): `from_qtensor`, `forward`,
  * the Python binding's `QTensor.matmul_t` (candle-pyo3/src/lib.rs:1250-1255) and
    `Tensor.quantize(str)` (lib.rs:1079-1102).
Tensors are torch CUDA tensors (torch only owns the memory and the stream); every operation runs in
the HIP library, and fails if that library or a GPU is missing.
"""
from __future__ import annotations

import enum

import numpy as np

from . import qhip


class GgmlDType(enum.IntEnum):
    """GGML type ids as stored in GGUF files (mod.rs:152-171 `from_u32`, :173-190 `to_u32`).
    Only the types this library computes with are listed."""
    F32 = 0
    F16 = 1
    Q4_0 = 2
    Q4_1 = 3
    Q5_0 = 6
    Q5_1 = 7
    Q8_0 = 8
    Q8_1 = 9
    Q2K = 10
    Q3K = 11
    Q4K = 12
    Q5K = 13
    Q6K = 14
    Q8K = 15

    @classmethod
    def from_str(cls, name: str) -> "GgmlDType":
        """Names accepted by the reference's Python `Tensor.quantize` (lib.rs:1082-1098)."""
        table = {"q4_0": cls.Q4_0, "q4_1": cls.Q4_1, "q5_0": cls.Q5_0, "q5_1": cls.Q5_1, "q8_0": cls.Q8_0, "q8_1": cls.Q8_1, "q2k": cls.Q2K, "q3k": cls.Q3K, "q4k": cls.Q4K,
                 "q5k": cls.Q5K, "q6k": cls.Q6K,
                 "q8k": cls.Q8K, "f32": cls.F32, "f16": cls.F16}
        key = name.lower()
        if key not in table:
            raise ValueError(f"'{name}' is not a valid quantization type or is not supported by this build")
        return table[key]

    def block_size(self) -> int:
        """mod.rs:234-246."""
        if self in (GgmlDType.F32, GgmlDType.F16):
            return 1
        return qhip.load().cq_block_size(int(self))

    def type_size(self) -> int:
        """Bytes per block (mod.rs:212-232)."""
        if self == GgmlDType.F32:
            return 4
        if self == GgmlDType.F16:
            return 2
        return qhip.load().cq_type_size(int(self))

    def vec_dot_type(self) -> "GgmlDType":
        """The activation type `matmul` quantizes to (`GgmlType::VecDotType`, k_quants.rs)."""
        return GgmlDType(qhip.load().cq_vec_dot_type(int(self)))


_WEIGHT_TYPES = (GgmlDType.Q4_0, GgmlDType.Q4_1, GgmlDType.Q5_0, GgmlDType.Q5_1, GgmlDType.Q8_0, GgmlDType.Q2K, GgmlDType.Q3K, GgmlDType.Q4K, GgmlDType.Q5K, GgmlDType.Q6K, GgmlDType.Q8K)


class QTensor:
    """A quantized tensor on the device (mod.rs:318-392).  The matmul path takes rank-2 `[n, k]`
    tensors; higher ranks are kept as their shape with the leading dims flattened into `n`."""

    def __init__(self, weight: qhip.QWeight, shape):
        """`QTensor::new(storage, shape)` (mod.rs:318-323): the shape is checked against the block size and
        the storage's element count, and becomes the [rows, k] the matmul entry points read the storage as."""
        self._w = weight
        self._shape = tuple(int(s) for s in shape)
        _check_shape(self._shape, qhip.load().cq_block_size(weight.dtype))
        k = self._shape[-1]
        rows = int(np.prod(self._shape[:-1])) if len(self._shape) > 1 else 1
        # The shape is state of the storage handle (the entry points without a shape argument read it): a second
        # QTensor over the same storage with another shape would silently re-shape the first.
        fixed = getattr(weight, "_qtensor_dims", None)
        if fixed is not None and fixed != (rows, k):
            raise qhip.QHipError(f"storage is already viewed as {fixed} by another QTensor; a second view {(rows, k)} "
                                 "goes through qhip.qmatmul_shaped, which takes the shape with the call")
        weight.set_shape(rows, k)
        weight._qtensor_dims = (rows, k)

    # ---- constructors ---------------------------------------------------------------------
    @classmethod
    def quantize(cls, src, dtype) -> "QTensor":
        """`QTensor::quantize(src, dtype)` (mod.rs:325-343): src f32, last dim a multiple of the
        block size.  Quantizes on the device, bit-identical to the CPU `from_float`."""
        dtype = GgmlDType.from_str(dtype) if isinstance(dtype, str) else GgmlDType(dtype)
        if dtype not in _WEIGHT_TYPES:
            raise qhip.QHipError(f"quantize: unsupported dtype {dtype.name}")
        shape = tuple(src.shape)
        _check_shape(shape, dtype.block_size())
        # Device::qzeros(elem_count, dtype) then QStorage::quantize (mod.rs:331-338): the storage has no shape
        w = qhip.QWeight.zeros_flat(int(dtype), int(np.prod(shape)), dev=src.device.index or 0)
        w.quantize_(src.contiguous() if not src.is_contiguous() else src)
        return cls(w, shape)

    @classmethod
    def from_ggml(cls, dtype, blocks: np.ndarray, shape, dev: int = 0) -> "QTensor":
        """Host GGML blocks -> device (the loader funnel `ggml_file.rs:120-135` -> `cuda.rs:591-612`)."""
        dtype = GgmlDType(dtype)
        shape = tuple(int(s) for s in shape)
        _check_shape(shape, dtype.block_size())
        return cls(qhip.QWeight.from_ggml_flat(int(dtype), blocks, dev), shape)

    # ---- getters (mod.rs:345-359; lib.rs:1214-1240) ---------------------------------------------
    @property
    def ggml_dtype(self) -> str:
        return GgmlDType(self._w.dtype).name

    def dtype(self) -> GgmlDType:
        return GgmlDType(self._w.dtype)

    @property
    def shape(self):
        return self._shape

    def rank(self) -> int:
        return len(self._shape)

    def storage_size_in_bytes(self) -> int:
        return self._w.size_in_bytes

    @property
    def weight(self) -> qhip.QWeight:
        return self._w

    # ---- operations -----------------------------------------------------------------------------
    def dequantize(self):
        """mod.rs:361-365."""
        return self._w.dequantize().reshape(self._shape)

    def dequantize_f16(self):
        """mod.rs:367-382: equals `dequantize().to(f16)` bit for bit."""
        return self._w.dequantize_f16().reshape(self._shape)

    def data(self) -> np.ndarray:
        """The GGML blocks on the host (`QTensor::data`, mod.rs:388-391).  The reference's device
        backends bail here; this build offers the inverse re-pack instead."""
        return self._w.to_ggml()

    def matmul_t(self, lhs):
        """`lhs @ self.T` (lib.rs:1250-1255)."""
        return QMatMul.from_qtensor(self).forward(lhs)

    def __repr__(self) -> str:
        return f"QTensor[{self._shape}; {self.ggml_dtype.lower()}]"


def _check_shape(shape, block_size: int):
    """`check_shape` (mod.rs:304-316)."""
    if len(shape) == 0:
        raise qhip.QHipError("scalar tensor cannot be quantized")
    if shape[-1] % block_size != 0:
        raise qhip.QHipError(f"quantized tensor must have their last dim divisible by block size "
                             f"{tuple(shape)} {block_size}")


def _env_switch(name: str) -> bool:
    """mod.rs:400-420: set and neither empty nor "0"."""
    import os
    v = os.environ.get(name)
    return v is not None and v != "" and v != "0"


class QMatMul:
    """`QMatMul` (mod.rs:394-462): y = x . W^T.  The `QTensor` arm keeps W quantized and runs the device
    kernels; `from_arc` picks the `Tensor` / `TensorF16` arms (W dequantized once, then the host
    framework's dense matmul: torch here, candle's own on the Rust side) when `CANDLE_DEQUANTIZE_ALL` /
    `CANDLE_DEQUANTIZE_ALL_F16` ask for it (mod.rs:423-438)."""

    def __init__(self, qtensor: QTensor, arm: str = "QTensor", dense=None):
        if qtensor.rank() != 2:
            raise qhip.QHipError(f"QMatMul needs a rank-2 weight, got {qtensor.shape}")
        self.qtensor = qtensor
        self.arm = arm          # "QTensor" | "Tensor" | "TensorF16"
        self.dense = dense      # the dequantized weight of the two dense arms
        self._ws = qhip.Workspace()

    @classmethod
    def from_qtensor(cls, qtensor: QTensor) -> "QMatMul":
        return cls.from_arc(qtensor)

    @classmethod
    def from_arc(cls, qtensor: QTensor) -> "QMatMul":
        if _env_switch("CANDLE_DEQUANTIZE_ALL"):
            return cls(qtensor, "Tensor", qtensor.dequantize())
        if _env_switch("CANDLE_DEQUANTIZE_ALL_F16"):
            return cls(qtensor, "TensorF16", qtensor.dequantize_f16())
        return cls(qtensor)

    def forward(self, xs):
        """mod.rs:528-550 -> `cpu_fwd` semantics (mod.rs:469-500): xs f32, contiguous, rank >= 2,
        last dim == k; result has xs' shape with the last dim replaced by n."""
        if self.arm == "Tensor":        # mod.rs:531-538
            return xs.matmul(self.dense.t())
        if self.arm == "TensorF16":     # mod.rs:539-547
            return xs.to(self.dense.dtype).matmul(self.dense.t()).to(xs.dtype)
        return qhip.qmatmul(self.qtensor.weight, xs, workspace=self._ws)

    def forward_via_f16(self, xs):
        """mod.rs:452-461."""
        w = self.dequantize_f16()
        return xs.to(w.dtype).matmul(w.t()).to(xs.dtype)

    def forward_rms_norm(self, xs, alpha, eps: float):
        """`self.forward(rms_norm(xs, alpha, eps))` (RmsNorm::forward, candle-transformers/src/
        quantized_nn.rs:121-125, in front of a projection as in quantized_llama.rs:453-466) without
        the normalised tensor going to memory."""
        return qhip.qmatmul(self.qtensor.weight, xs, workspace=self._ws, pre=qhip.PRE_RMS_NORM, aux=alpha, eps=eps)

    def forward_silu_mul(self, gate, up):
        """`self.forward(silu(gate) * up)`: the feed-forward's w2 applied to silu(w1 x) * (w3 x)
        (Mlp::forward, quantized_llama.rs:56-63)."""
        return qhip.qmatmul(self.qtensor.weight, gate, workspace=self._ws, pre=qhip.PRE_SILU_MUL, aux=up)

    @staticmethod
    def forward_multi(mats, xs, alpha=None, eps: float = 0.0):
        """`[m.forward(xs) for m in mats]` (with `alpha`: of rms_norm(xs, alpha, eps)) for matrices of one
        dtype and row length, as the q, k, v projections (quantized_llama.rs:206-208) or w1 and w3
        (:60-61): one launch for one activation row, the rows quantized once otherwise."""
        mats = list(mats)
        pre = qhip.PRE_NONE if alpha is None else qhip.PRE_RMS_NORM
        return qhip.qmatmul_multi([m.qtensor.weight for m in mats], xs, workspace=mats[0]._ws, pre=pre, aux=alpha, eps=eps)

    def dequantize_f16(self):
        """mod.rs:444-450."""
        if self.arm == "Tensor":
            return self.dense.half()
        if self.arm == "TensorF16":
            return self.dense
        return self.qtensor.dequantize_f16()
