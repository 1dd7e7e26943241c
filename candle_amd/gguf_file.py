"""GGUF files -> quantized tensors on the device, and back.

Mirrors `candle-core/src/quantized/gguf_file.rs`:
  * `VersionedMagic` (:13-47): magic 0x46554747 ("GGUF"), versions 1-3; version 1 stores counts and
    string lengths as u32, versions 2 and 3 as u64,
  * `ValueType` / `Value` (:107-353) with the ids of `from_u32` (:355-373),
  * `TensorInfo` (:50-80) and `Content::read` / `Content::tensor` (:395-480),
  * `write` (:490-538): always version 2, 32-byte padding between tensors,
and the Python binding's `load_gguf` / `save_gguf` (candle-pyo3/src/lib.rs:1326-1459).

The tensor bytes of a file are GGML blocks; `Content.tensor` hands them to the device library,
which re-packs them into its own plane layout on upload (the loader funnel
`ggml_file.rs:120-188` `qtensor_from_ggml` -> `cuda.rs:591-612` `load_quantized`).  Parsing and
writing are host work and need neither the library nor a GPU; only `to_device` does.
"""
from __future__ import annotations

import enum
import io
import struct
from dataclasses import dataclass
from typing import Any, BinaryIO, Dict, Iterable, List, Sequence, Tuple

import numpy as np

GGUF_MAGIC = 0x46554747          # gguf_file.rs:17, the bytes "GGUF" read as a little-endian u32
DEFAULT_ALIGNMENT = 32           # gguf_file.rs:11


class GgufError(Exception):
    pass


# GGML type id -> (name, elements per block, bytes per block); ids from `GgmlDType::from_u32`
# (mod.rs:152-171), sizes from the block structs' size assertions (k_quants.rs:48-155).
_GGML_TYPES = {
    0: ("F32", 1, 4), 1: ("F16", 1, 2), 2: ("Q4_0", 32, 18), 3: ("Q4_1", 32, 20), 6: ("Q5_0", 32, 22),
    7: ("Q5_1", 32, 24), 8: ("Q8_0", 32, 34), 9: ("Q8_1", 32, 36), 10: ("Q2K", 256, 84),
    11: ("Q3K", 256, 110), 12: ("Q4K", 256, 144), 13: ("Q5K", 256, 176), 14: ("Q6K", 256, 210),
    15: ("Q8K", 256, 292),
}
# Types the device library holds as weights (everything else parses but cannot be uploaded).
DEVICE_WEIGHT_TYPES = (2, 3, 6, 7, 8, 10, 11, 12, 13, 14, 15)


def ggml_type_name(dtype: int) -> str:
    return _info(dtype)[0]


def ggml_block_size(dtype: int) -> int:
    return _info(dtype)[1]


def ggml_type_size(dtype: int) -> int:
    return _info(dtype)[2]


def _info(dtype: int):
    if dtype not in _GGML_TYPES:
        raise GgufError(f"unknown dtype for tensor {dtype}")
    return _GGML_TYPES[dtype]


class ValueType(enum.IntEnum):
    """gguf_file.rs:355-391."""
    U8 = 0
    I8 = 1
    U16 = 2
    I16 = 3
    U32 = 4
    I32 = 5
    F32 = 6
    BOOL = 7
    STRING = 8
    ARRAY = 9
    U64 = 10
    I64 = 11
    F64 = 12


_SCALAR_FMT = {ValueType.U8: "<B", ValueType.I8: "<b", ValueType.U16: "<H", ValueType.I16: "<h",
               ValueType.U32: "<I", ValueType.I32: "<i", ValueType.U64: "<Q", ValueType.I64: "<q",
               ValueType.F32: "<f", ValueType.F64: "<d"}


@dataclass(frozen=True)
class Value:
    """A typed metadata value (`Value`, gguf_file.rs:140-155).  `v` is an int, float, bool, str, or
    for ARRAY a list of `Value`s."""
    type: ValueType
    v: Any

    def to_python(self):
        """Plain Python object, as the reference's binding returns it (lib.rs:1339-1362)."""
        if self.type == ValueType.ARRAY:
            return [e.to_python() for e in self.v]
        return self.v

    @classmethod
    def infer(cls, obj) -> "Value":
        """Type a plain Python object: bool -> BOOL, int -> the first of u8, i8, u16, i16, u32, i32,
        u64, i64 that holds it, float -> F32, str -> STRING, list/tuple -> ARRAY (the extraction order
        of lib.rs:1394-1424; a Python bool is typed BOOL here)."""
        if isinstance(obj, Value):
            return obj
        if isinstance(obj, (bool, np.bool_)):
            return cls(ValueType.BOOL, bool(obj))
        if isinstance(obj, (int, np.integer)):
            obj = int(obj)
            for t, lo, hi in ((ValueType.U8, 0, 2**8), (ValueType.I8, -2**7, 2**7),
                              (ValueType.U16, 0, 2**16), (ValueType.I16, -2**15, 2**15),
                              (ValueType.U32, 0, 2**32), (ValueType.I32, -2**31, 2**31),
                              (ValueType.U64, 0, 2**64), (ValueType.I64, -2**63, 2**63)):
                if lo <= obj < hi:
                    return cls(t, obj)
            raise GgufError(f"unsupported type {obj!r}")
        if isinstance(obj, (float, np.floating)):
            return cls(ValueType.F32, float(obj))
        if isinstance(obj, str):
            return cls(ValueType.STRING, obj)
        if isinstance(obj, (list, tuple)):
            return cls(ValueType.ARRAY, [cls.infer(e) for e in obj])
        raise GgufError(f"unsupported type {obj!r}")


def _read_exact(r: BinaryIO, n: int) -> bytes:
    b = r.read(n)
    if len(b) != n:
        raise GgufError("failed to fill whole buffer")      # std::io::ErrorKind::UnexpectedEof
    return b


def _read(r: BinaryIO, fmt: str):
    return struct.unpack(fmt, _read_exact(r, struct.calcsize(fmt)))[0]


def _read_len(r: BinaryIO, version: int) -> int:
    return _read(r, "<I") if version == 1 else _read(r, "<Q")


def _read_string(r: BinaryIO, version: int) -> str:
    """gguf_file.rs:91-105: length-prefixed, trailing NULs dropped, invalid UTF-8 replaced."""
    raw = _read_exact(r, _read_len(r, version))
    return raw.rstrip(b"\x00").decode("utf-8", errors="replace")


def _value_type(u: int) -> ValueType:
    try:
        return ValueType(u)
    except ValueError:
        raise GgufError(f"unrecognized value-type {u:#08x}") from None


def _read_value(r: BinaryIO, t: ValueType, version: int) -> Value:
    """`Value::read` (gguf_file.rs:274-314)."""
    if t in _SCALAR_FMT:
        return Value(t, _read(r, _SCALAR_FMT[t]))
    if t == ValueType.BOOL:
        b = _read(r, "<B")
        if b > 1:
            raise GgufError(f"unexpected bool value {b}")
        return Value(t, bool(b))
    if t == ValueType.STRING:
        return Value(t, _read_string(r, version))
    elem_t = _value_type(_read(r, "<I"))
    n = _read_len(r, version)
    return Value(t, [_read_value(r, elem_t, version) for _ in range(n)])


def _write_string(w: BinaryIO, s: str):
    b = s.encode("utf-8")
    w.write(struct.pack("<Q", len(b)))
    w.write(b)


def _write_value(w: BinaryIO, val: Value):
    """`Value::write` (gguf_file.rs:316-353)."""
    t = val.type
    if t in _SCALAR_FMT:
        try:
            w.write(struct.pack(_SCALAR_FMT[t], val.v))
        except struct.error as e:
            raise GgufError(f"{val.v!r} does not fit {t.name}: {e}") from None
    elif t == ValueType.BOOL:
        w.write(struct.pack("<B", 1 if val.v else 0))
    elif t == ValueType.STRING:
        _write_string(w, val.v)
    else:
        kinds = {e.type for e in val.v}
        if len(kinds) > 1:
            raise GgufError(f"multiple value-types in the same array {sorted(k.name for k in kinds)}")
        elem_t = kinds.pop() if kinds else ValueType.U32      # an empty array is written as u32[0]
        w.write(struct.pack("<IQ", int(elem_t), len(val.v)))
        for e in val.v:
            _write_value(w, e)


class HostQTensor:
    """GGML blocks in host memory with their type and shape: what a file holds for one tensor and
    what `write` needs of one.  No arithmetic happens on it; `to_device` uploads it."""

    def __init__(self, dtype: int, blocks, shape: Sequence[int]):
        self._dtype = int(dtype)
        self._shape = tuple(int(s) for s in shape)
        self._blocks = np.ascontiguousarray(np.frombuffer(blocks, dtype=np.uint8)
                                            if isinstance(blocks, (bytes, bytearray, memoryview))
                                            else np.asarray(blocks)).view(np.uint8).reshape(-1)
        want = tensor_size_in_bytes(self._dtype, self._shape)
        if self._blocks.size != want:
            raise GgufError(f"{self._blocks.size} bytes given for a {ggml_type_name(self._dtype)} tensor of "
                            f"shape {self._shape}, which takes {want}")

    def dtype(self) -> int:
        return self._dtype

    @property
    def ggml_dtype(self) -> str:
        return ggml_type_name(self._dtype)

    @property
    def shape(self) -> Tuple[int, ...]:
        return self._shape

    def storage_size_in_bytes(self) -> int:
        return self._blocks.size

    def data(self) -> np.ndarray:
        return self._blocks

    def to_device(self, dev: int = 0):
        """Upload: quantized types become a `QTensor` on the device; F32 / F16 tensors (norm weights,
        biases) become a plain torch tensor of that dtype."""
        if self._dtype in (0, 1):
            import torch
            host = self._blocks.view(np.float32 if self._dtype == 0 else np.float16).reshape(self._shape)
            return torch.from_numpy(host.copy()).to(f"cuda:{dev}")
        if self._dtype not in DEVICE_WEIGHT_TYPES:
            raise GgufError(f"{self.ggml_dtype} tensors are not supported on the device "
                            f"(supported: {', '.join(ggml_type_name(t) for t in DEVICE_WEIGHT_TYPES)}, F32, F16)")
        from .quantized import QTensor
        return QTensor.from_ggml(self._dtype, self._blocks, self._shape, dev)


def tensor_size_in_bytes(dtype: int, shape: Sequence[int]) -> int:
    """gguf_file.rs:62-69: whole blocks only."""
    elems = 1
    for s in shape:
        elems *= int(s)
    bs = ggml_block_size(dtype)
    if elems % bs != 0:
        raise GgufError(f"the number of elements {elems} is not divisible by the block size {bs}")
    return elems // bs * ggml_type_size(dtype)


@dataclass(frozen=True)
class TensorInfo:
    """gguf_file.rs:50-54.  `shape` is outermost first (the file stores it innermost first);
    `offset` counts from `Content.tensor_data_offset`."""
    ggml_dtype: int
    shape: Tuple[int, ...]
    offset: int

    def read(self, r: BinaryIO, tensor_data_offset: int) -> HostQTensor:
        """gguf_file.rs:56-79."""
        size = tensor_size_in_bytes(self.ggml_dtype, self.shape)
        r.seek(tensor_data_offset + self.offset)
        buf = np.empty(size, dtype=np.uint8)
        got = r.readinto(memoryview(buf)) if hasattr(r, "readinto") else None
        if got is None:
            buf = np.frombuffer(_read_exact(r, size), dtype=np.uint8)
        elif got != size:
            raise GgufError("failed to fill whole buffer")
        return HostQTensor(self.ggml_dtype, buf, self.shape)


class Content:
    """The header of a GGUF file (gguf_file.rs:84-89)."""

    def __init__(self, version: int, metadata: Dict[str, Value], tensor_infos: Dict[str, TensorInfo],
                 tensor_data_offset: int):
        self.version = version
        self.metadata = metadata
        self.tensor_infos = tensor_infos
        self.tensor_data_offset = tensor_data_offset

    @classmethod
    def read(cls, r: BinaryIO) -> "Content":
        """`Content::read` (gguf_file.rs:395-468)."""
        magic = _read(r, "<I")
        if magic != GGUF_MAGIC:
            raise GgufError(f"unknown magic 0x{magic:08x}")
        version = _read(r, "<I")
        if version not in (1, 2, 3):
            raise GgufError(f"gguf: unsupported magic/version Gguf/{version}")
        tensor_count = _read_len(r, version)
        kv_count = _read_len(r, version)
        metadata: Dict[str, Value] = {}
        for _ in range(kv_count):
            key = _read_string(r, version)
            t = _value_type(_read(r, "<I"))
            metadata[key] = _read_value(r, t, version)
        infos: Dict[str, TensorInfo] = {}
        for _ in range(tensor_count):
            name = _read_string(r, version)
            n_dims = _read(r, "<I")
            fmt = "<I" if version == 1 else "<Q"
            dims = [_read(r, fmt) for _ in range(n_dims)]
            dims.reverse()
            dtype = _read(r, "<I")
            _info(dtype)
            offset = _read(r, "<Q")
            infos[name] = TensorInfo(dtype, tuple(dims), offset)
        position = r.tell()
        alignment = DEFAULT_ALIGNMENT
        a = metadata.get("general.alignment")
        if a is not None and a.type in (ValueType.U8, ValueType.U16, ValueType.U32, ValueType.I8,
                                        ValueType.I16, ValueType.I32) and a.v >= 0:
            alignment = a.v
        if alignment == 0:
            raise GgufError("general.alignment is zero")
        return cls(version, metadata, infos, -(-position // alignment) * alignment)

    def tensor_host(self, r: BinaryIO, name: str) -> HostQTensor:
        info = self.tensor_infos.get(name)
        if info is None:
            raise GgufError(f"cannot find tensor info for {name}")
        return info.read(r, self.tensor_data_offset)

    def tensor_view(self, buf, name: str) -> HostQTensor:
        """The tensor's blocks as a view into `buf`, the whole file as a buffer (an `mmap`, `bytes`):
        nothing is copied on the host, the upload reads the file's pages directly (what the
        reference's reader leaves as a TODO, ggml_file.rs:213)."""
        info = self.tensor_infos.get(name)
        if info is None:
            raise GgufError(f"cannot find tensor info for {name}")
        size = tensor_size_in_bytes(info.ggml_dtype, info.shape)
        start = self.tensor_data_offset + info.offset
        if start + size > len(buf):
            raise GgufError("failed to fill whole buffer")
        return HostQTensor(info.ggml_dtype, np.frombuffer(buf, dtype=np.uint8, count=size, offset=start), info.shape)

    def tensor(self, r: BinaryIO, name: str, dev: int = 0):
        """`Content::tensor` (gguf_file.rs:470-481) with a device: read the blocks, upload, re-pack."""
        return self.tensor_host(r, name).to_device(dev)


def _pad32(n: int) -> int:
    return 31 - (31 + n) % 32


def write(w: BinaryIO, metadata: Iterable[Tuple[str, Any]], tensors: Iterable[Tuple[str, Any]]):
    """`gguf_file::write` (gguf_file.rs:490-538).  `metadata` values are `Value`s or plain Python
    objects (typed by `Value.infer`); a tensor is anything with `shape`, `dtype()` (GGML type id),
    `storage_size_in_bytes()` and `data()` (GGML blocks as bytes): a `HostQTensor`, or a device
    `QTensor`, whose blocks are brought back in GGML order."""
    metadata = [(k, Value.infer(v)) for k, v in metadata]
    tensors = list(tensors)
    start = w.tell()
    w.write(struct.pack("<IIQQ", GGUF_MAGIC, 2, len(tensors), len(metadata)))
    for key, val in metadata:
        _write_string(w, key)
        w.write(struct.pack("<I", int(val.type)))
        _write_value(w, val)
    offset = 0
    offsets: List[int] = []
    for name, t in tensors:
        _write_string(w, name)
        dims = tuple(int(d) for d in t.shape)
        w.write(struct.pack("<I", len(dims)))
        for d in reversed(dims):
            w.write(struct.pack("<Q", d))
        w.write(struct.pack("<IQ", int(t.dtype()), offset))
        offsets.append(offset)
        size = int(t.storage_size_in_bytes())
        offset += size + _pad32(size)
    pos = w.tell() - start
    w.write(bytes(_pad32(pos)))
    tensor_start = w.tell() - start
    for off, (name, t) in zip(offsets, tensors):
        pos = w.tell() - start
        if tensor_start + off != pos:
            raise GgufError(f"internal error, unexpected current position {tensor_start} {off} {pos}")
        data = np.ascontiguousarray(t.data()).view(np.uint8).reshape(-1)
        if data.size != int(t.storage_size_in_bytes()):
            raise GgufError(f"tensor {name}: data() holds {data.size} bytes, "
                            f"storage_size_in_bytes() says {t.storage_size_in_bytes()}")
        w.write(data.tobytes())
        w.write(bytes(_pad32(data.size)))


def load_gguf(path: str, dev: int = 0):
    """`load_gguf(path, device)` of the Python binding (lib.rs:1326-1382): every tensor of the file on
    the device, and the metadata as plain Python objects."""
    import mmap
    with open(path, "rb") as f:
        content = Content.read(f)
        if not content.tensor_infos:
            return {}, {k: v.to_python() for k, v in content.metadata.items()}
        # The tensor bytes go from the page cache to the device without a host copy of our own.  The
        # mapping is not closed by hand: it goes away with the last view into it (an upload that
        # raises still holds one in its traceback, and closing under it would be an error of its own).
        mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
        tensors = {name: content.tensor_view(mm, name).to_device(dev) for name in content.tensor_infos}
    return tensors, {k: v.to_python() for k, v in content.metadata.items()}


def save_gguf(path: str, tensors: Dict[str, Any], metadata: Dict[str, Any]):
    """`save_gguf(path, tensors, metadata)` (lib.rs:1384-1459)."""
    if not isinstance(tensors, dict):
        raise ValueError("expected a dict")
    if not isinstance(metadata, dict):
        raise ValueError("expected a dict")
    for k in list(tensors) + list(metadata):
        if not isinstance(k, str):
            raise ValueError("keys must be strings")
    with open(path, "wb") as f:
        write(f, list(metadata.items()), list(tensors.items()))


def read_bytes(buf: bytes) -> Content:
    return Content.read(io.BytesIO(buf))
