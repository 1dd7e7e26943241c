"""Legacy GGML / GGMF / GGJT files -> quantized tensors on the device.

Mirrors `candle-core/src/quantized/ggml_file.rs`:
  * `VersionedMagic` (:33-66): magic "ggml" (no version word), "ggmf" version 1, "ggjt" versions
    1-3; the ggjt variants align tensor data to 32 bytes,
  * `HParams` (:68-99): seven u32 in file order,
  * `Vocab` (:101-120): per token a u32 length, the bytes and an f32 score (read for every
    magic, as the reference does),
  * `read_one_tensor` (:190-223): u32 n_dims, name length, GGML type id; dims stored innermost
    first and reversed on the way in; name; padding; the block bytes,
  * `Content::read` / `remove` (:225-268): tensors until the end of the file,
and the Python binding's `load_ggml` (candle-pyo3/src/lib.rs:1290-1324), which returns the
tensors, the hyper-parameters as a dict and the vocabulary as (lossily decoded) strings.

Tensor bytes go to the device through the same funnel as GGUF tensors (`qtensor_from_ggml`,
:138-188): `HostQTensor.to_device`.  Parsing needs neither the library nor a GPU.
"""
from __future__ import annotations

import enum
import io
import os
import struct
from dataclasses import dataclass
from typing import BinaryIO, Dict, List, Tuple

import numpy as np

from .gguf_file import HostQTensor, _GGML_TYPES, tensor_size_in_bytes


class GgmlFileError(Exception):
    pass


_MAGICS = {0x67676a74: "ggjt", 0x67676c61: "ggla", 0x67676d66: "ggmf", 0x67676d6c: "ggml", 0x6767736e: "ggsn"}


class VersionedMagic(enum.Enum):
    GgmlUnversioned = "ggml"
    GgmfV1 = "ggmf.1"
    GgjtV1 = "ggjt.1"
    GgjtV2 = "ggjt.2"
    GgjtV3 = "ggjt.3"

    def align32(self) -> bool:   # ggml_file.rs:60-65
        return self in (VersionedMagic.GgjtV1, VersionedMagic.GgjtV2, VersionedMagic.GgjtV3)


def _read_exact(r: BinaryIO, n: int) -> bytes:
    b = r.read(n)
    if len(b) != n:
        raise GgmlFileError(f"unexpected end of file: wanted {n} bytes, got {len(b)}")
    return b


def _u32(r: BinaryIO) -> int:
    return struct.unpack("<I", _read_exact(r, 4))[0]


def _read_magic(r: BinaryIO) -> VersionedMagic:
    value = _u32(r)
    if value not in _MAGICS:
        raise GgmlFileError(f"unknown magic {value:08x}")
    magic = _MAGICS[value]
    if magic == "ggml":
        return VersionedMagic.GgmlUnversioned
    version = _u32(r)
    try:
        return VersionedMagic(f"{magic}.{version}")
    except ValueError:
        raise GgmlFileError(f"ggml: unsupported magic/version {magic}/{version}") from None


@dataclass
class HParams:
    n_vocab: int
    n_embd: int
    n_mult: int
    n_head: int
    n_layer: int
    n_rot: int
    ftype: int

    @classmethod
    def read(cls, r: BinaryIO) -> "HParams":
        return cls(*struct.unpack("<7I", _read_exact(r, 28)))

    def as_dict(self) -> Dict[str, int]:   # the order of candle-pyo3/src/lib.rs:1306-1314
        return {"n_vocab": self.n_vocab, "n_embd": self.n_embd, "n_mult": self.n_mult, "n_head": self.n_head,
                "n_layer": self.n_layer, "n_rot": self.n_rot, "ftype": self.ftype}


@dataclass
class Vocab:
    token_score_pairs: List[Tuple[bytes, float]]

    @classmethod
    def read(cls, r: BinaryIO, n_vocab: int) -> "Vocab":
        pairs = []
        for _ in range(n_vocab):
            word = _read_exact(r, _u32(r))
            score = struct.unpack("<f", _read_exact(r, 4))[0]
            pairs.append((word, score))
        return cls(pairs)


def _read_one_tensor(r: BinaryIO, magic: VersionedMagic) -> Tuple[str, HostQTensor]:
    n_dims, name_len, dtype = struct.unpack("<3I", _read_exact(r, 12))
    if dtype not in _GGML_TYPES:
        raise GgmlFileError(f"unknown dtype for tensor {dtype}")     # GgmlDType::from_u32, mod.rs:152-171
    dims = list(struct.unpack(f"<{n_dims}I", _read_exact(r, 4 * n_dims)))
    dims.reverse()
    name = _read_exact(r, name_len).decode("utf-8", errors="replace")
    if magic.align32():
        pos = r.tell()
        r.seek((32 - pos % 32) % 32, os.SEEK_CUR)
    try:
        nbytes = tensor_size_in_bytes(dtype, dims)
    except Exception as e:   # element count not a multiple of the block size (ggml_file.rs:146-150)
        raise GgmlFileError(f"Error creating tensor {name}: {e}") from None
    blocks = np.frombuffer(_read_exact(r, nbytes), dtype=np.uint8).copy()
    return name, HostQTensor(dtype, blocks, dims)


class Content:
    """`ggml_file::Content` (:225-268): everything a legacy GGML file holds, tensors on the host."""

    def __init__(self, magic: VersionedMagic, hparams: HParams, vocab: Vocab, tensors: Dict[str, HostQTensor]):
        self.magic, self.hparams, self.vocab, self.tensors = magic, hparams, vocab, tensors

    @classmethod
    def read(cls, r: BinaryIO) -> "Content":
        last_position = r.seek(0, os.SEEK_END)
        r.seek(0)
        magic = _read_magic(r)
        hparams = HParams.read(r)
        vocab = Vocab.read(r, hparams.n_vocab)
        tensors: Dict[str, HostQTensor] = {}
        while r.tell() != last_position:
            name, t = _read_one_tensor(r, magic)
            tensors[name] = t
        return cls(magic, hparams, vocab, tensors)

    def remove(self, name: str) -> HostQTensor:
        if name not in self.tensors:
            raise GgmlFileError(f"cannot find tensor with name '{name}'")
        return self.tensors.pop(name)


def read_bytes(buf: bytes) -> Content:
    return Content.read(io.BytesIO(buf))


def load_ggml(path: str, dev: int = 0):
    """`candle.utils.load_ggml` (candle-pyo3/src/lib.rs:1290-1324): (tensors on device `dev`,
    hyper-parameters, vocabulary strings)."""
    with open(path, "rb") as f:
        content = Content.read(f)
    tensors = {name: t.to_device(dev) for name, t in content.tensors.items()}
    vocab = [w.decode("utf-8", errors="replace") for w, _ in content.vocab.token_score_pairs]
    return tensors, content.hparams.as_dict(), vocab
