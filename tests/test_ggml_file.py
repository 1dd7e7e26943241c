"""Legacy GGML / GGMF / GGJT reader (candle_amd/ggml_file.py, after ggml_file.rs) and its device loader.

The reference holds no fixture and no test of this module; the format is pinned by files spelled out
byte by byte from the layout its reader walks (ggml_file.rs:42-58, :79-99, :107-119, :195-222): magic
[, version], seven u32 hyper-parameters, n_vocab x (u32 length, bytes, f32 score), then per tensor
u32 n_dims, u32 name length, u32 type id, the dims innermost first, the name, for "ggjt" padding to
a multiple of 32, and the block bytes.
"""
import io
import struct

import numpy as np
import pytest

from candle_amd import ggml_file as GF
from candle_amd.ggml_file import Content, GgmlFileError, VersionedMagic


def u32(*vs):
    return b"".join(int(v).to_bytes(4, "little") for v in vs)


def f32(v):
    return struct.pack("<f", v)


HPARAMS = u32(2, 64, 256, 8, 1, 16, 7)                       # n_vocab = 2, ..., ftype = 7
VOCAB = u32(1) + b"a" + f32(-1.5) + u32(3) + b"\xe2\x82\xac" + f32(0.25)      # "a", the euro sign
Q8_0_ROWS = bytes(range(204))                                # 3 rows x 2 blocks x 34 bytes
F32_VALS = np.array([1.0, -2.0, 0.5, 3.0], np.float32)

# "ggjt" version 3: tensor data aligned to 32 bytes
GGJT_HEAD = b"tjgg" + u32(3) + HPARAMS + VOCAB
assert len(GGJT_HEAD) == 8 + 28 + 20
GGJT_T0 = u32(2, 1, 8) + u32(64, 3) + b"w"                    # Q8_0, dims stored as [64, 3], name "w"
assert len(GGJT_HEAD + GGJT_T0) == 77
GGJT_FILE = GGJT_HEAD + GGJT_T0 + bytes(19) + Q8_0_ROWS       # data at 96
GGJT_T1 = u32(1, 4, 0) + u32(4) + b"norm"                     # F32 [4], name "norm"
assert len(GGJT_FILE + GGJT_T1) == 300 + 20
GGJT_FILE += GGJT_T1 + F32_VALS.tobytes()                     # 320 is already a multiple of 32

# unversioned "ggml": no version word, no padding
GGML_FILE = b"lmgg" + HPARAMS + VOCAB + u32(2, 2, 8) + u32(32, 2) + b"ab" + Q8_0_ROWS[:68]
# "ggmf" version 1: a version word, no padding
GGMF_FILE = b"fmgg" + u32(1) + HPARAMS + VOCAB + u32(1, 1, 1) + u32(3) + b"h" + np.arange(3, dtype=np.float16).tobytes()


def test_read_ggjt_literal():
    c = Content.read(io.BytesIO(GGJT_FILE))
    assert c.magic == VersionedMagic.GgjtV3 and c.magic.align32()
    assert c.hparams.as_dict() == {"n_vocab": 2, "n_embd": 64, "n_mult": 256, "n_head": 8, "n_layer": 1, "n_rot": 16,
                                   "ftype": 7}
    assert c.vocab.token_score_pairs == [(b"a", -1.5), ("€".encode(), 0.25)]
    assert sorted(c.tensors) == ["norm", "w"]
    w = c.tensors["w"]
    assert (w.dtype(), w.shape, w.ggml_dtype) == (8, (3, 64), "Q8_0")      # dims reversed on read
    assert w.data().tobytes() == Q8_0_ROWS
    n = c.tensors["norm"]
    assert (n.dtype(), n.shape) == (0, (4,)) and n.data().tobytes() == F32_VALS.tobytes()
    assert c.remove("w") is w and "w" not in c.tensors
    with pytest.raises(GgmlFileError, match="cannot find tensor"):
        c.remove("w")


def test_read_unversioned_and_ggmf_literals():
    c = GF.read_bytes(GGML_FILE)
    assert c.magic == VersionedMagic.GgmlUnversioned and not c.magic.align32()
    assert c.tensors["ab"].shape == (2, 32) and c.tensors["ab"].data().tobytes() == Q8_0_ROWS[:68]
    c = GF.read_bytes(GGMF_FILE)
    assert c.magic == VersionedMagic.GgmfV1 and not c.magic.align32()
    t = c.tensors["h"]
    assert (t.dtype(), t.shape) == (1, (3,))
    assert t.data().view(np.float16).tolist() == [0.0, 1.0, 2.0]


def test_every_ggjt_version_and_errors():
    for v, want in ((1, VersionedMagic.GgjtV1), (2, VersionedMagic.GgjtV2), (3, VersionedMagic.GgjtV3)):
        assert GF.read_bytes(b"tjgg" + u32(v) + GGJT_FILE[8:]).magic == want
    with pytest.raises(GgmlFileError, match="unknown magic 46554747"):
        GF.read_bytes(b"GGUF" + GGJT_FILE[4:])
    with pytest.raises(GgmlFileError, match="unsupported magic/version ggjt/4"):
        GF.read_bytes(b"tjgg" + u32(4) + GGJT_FILE[8:])
    with pytest.raises(GgmlFileError, match="unsupported magic/version ggmf/2"):
        GF.read_bytes(b"fmgg" + u32(2) + GGMF_FILE[8:])
    with pytest.raises(GgmlFileError, match="unsupported magic/version ggla/1"):     # known magic, no reader for it
        GF.read_bytes(b"algg" + u32(1) + GGJT_FILE[8:])
    with pytest.raises(GgmlFileError, match="unexpected end of file"):
        GF.read_bytes(GGJT_FILE[:-3])
    with pytest.raises(GgmlFileError, match="unknown dtype for tensor 5"):
        GF.read_bytes(GGJT_HEAD + u32(1, 1, 5) + u32(32) + b"x" + bytes(64))
    with pytest.raises(GgmlFileError, match="Error creating tensor x: .*not divisible by the block size"):
        GF.read_bytes(GGJT_HEAD + u32(1, 1, 8) + u32(33) + b"x" + bytes(64))
    # a name that is not UTF-8 is decoded lossily, as String::from_utf8_lossy does
    c = GF.read_bytes(b"lmgg" + HPARAMS + VOCAB + u32(1, 2, 0) + u32(1) + b"\xff!" + f32(2.0))
    assert list(c.tensors) == ["�!"]


def test_zero_tokens_and_no_tensors():
    c = GF.read_bytes(b"lmgg" + u32(0, 1, 2, 3, 4, 5, 6))
    assert c.vocab.token_score_pairs == [] and c.tensors == {} and c.hparams.ftype == 6


@pytest.mark.gpu
def test_load_ggml_to_device_and_matmul(tmp_path):
    torch = pytest.importorskip("torch")
    from oracle import cpu_oracle as orc
    from candle_amd.quantized import QMatMul
    rng = np.random.default_rng(3)
    n, k = 48, 512
    w = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    blocks = orc.quantize(orc.Q4K, w)
    norm = rng.standard_normal(k).astype(np.float32)
    head = b"tjgg" + u32(3) + u32(1, k, 256, 8, 1, 64, 15) + u32(2) + b"hi" + f32(0.0)
    body = head + u32(2, 6, 12) + u32(k, n) + b"blk.wq"
    body += bytes((32 - len(body) % 32) % 32) + blocks.tobytes()
    body += u32(1, 4, 0) + u32(k) + b"norm"
    body += bytes((32 - len(body) % 32) % 32) + norm.tobytes()
    path = tmp_path / "model.ggml"
    path.write_bytes(body)
    tensors, hparams, vocab = GF.load_ggml(str(path))
    assert hparams["n_embd"] == k and hparams["ftype"] == 15 and vocab == ["hi"]
    assert tensors["blk.wq"].shape == (n, k) and tensors["blk.wq"].ggml_dtype == "Q4K"
    assert np.array_equal(tensors["blk.wq"].data(), blocks)
    assert torch.equal(tensors["norm"].cpu(), torch.from_numpy(norm))
    x = rng.standard_normal((3, k)).astype(np.float32)
    got = QMatMul.from_qtensor(tensors["blk.wq"]).forward(torch.from_numpy(x).cuda()).cpu().numpy()
    want = orc.matmul(orc.Q4K, x, blocks, n)
    assert np.linalg.norm(got - want) <= 1e-4 * np.linalg.norm(want)
