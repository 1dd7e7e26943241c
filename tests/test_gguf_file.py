"""GGUF reader / writer (candle_amd/gguf_file.py, after gguf_file.rs) and the file -> device loader.

The reference holds no GGUF fixture and no test of this module, so the format is pinned here by files
spelled out byte by byte from the published GGUF layout (little-endian; header = magic, version,
tensor count, key/value count; strings length-prefixed; tensor dims innermost first; tensor data at
the next multiple of `general.alignment`), not produced by the writer under test.
"""
import io
import os

import numpy as np
import pytest

from candle_amd import gguf_file as G
from candle_amd.gguf_file import Content, GgufError, HostQTensor, Value, ValueType


def u32(v):
    return int(v).to_bytes(4, "little")


def u64(v):
    return int(v).to_bytes(8, "little")


Q8_0_ROWS = bytes(range(204))          # 3 rows x 2 blocks x 34 bytes of arbitrary block bytes

# Version 3: u64 counts and lengths, alignment 64 from the metadata.
V3_FILE = (
    b"GGUF" + u32(3) + u64(1) + u64(2)
    + u64(17) + b"general.alignment" + u32(4) + u32(64)               # u32 value
    + u64(4) + b"name" + u32(8) + u64(3) + b"abc"                     # string value
    + u64(1) + b"w" + u32(2) + u64(64) + u64(3) + u32(8) + u64(0)     # Q8_0, dims stored as [64, 3]
)
assert len(V3_FILE) == 125
V3_FILE += bytes(3) + Q8_0_ROWS                                       # data starts at 128

# Version 1: u32 counts, string lengths, array lengths and dims; default alignment 32.
V1_FILE = (
    b"GGUF" + u32(1) + u32(2) + u32(3)
    + u32(2) + b"k\x00" + u32(5) + (-7).to_bytes(4, "little", signed=True)          # key with a trailing NUL
    + u32(1) + b"a" + u32(9) + u32(2) + u32(3) + (513).to_bytes(2, "little") * 3    # array of three u16
    + u32(1) + b"b" + u32(7) + b"\x01"                                              # bool
    + u32(2) + b"t0" + u32(1) + u32(4) + u32(0) + u64(0)                            # F32 [4]
    + u32(2) + b"t1" + u32(3) + u32(2) + u32(1) + u32(5) + u32(1) + u64(32)         # F16, dims [2,1,5]
)
assert len(V1_FILE) == 123
V1_T0 = np.array([1.0, -2.0, 0.5, 3.0], np.float32)
V1_T1 = np.arange(10, dtype=np.float16)
V1_FILE += bytes(5) + V1_T0.tobytes() + bytes(16) + V1_T1.tobytes()                # data starts at 128


def test_read_v3_literal():
    f = io.BytesIO(V3_FILE)
    c = Content.read(f)
    assert c.version == 3 and c.tensor_data_offset == 128
    assert c.metadata == {"general.alignment": Value(ValueType.U32, 64), "name": Value(ValueType.STRING, "abc")}
    info = c.tensor_infos["w"]
    assert (info.ggml_dtype, info.shape, info.offset) == (8, (3, 64), 0)      # dims reversed on read
    t = c.tensor_host(f, "w")
    assert t.ggml_dtype == "Q8_0" and t.shape == (3, 64) and t.data().tobytes() == Q8_0_ROWS
    with pytest.raises(GgufError, match="cannot find tensor info for nope"):
        c.tensor_host(f, "nope")


def test_read_v1_literal():
    f = io.BytesIO(V1_FILE)
    c = Content.read(f)
    assert c.version == 1 and c.tensor_data_offset == 128
    assert c.metadata["k"] == Value(ValueType.I32, -7)                        # trailing NUL dropped
    assert c.metadata["a"].to_python() == [513, 513, 513]
    assert c.metadata["a"].v[0].type == ValueType.U16
    assert c.metadata["b"] == Value(ValueType.BOOL, True)
    assert c.tensor_infos["t1"].shape == (5, 1, 2) and c.tensor_infos["t1"].offset == 32
    assert np.array_equal(c.tensor_host(f, "t0").data().view(np.float32), V1_T0)
    assert np.array_equal(c.tensor_host(f, "t1").data().view(np.float16), V1_T1)


def test_write_literal():
    """The writer's bytes for one u8 key and one F32 [2,3] tensor: version 2, dims innermost first,
    header padded to 32, tensor padded to 32."""
    data = np.arange(6, dtype=np.float32)
    out = io.BytesIO()
    G.write(out, [("a", Value(ValueType.U8, 7))], [("t", HostQTensor(0, data, (2, 3)))])
    want = (b"GGUF" + u32(2) + u64(1) + u64(1)
            + u64(1) + b"a" + u32(0) + b"\x07"
            + u64(1) + b"t" + u32(2) + u64(3) + u64(2) + u32(0) + u64(0))
    assert len(want) == 79
    want += bytes(17) + data.tobytes() + bytes(8)
    assert out.getvalue() == want


def test_write_offsets_and_padding():
    """Several tensors whose sizes are not multiples of 32: each starts on a 32-byte boundary."""
    rng = np.random.default_rng(0)
    ts = [("q4", HostQTensor(2, rng.integers(0, 256, 18 * 3, dtype=np.uint8), (3, 32))),       # 54 B
          ("q6", HostQTensor(14, rng.integers(0, 256, 210, dtype=np.uint8), (1, 256))),        # 210 B
          ("f16", HostQTensor(1, rng.integers(0, 256, 14, dtype=np.uint8), (7,))),             # 14 B
          ("q4k", HostQTensor(12, rng.integers(0, 256, 288, dtype=np.uint8), (2, 256)))]       # 288 B
    out = io.BytesIO()
    G.write(out, [], ts)
    f = io.BytesIO(out.getvalue())
    c = Content.read(f)
    assert c.version == 2 and c.tensor_data_offset % 32 == 0
    assert [c.tensor_infos[n].offset for n, _ in ts] == [0, 64, 288, 320]
    assert len(out.getvalue()) == c.tensor_data_offset + 320 + 288
    for name, t in ts:
        back = c.tensor_host(f, name)
        assert back.shape == t.shape and back.dtype() == t.dtype()
        assert np.array_equal(back.data(), t.data())


def test_metadata_roundtrip_all_types():
    md = [("u8", Value(ValueType.U8, 255)), ("i8", Value(ValueType.I8, -128)),
          ("u16", Value(ValueType.U16, 65535)), ("i16", Value(ValueType.I16, -32768)),
          ("u32", Value(ValueType.U32, 2**32 - 1)), ("i32", Value(ValueType.I32, -2**31)),
          ("u64", Value(ValueType.U64, 2**64 - 1)), ("i64", Value(ValueType.I64, -2**63)),
          ("f32", Value(ValueType.F32, 0.5)), ("f64", Value(ValueType.F64, 1e300)),
          ("t", Value(ValueType.BOOL, True)), ("f", Value(ValueType.BOOL, False)),
          ("s", Value(ValueType.STRING, "tokenizer é中")),
          ("empty", Value(ValueType.ARRAY, [])),
          ("strs", Value(ValueType.ARRAY, [Value(ValueType.STRING, s) for s in ("<s>", "</s>", "")])),
          ("nested", Value(ValueType.ARRAY, [Value(ValueType.ARRAY, [Value(ValueType.F32, 1.5)]),
                                             Value(ValueType.ARRAY, [Value(ValueType.F32, -2.0)] * 2)]))]
    out = io.BytesIO()
    G.write(out, md, [])
    c = G.read_bytes(out.getvalue())
    assert list(c.metadata) == [k for k, _ in md] and c.tensor_infos == {}
    for k, v in md:
        assert c.metadata[k] == v, k
    assert len(out.getvalue()) % 32 == 0


def test_value_infer_order():
    """Plain Python values take the first integer type that holds them (u8, i8, u16, i16, u32, i32, u64,
    i64), floats f32 (candle-pyo3/src/lib.rs:1394-1424)."""
    cases = [(0, ValueType.U8), (255, ValueType.U8), (-1, ValueType.I8), (256, ValueType.U16),
             (-129, ValueType.I16), (65536, ValueType.U32), (-32769, ValueType.I32), (2**32, ValueType.U64),
             (-2**31 - 1, ValueType.I64), (1.25, ValueType.F32), ("x", ValueType.STRING), (True, ValueType.BOOL)]
    for obj, t in cases:
        assert Value.infer(obj).type == t, obj
    arr = Value.infer([1, 2, 3])
    assert arr.type == ValueType.ARRAY and arr.to_python() == [1, 2, 3]
    with pytest.raises(GgufError):
        Value.infer(2**64)
    with pytest.raises(GgufError):
        Value.infer(object())


def test_errors():
    with pytest.raises(GgufError, match="unknown magic"):
        G.read_bytes(b"GGML" + V3_FILE[4:])
    with pytest.raises(GgufError, match="unsupported magic/version"):
        G.read_bytes(b"GGUF" + u32(4) + V3_FILE[8:])
    with pytest.raises(GgufError, match="failed to fill whole buffer"):
        G.read_bytes(V3_FILE[:60])
    bad_type = b"GGUF" + u32(3) + u64(0) + u64(1) + u64(1) + b"k" + u32(13) + u32(0)
    with pytest.raises(GgufError, match="unrecognized value-type"):
        G.read_bytes(bad_type)
    bad_bool = b"GGUF" + u32(3) + u64(0) + u64(1) + u64(1) + b"k" + u32(7) + b"\x02"
    with pytest.raises(GgufError, match="unexpected bool value 2"):
        G.read_bytes(bad_bool)
    bad_dtype = b"GGUF" + u32(3) + u64(1) + u64(0) + u64(1) + b"w" + u32(1) + u64(32) + u32(5) + u64(0)
    with pytest.raises(GgufError, match="unknown dtype for tensor 5"):
        G.read_bytes(bad_dtype)
    # 48 elements are not whole Q8_0 blocks: the header parses, reading the tensor fails.
    ragged = b"GGUF" + u32(3) + u64(1) + u64(0) + u64(1) + b"w" + u32(1) + u64(48) + u32(8) + u64(0) + bytes(64)
    f = io.BytesIO(ragged)
    c = Content.read(f)
    with pytest.raises(GgufError, match="48 is not divisible by the block size 32"):
        c.tensor_host(f, "w")
    # the tensor bytes run past the end of the file
    f = io.BytesIO(V3_FILE[:-1])
    with pytest.raises(GgufError, match="failed to fill whole buffer"):
        Content.read(f).tensor_host(f, "w")
    with pytest.raises(GgufError, match="multiple value-types"):
        G.write(io.BytesIO(), [("k", Value(ValueType.ARRAY, [Value(ValueType.U8, 1), Value(ValueType.I8, 1)]))], [])
    with pytest.raises(GgufError, match="bytes given"):
        HostQTensor(12, bytes(100), (1, 256))
    with pytest.raises(ValueError, match="keys must be strings"):
        G.save_gguf(os.devnull, {1: None}, {})


def test_alignment_key_kinds():
    """Only unsigned / non-negative signed 8-32 bit integers set the alignment (gguf_file.rs:452-460);
    anything else leaves the default 32."""
    def offset_with(val):
        out = io.BytesIO()
        G.write(out, [("general.alignment", val)], [])
        return G.read_bytes(out.getvalue() + bytes(512)).tensor_data_offset
    base = offset_with(Value(ValueType.U64, 256))            # u64 is ignored: default alignment
    assert base % 32 == 0 and base < 96
    assert offset_with(Value(ValueType.U16, 256)) == 256
    assert offset_with(Value(ValueType.I32, 128)) == 128
    assert offset_with(Value(ValueType.I8, -1)) == base
    assert offset_with(Value(ValueType.STRING, "64")) % 32 == 0


def test_type_table_matches_library():
    """The parser's own size table against the device library's `cq_block_size` / `cq_type_size`."""
    from candle_amd import qhip
    L = qhip.load()
    for t in (2, 3, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15):
        assert G.ggml_block_size(t) == L.cq_block_size(t), t
        assert G.ggml_type_size(t) == L.cq_type_size(t), t


def _model_file(tmp_path, rng):
    """A llama-shaped miniature: one tensor of every weight type, F32 norms, an F16 tensor."""
    from oracle import cpu_oracle as O
    k, n = 512, 96
    host = {}
    for name, dt in (("blk.0.attn_q.weight", 12), ("blk.0.ffn_down.weight", 14),
                     ("blk.0.attn_k.weight", 2), ("token_embd.weight", 8),
                     ("blk.0.attn_v.weight", 6), ("blk.0.ffn_up.weight", 11), ("blk.0.ffn_gate.weight", 13),
                     ("blk.0.attn_output.weight", 3), ("output.weight", 7), ("blk.1.ffn_up.weight", 10),
                     ("blk.1.ffn_down.weight", 15)):
        w = (rng.standard_normal((n, k)) * 0.1).astype(np.float32)
        host[name] = HostQTensor(dt, O.quantize(dt, w), (n, k))
    host["blk.0.attn_norm.weight"] = HostQTensor(0, rng.standard_normal(k).astype(np.float32), (k,))
    host["rope_freqs.weight"] = HostQTensor(1, rng.standard_normal(64).astype(np.float16), (64,))
    md = {"general.architecture": "llama", "llama.block_count": 1, "llama.attention.head_count": 8,
          "llama.rope.freq_base": 10000.0, "tokenizer.ggml.tokens": ["<unk>", "<s>", "</s>"],
          "llama.attention.layer_norm_rms_epsilon": Value(ValueType.F32, 1e-5)}
    path = str(tmp_path / "tiny.gguf")
    G.save_gguf(path, host, md)
    return path, host, md


@pytest.mark.gpu
def test_load_gguf_to_device_and_matmul(tmp_path):
    """File -> device: every tensor's blocks come back bit-exact from the device layout, the matmul of a
    loaded tensor equals the one of a directly uploaded tensor bit for bit and the oracle within the
    path's tolerance (rel-L2 <= 1e-4), and saving the device tensors reproduces the file byte for byte."""
    import torch
    from oracle import cpu_oracle as O
    from candle_amd.quantized import QTensor
    rng = np.random.default_rng(5)
    path, host, md = _model_file(tmp_path, rng)
    tensors, metadata = G.load_gguf(path)
    assert metadata["general.architecture"] == "llama" and metadata["llama.block_count"] == 1
    assert metadata["tokenizer.ggml.tokens"] == ["<unk>", "<s>", "</s>"]
    assert metadata["llama.rope.freq_base"] == 10000.0
    assert set(tensors) == set(host)
    xs = rng.standard_normal((5, 512)).astype(np.float32)
    xd = torch.from_numpy(xs).cuda()
    for name, h in host.items():
        t = tensors[name]
        if h.dtype() in (0, 1):
            assert t.is_cuda and tuple(t.shape) == h.shape
            assert t.cpu().numpy().tobytes() == h.data().tobytes()
            continue
        assert isinstance(t, QTensor) and t.shape == h.shape and int(t.dtype()) == h.dtype()
        assert np.array_equal(t.data(), h.data()), name
        y = t.matmul_t(xd)
        direct = QTensor.from_ggml(h.dtype(), h.data(), h.shape).matmul_t(xd)
        assert torch.equal(y, direct), name
        want = O.matmul(h.dtype(), xs, h.data(), h.shape[0])
        got = y.cpu().numpy()
        assert np.linalg.norm(got - want) <= 1e-4 * np.linalg.norm(want), name
    again = str(tmp_path / "again.gguf")
    G.save_gguf(again, {name: tensors[name] if host[name].dtype() > 1 else host[name] for name in host}, md)
    with open(path, "rb") as a, open(again, "rb") as b:
        assert a.read() == b.read()


@pytest.mark.gpu
def test_load_gguf_rejects_types_without_device_kernels(tmp_path):
    path = str(tmp_path / "q8_1.gguf")
    G.save_gguf(path, {"w": HostQTensor(9, bytes(36), (1, 32))}, {})   # an activation format, not a weight type
    with pytest.raises(GgufError, match="Q8_1 tensors are not supported on the device"):
        G.load_gguf(path)
