"""The host layers above the C ABI: the C++ mirror of candle's QTensor / QMatMul
(candle_amd/host/quantized.hpp) and the Python one (candle_amd/quantized.py)."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "candle_amd", "host")
SELFTEST = os.path.join(HOST, "selftest")


def _selftest_binary():
    if not os.path.exists(SELFTEST):
        from candle_amd import build as qbuild, qhip
        if not os.path.exists(qhip.LIB_PATH):
            qbuild.build(verbose=False)
        subprocess.check_call(["make", "-C", HOST], stdout=subprocess.DEVNULL)
    return SELFTEST


def test_cpp_host_layer_host_only_checks():
    """GgmlDType sizes and the shape checks' error behaviour; nothing touches a GPU."""
    r = subprocess.run([_selftest_binary(), "--host-only"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "selftest: ok" in r.stdout


def test_python_mirror_dtype_table():
    from candle_amd.quantized import GgmlDType
    assert GgmlDType.from_str("q4k") == GgmlDType.Q4K == 12
    assert (GgmlDType.Q6K.block_size(), GgmlDType.Q6K.type_size()) == (256, 210)
    assert (GgmlDType.Q4_0.block_size(), GgmlDType.Q4_0.type_size()) == (32, 18)
    assert GgmlDType.Q4K.vec_dot_type() == GgmlDType.Q8K
    assert GgmlDType.Q8_0.vec_dot_type() == GgmlDType.Q8_0
    assert GgmlDType.from_str("q5_0") == GgmlDType.Q5_0 == 6 and GgmlDType.from_str("q3k") == GgmlDType.Q3K == 11
    assert (GgmlDType.Q5_0.block_size(), GgmlDType.Q5_0.type_size(), GgmlDType.Q5_0.vec_dot_type()) == (32, 22, GgmlDType.Q8_0)
    assert (GgmlDType.Q3K.block_size(), GgmlDType.Q3K.type_size(), GgmlDType.Q3K.vec_dot_type()) == (256, 110, GgmlDType.Q8K)
    with pytest.raises(ValueError):
        GgmlDType.from_str("q9_9")


def test_python_mirror_check_shape():
    from candle_amd import qhip
    from candle_amd.quantized import _check_shape
    _check_shape((4, 64), 32)
    with pytest.raises(qhip.QHipError):
        _check_shape((), 32)
    with pytest.raises(qhip.QHipError):
        _check_shape((4, 33), 32)


@pytest.mark.gpu
def test_cpp_host_layer_reference_goldens():
    """quantized_tests.rs `quantized_matmul` / `quantized_matmul_neg` through the C++ QMatMul."""
    r = subprocess.run([_selftest_binary()], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "selftest: ok" in r.stdout


@pytest.mark.gpu
def test_python_qtensor_matmul_t_goldens(goldens):
    """The same two reference tests through the Python QTensor.matmul_t, and the getters the
    reference's Python test checks (candle-pyo3/tests/native/test_tensor.py:23-38)."""
    import torch
    from candle_amd.quantized import QMatMul, QTensor
    m, k, n = 3, 64, 4
    for key, ls, rs in (("q4_0_matmul_m3_k64_n4", 0.0, 0.0),
                        ("q4_0_matmul_neg_m3_k64_n4", np.float32(m * k) / np.float32(2.0), np.float32(k * n) / np.float32(3.0))):
        lhs = (np.arange(m * k, dtype=np.float32) - np.float32(ls)).reshape(m, k)
        rhs = (np.arange(k * n, dtype=np.float32) - np.float32(rs)).reshape(n, k)
        q = QTensor.quantize(torch.from_numpy(rhs).cuda(), "q4_0")
        assert q.ggml_dtype == "Q4_0" and q.shape == (n, k) and q.rank() == 2
        assert q.storage_size_in_bytes() == 8 * 18
        y = q.matmul_t(torch.from_numpy(lhs).cuda())
        assert tuple(y.shape) == (m, n)
        assert np.round(y.cpu().numpy()).ravel().tolist() == goldens[key]["rounded"]
        y3 = QMatMul.from_qtensor(q).forward(torch.from_numpy(lhs).cuda().reshape(1, m, k))
        assert tuple(y3.shape) == (1, m, n) and torch.equal(y3.reshape(m, n), y)


@pytest.mark.gpu
def test_python_qtensor_roundtrip_and_f16():
    import torch
    from candle_amd.quantized import QTensor
    src = torch.linspace(-0.5, 0.5, 4 * 1024, device="cuda").reshape(4, 1024)
    for name, bound in (("q4k", 0.017), ("q6k", 0.008), ("q8_0", 0.005), ("q4_0", 0.05), ("q5_0", 0.02), ("q3k", 0.03), ("q4_1", 0.04), ("q5_1", 0.02), ("q2k", 0.1), ("q8k", 0.005)):
        q = QTensor.quantize(src, name)
        back = q.dequantize()
        assert back.shape == src.shape and float((back - src).abs().max()) < bound, name
        assert torch.equal(q.dequantize_f16(), back.to(torch.float16)), name   # quantized_tests.rs:229-234


@pytest.mark.gpu
def test_python_qtensor_second_view_of_a_storage():
    """The [rows, k] a storage is read as is state of its handle: a second QTensor with another shape over the same
    storage is refused (it would re-shape the first); the same shape is fine, and a differently shaped view goes
    through the call that takes the shape with it (QCudaStorage::fwd, cuda.rs:478-499)."""
    import torch
    from candle_amd import qhip
    from candle_amd.quantized import QTensor
    src = torch.linspace(-1, 1, 8 * 512, device="cuda").reshape(8, 512)
    q = QTensor.quantize(src, "q4k")
    QTensor(q._w, (8, 512))
    with pytest.raises(qhip.QHipError):
        QTensor(q._w, (16, 256))
    x = torch.randn((3, 256), device="cuda")
    y = qhip.qmatmul_shaped(q._w, (16, 256), x)
    assert tuple(y.shape) == (3, 16) and q.shape == (8, 512)
    assert tuple(q.matmul_t(torch.randn((2, 512), device="cuda")).shape) == (2, 8)
