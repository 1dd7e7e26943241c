"""The storage half of the boundary as the reference shapes it: storage created from an element count
(`QCudaStorage::zeros(device, el_count, dtype)`, cuda.rs:368-381; `load_quantized(device, data)`, cuda.rs:591-612),
quantized into (`QCudaStorage::quantize`, cuda.rs:448-472), and the shape handed over at the call
(`fwd(&self, self_shape, ..)`, cuda.rs:478-499).  Plus the aliasing rule of the matmul calls."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from oracle import cpu_oracle as orc  # noqa: E402  (checker only)


@pytest.fixture(scope="module")
def qh():
    from candle_amd import qhip
    qhip.load()
    assert qhip.load().cq_device_count() >= 1, "no HIP device visible"
    return qhip


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_flat_storage_runs_the_reference_goldens(qh, goldens, seeded_inputs):
    """G1/G2 (quantized_tests.rs:49-64, :109-129) and G7 (:1051-1151) with storage that never saw a shape."""
    m, k, n = 3, 64, 4
    lhs = np.arange(m * k, dtype=np.float32).reshape(m, k)
    rhs = np.arange(k * n, dtype=np.float32).reshape(n, k)
    # load_quantized: blocks only
    qw = qh.QWeight.from_ggml_flat(orc.Q4_0, orc.quantize(orc.Q4_0, rhs))
    assert qw.elem_count == n * k and qw.shape == (n * k // 32, 32)
    got = qh.qmatmul_shaped(qw, (n, k), dev(lhs)).cpu().numpy()
    assert np.round(got).ravel().tolist() == goldens["q4_0_matmul_m3_k64_n4"]["rounded"]
    # zeros(el_count) + quantize(src)
    lhs = (np.arange(m * k, dtype=np.float32) - np.float32(m * k) / 2).reshape(m, k)
    rhs = (np.arange(k * n, dtype=np.float32) - np.float32(k * n) / np.float32(3.0)).reshape(n, k)
    qw = qh.QWeight.zeros_flat(orc.Q4_0, n * k).quantize_(dev(rhs))
    got = qh.qmatmul_shaped(qw, (n, k), dev(lhs)).cpu().numpy()
    assert np.round(got).ravel().tolist() == goldens["q4_0_matmul_neg_m3_k64_n4"]["rounded"]
    assert np.array_equal(qw.to_ggml(), orc.quantize(orc.Q4_0, rhs))
    g = goldens["seeded_matmul_m11_k512_n21"]
    lhs, rhs = seeded_inputs
    for name, dt in (("q4k", orc.Q4K), ("q5k", orc.Q5K), ("q6k", orc.Q6K), ("q8k", orc.Q8K)):
        qw = qh.QWeight.zeros_flat(dt, 21 * 512).quantize_(dev(rhs))
        out = qh.qmatmul_shaped(qw, (21, 512), dev(lhs)).cpu().numpy().ravel()
        spot = [float(np.round(np.float32(1000.0) * out[i]) / np.float32(1000.0)) for i in g["flat_indices"]]
        assert spot == [float(np.float32(v)) for v in g[name]], (name, spot)
        # the same through the shape-less entry point once the shape is fixed (QTensor::new)
        out2 = qh.qmatmul(qw.set_shape(21, 512), dev(lhs)).cpu().numpy().ravel()
        assert np.array_equal(out, out2)


@pytest.mark.parametrize("dt", [orc.Q4_0, orc.Q4_1, orc.Q5_0, orc.Q5_1, orc.Q8_0, orc.Q2K, orc.Q3K, orc.Q4K, orc.Q5K, orc.Q6K])
@pytest.mark.parametrize("m", [1, 3, 16, 80])
def test_shape_at_call_equals_shape_at_creation(qh, dt, m):
    """Every kernel family (one-launch decode, split-K, tile) reads flat storage like shaped storage, and one
    storage serves two readings of its blocks."""
    rng = np.random.default_rng(100 + m)
    n, k = 192, 1024
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    blocks = orc.quantize(dt, w)
    flat = qh.QWeight.from_ggml_flat(dt, blocks)
    shaped = qh.QWeight.from_ggml(dt, blocks, n, k)
    x = dev(rng.standard_normal((m, k)).astype(np.float32))
    a = qh.qmatmul_shaped(flat, (n, k), x).cpu().numpy()
    b = qh.qmatmul(shaped, x).cpu().numpy()
    assert np.array_equal(a, b)
    ref = orc.matmul(dt, x.cpu().numpy(), blocks, n)
    assert np.linalg.norm(a - ref) <= 1e-4 * np.linalg.norm(ref)
    # the same blocks read as [2n, k/2]: rows of the original split in two
    x2 = dev(rng.standard_normal((m, k // 2)).astype(np.float32))
    a2 = qh.qmatmul_shaped(flat, (2 * n, k // 2), x2).cpu().numpy()
    ref2 = orc.matmul(dt, x2.cpu().numpy(), blocks, 2 * n)
    assert np.linalg.norm(a2 - ref2) <= 1e-4 * np.linalg.norm(ref2)
    assert np.array_equal(flat.dequantize().cpu().numpy().ravel(), orc.dequantize(dt, blocks))


@pytest.mark.parametrize("dt", [orc.Q4_1, orc.Q5_0, orc.Q5_1])
@pytest.mark.parametrize("m", [1, 3, 40])
def test_odd_block_counts_are_refused_like_the_reference(qh, dt, m):
    """vec_dot of Q4_1, Q5_0 and Q5_1 bails out on rows with an odd number of blocks (k_quants.rs:273, 363, 469), and
    with it the matmul; weights of such shapes can still be created, read back and dequantized.  Q4_0 and Q8_0 have
    no such rule."""
    rng = np.random.default_rng(7 * int(dt) + m)
    n, k = 16, 96
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    blocks = orc.quantize(dt, w)
    q = qh.QWeight.from_ggml(dt, blocks, n, k)
    assert np.array_equal(q.to_ggml(), blocks)
    assert np.array_equal(q.dequantize().cpu().numpy(), orc.dequantize(dt, blocks).reshape(n, k))
    with pytest.raises(ValueError):
        orc.matmul(dt, x, blocks, n)
    for flags in (0, qh.FLAG_STAGED_ACT, qh.FLAG_FORCE_MATVEC):
        with pytest.raises(qh.QHipError, match="nb is not divisible by 2"):
            qh.qmatmul(q, dev(x), flags)
    with pytest.raises(qh.QHipError, match="nb is not divisible by 2"):
        qh.qmatmul_multi([q, q], dev(x))
    assert qh.qmatmul(q, dev(x[:0])).shape == (0, n)          # no rows: no vec_dot, no error
    for ok in (orc.Q4_0, orc.Q8_0):
        b = orc.quantize(ok, w)
        got = qh.qmatmul(qh.QWeight.from_ggml(ok, b, n, k), dev(x)).cpu().numpy()
        ref = orc.matmul(ok, x, b, n)
        assert np.linalg.norm(got - ref) <= 1e-4 * np.linalg.norm(ref)


@pytest.mark.parametrize("dt", [orc.Q4_1, orc.Q5_0, orc.Q5_1, orc.Q2K, orc.Q3K])
def test_types_held_in_another_types_planes(qh, dt):
    """Q5_0 lives in Q8_0 planes, Q3K in Q6K planes, Q4_1 and Q5_1 in Q8_0 planes plus a plane of minima: the caller sees the type it created (dtype, GGML byte size,
    all-zero blocks from `zeros`, its own bytes back), whatever the device holds; the prefill tile kernel and the
    Q8K-formulation integers follow the oracle's Q5_0 / Q3K code."""
    rng = np.random.default_rng(int(dt))
    n, k = 64, 1024
    nbytes = n * k // orc.BLOCK_SIZE[dt] * orc.TYPE_SIZE[dt]
    z = qh.QWeight.zeros(dt, n, k)
    assert z.dtype == dt and z.size_in_bytes == nbytes
    assert not z.to_ggml().any()
    assert not z.dequantize().cpu().numpy().any()
    flat = qh.QWeight.zeros_flat(dt, n * k)
    assert flat.dtype == dt and not flat.to_ggml().any()
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    q = z.quantize_(dev(w))                                   # QTensor::quantize into existing storage
    blocks = orc.quantize(dt, w)
    assert np.array_equal(q.to_ggml(), blocks)
    x = rng.standard_normal((70, k)).astype(np.float32)      # more than 32 rows: the tile kernels
    got = qh.qmatmul(q, dev(x)).cpu().numpy()
    ref = orc.matmul(dt, x, blocks, n)
    assert np.linalg.norm(got - ref) <= 1e-4 * np.linalg.norm(ref)
    with pytest.raises(qh.QHipError, match="Q8_1 activations are for Q4K and Q6K"):
        qh.qmatmul(q, dev(x), flags=qh.FLAG_ACT_Q8_1)
    if dt in (orc.Q4_1, orc.Q5_1, orc.Q2K):
        # the offset term (almost) alone: Q4_1 / Q5_1 store a constant block as d = 0, m = c; Q2K a block of -0.375
        # with a few -0.25 as minima of 0.375 and small scales
        const = np.full((n, k), 0.375, np.float32)
        if dt == orc.Q2K:
            const = -const
            const[:, ::16] = -0.25
        qc = qh.QWeight.from_ggml(dt, orc.quantize(dt, const), n, k)
        got_c = qh.qmatmul(qc, dev(x[:3])).cpu().numpy()
        ref_c = orc.matmul(dt, x[:3], orc.quantize(dt, const), n)
        assert np.abs(got_c - ref_c).max() <= 1e-4 * np.abs(ref_c).max()
        assert np.abs(ref_c).max() > 1.0     # the term is not negligible here


@pytest.mark.parametrize("m,k,n", [(1, 256, 7), (3, 4096, 64), (40, 1024, 33), (2, 11008, 5)])
def test_q8k_as_a_weight_type(qh, m, k, n):
    """BlockQ8K as GgmlType (k_quants.rs:1749-1839; the reference's tests quantize to it and multiply by it,
    quantized_tests.rs:672-717, :1124-1150): bytes back (any pattern, all-zero blocks from `zeros`), dequantize and the
    device quantizer bit-exact, the product against the oracle, rows independent of their neighbours."""
    rng = np.random.default_rng(m * k + n)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    w[0] = 0.0
    blocks = orc.quantize(orc.Q8K, w)
    qw = qh.QWeight.from_ggml(orc.Q8K, blocks, n, k)
    assert qw.dtype == orc.Q8K and qw.size_in_bytes == blocks.size and np.array_equal(qw.to_ggml(), blocks)
    rnd = rng.integers(0, 256, size=blocks.size, dtype=np.uint8)
    assert np.array_equal(qh.QWeight.from_ggml(orc.Q8K, rnd, n, k).to_ggml(), rnd)
    assert not qh.QWeight.zeros(orc.Q8K, n, k).to_ggml().any()
    want = orc.dequantize(orc.Q8K, blocks).reshape(n, k)
    assert np.array_equal(qw.dequantize().cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert np.array_equal(qw.dequantize_f16().cpu().numpy().view(np.uint16), want.astype(np.float16).view(np.uint16))
    assert np.array_equal(qh.QWeight.zeros(orc.Q8K, n, k).quantize_(dev(w)).to_ggml(), blocks)
    x = rng.standard_normal((m, k)).astype(np.float32)
    got = qh.qmatmul(qw, dev(x)).cpu().numpy()
    ref = orc.matmul(orc.Q8K, x, blocks, n)
    for r in range(m):
        assert np.linalg.norm(got[r] - ref[r]) <= 1e-4 * max(np.linalg.norm(ref[r]), 1e-30)
    if m > 1:
        assert np.array_equal(qh.qmatmul(qw, dev(x[1:2])).cpu().numpy()[0], got[1])
    with pytest.raises(qh.QHipError, match="dot-product kernel only"):
        qh.qmatmul(qw, dev(x), flags=qh.FLAG_FORCE_GEMM)


def test_shape_errors(qh):
    L = qh.load()
    h = C.c_void_p()
    assert L.cq_weight_zeros_flat(0, orc.Q4K, 300, C.byref(h)) == -1          # not whole blocks
    assert b"block size" in L.cq_last_error()
    assert L.cq_weight_create_flat(0, orc.Q4K, None, 145, C.byref(h)) == -1  # not whole blocks of bytes
    assert L.cq_weight_zeros_flat(0, 1, 256, C.byref(h)) == -2               # F16: not a quantized storage of this library
    qw = qh.QWeight.zeros_flat(orc.Q4K, 4 * 512)
    with pytest.raises(qh.QHipError, match="does not cover"):
        qw.set_shape(3, 512)
    with pytest.raises(qh.QHipError, match="divisible by block size"):
        qw.set_shape(16, 128)
    with pytest.raises(qh.QHipError, match="does not cover"):
        qh.qmatmul_shaped(qw, (8, 512), torch.zeros((1, 512), device="cuda"))
    assert L.cq_workspace_bytes_shaped(qw.handle, 8, 512, 1, 0) == 0
    assert L.cq_workspace_bytes_shaped(qw.handle, 4, 512, 1, 0) == L.cq_workspace_bytes(qw.set_shape(4, 512).handle, 1, 0)


@pytest.mark.parametrize("dt", [orc.Q4_0, orc.Q8_0, orc.Q4K, orc.Q6K])
@pytest.mark.parametrize("m", [1, 3, 4])
def test_in_place_call_equals_out_of_place(qh, dt, m):
    """n == k called with out = x: the one-launch kernels would read activations that other workgroups have
    already overwritten, so such a call takes the quantizer launch first; same bits as out of place."""
    rng = np.random.default_rng(7 + m)
    n = k = 2048
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    qw = qh.QWeight.from_ggml(dt, orc.quantize(dt, w), n, k)
    x = dev(rng.standard_normal((m, k)).astype(np.float32))
    want = qh.qmatmul(qw, x).clone()
    # the two-launch path an in-place call takes, out of place: what the in-place call must equal bit for bit
    staged = qh.qmatmul(qw, x, flags=qh.FLAG_STAGED_ACT).clone()
    assert (staged - want).norm() <= 1e-5 * want.norm()
    if m == 1:
        assert torch.equal(staged, want)
    for _ in range(3):
        buf = x.clone()
        got = qh.qmatmul(qw, buf, out=buf)
        assert got.data_ptr() == buf.data_ptr()
        assert torch.equal(got, staged)
    # partial overlap: y starts in the middle of x
    big = torch.zeros(2 * m * k, device="cuda")
    big[: m * k] = x.ravel()
    xin = big[: m * k].view(m, k)
    yout = big[m * k // 2: m * k // 2 + m * n].view(m, n)
    assert torch.equal(qh.qmatmul(qw, xin, out=yout), staged)


def test_in_place_fused_steps(qh):
    """The same with a fused step whose second operand is overwritten (silu * mul: aux shaped like x)."""
    rng = np.random.default_rng(3)
    n = k = 2048
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    qw = qh.QWeight.from_ggml(orc.Q6K, orc.quantize(orc.Q6K, w), n, k)
    gate = dev(rng.standard_normal((1, k)).astype(np.float32))
    up = dev(rng.standard_normal((1, k)).astype(np.float32))
    want = qh.qmatmul(qw, gate, pre=qh.PRE_SILU_MUL, aux=up).clone()
    buf = up.clone()
    assert torch.equal(qh.qmatmul(qw, gate, out=buf, pre=qh.PRE_SILU_MUL, aux=buf), want)
    alpha = dev((1 + 0.1 * rng.standard_normal(k)).astype(np.float32))
    want = qh.qmatmul(qw, gate, pre=qh.PRE_RMS_NORM, aux=alpha, eps=1e-5).clone()
    buf = alpha.clone().view(1, k)
    got = qh.qmatmul(qw, gate, out=buf, pre=qh.PRE_RMS_NORM, aux=buf.view(k), eps=1e-5)
    # (one launch scales the row results, the staged path scales the block scales: equal to rounding)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)


def test_multi_refuses_in_place(qh):
    rng = np.random.default_rng(5)
    n = k = 1024
    ws = [qh.QWeight.from_ggml(orc.Q4K, orc.quantize(orc.Q4K, (rng.standard_normal((n, k)) * 0.02).astype(np.float32)), n, k)
          for _ in range(2)]
    x = dev(rng.standard_normal((1, k)).astype(np.float32))
    L = qh.load()
    vp = C.c_void_p
    other = torch.empty((1, n), device="cuda")
    handles = (vp * 2)(*[w.handle for w in ws])
    ys = (vp * 2)(other.data_ptr(), x.data_ptr())
    wsb = torch.empty(L.cq_workspace_bytes(ws[0].handle, 1, 0), dtype=torch.uint8, device="cuda")
    rc = L.cq_qmatmul_multi(handles, 2, 0, vp(x.data_ptr()), None, 0.0, 1, ys, 0, vp(wsb.data_ptr()), wsb.numel(), None)
    assert rc == -1 and b"in place" in L.cq_last_error()


@pytest.mark.parametrize("dt,k", [(orc.Q8_0, 53248), (orc.Q4K, 65536), (orc.Q6K, 131072)])
def test_long_rows(qh, dt, k):
    """Rows whose quantized image needs more than 64 KiB of LDS (e.g. a 53248-wide Q8_0 down projection): the
    dot-product kernels take up to 160 KiB; beyond that the call is refused with a message naming the limit."""
    rng = np.random.default_rng(k)
    n = 24
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    for m in (1, 2):
        x = rng.standard_normal((m, k)).astype(np.float32)
        got = qh.qmatmul(qw, dev(x)).cpu().numpy()
        ref = orc.matmul(dt, x, blocks, n)
        assert np.linalg.norm(got - ref) <= 1e-4 * np.linalg.norm(ref)


@pytest.mark.parametrize("dt", [orc.Q4_0, orc.Q8_0, orc.Q4K, orc.Q5K, orc.Q6K, orc.Q2K, orc.Q5_1])
@pytest.mark.parametrize("m", [1, 3, 6])
def test_rows_beyond_the_lds(qh, dt, m):
    """k_quants::matmul (k_quants.rs:1842-1883) has no limit on the row length.  Rows whose quantized image exceeds the
    160 KiB of LDS (K = 262 144 here, and a K that is not a whole number of chunks) are walked in chunks by the
    dot-product kernel; one, several and more than four activation rows against the oracle."""
    for k, n in ((262144, 24), (163840 + 2048, 9)):
        rng = np.random.default_rng(int(dt) * 10 + m + k)
        w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
        x = rng.standard_normal((m, k)).astype(np.float32)
        blocks = orc.quantize(dt, w)
        qw = qh.QWeight.from_ggml(dt, blocks, n, k)
        got = qh.qmatmul(qw, dev(x)).cpu().numpy()
        ref = orc.matmul(dt, x, blocks, n)
        for r in range(m):
            nrm = np.linalg.norm(ref[r])
            assert np.linalg.norm(got[r] - ref[r]) <= 1e-4 * nrm and np.abs(got[r] - ref[r]).max() <= 1e-3 * nrm


def test_chunked_rows_equal_whole_rows_bit_for_bit(qh):
    """The chunked kernel adds a lane's units in the order of the kernel that holds the whole row in LDS: a row split as
    [n, k] = [4, 131072] (fits, whole) and the same storage read as [2, 262144] (chunked) share their first halves'
    sums only through the oracle, so this compares each against it and, for a K that fits either way, checks that
    batch invariance holds across the two kernels' launches of 4 + 2 rows."""
    k, n = 262144, 8
    rng = np.random.default_rng(77)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((6, k)).astype(np.float32)
    blocks = orc.quantize(orc.Q4K, w)
    qw = qh.QWeight.from_ggml(orc.Q4K, blocks, n, k)
    all6 = qh.qmatmul(qw, dev(x))
    for r in range(6):   # quantized_tests.rs:181-216: a row's result does not depend on the rows stacked with it
        assert torch.equal(qh.qmatmul(qw, dev(x[r:r + 1])), all6[r:r + 1])


def test_qmatmul_dense_arms(qh, monkeypatch):
    """`QMatMul::from_arc` (mod.rs:423-438): CANDLE_DEQUANTIZE_ALL / CANDLE_DEQUANTIZE_ALL_F16 select the
    dequantize-once arms; their forward is x . dequantize(W)^T (mod.rs:531-547)."""
    from candle_amd.quantized import QMatMul, QTensor
    rng = np.random.default_rng(9)
    n, k = 64, 512
    w = dev((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    x = dev(rng.standard_normal((3, k)).astype(np.float32))
    q = QTensor.quantize(w, "q4k")
    base = QMatMul.from_qtensor(q)
    assert base.arm == "QTensor"
    monkeypatch.setenv("CANDLE_DEQUANTIZE_ALL", "1")
    dense = QMatMul.from_qtensor(q)
    assert dense.arm == "Tensor" and dense.dense.dtype == torch.float32
    want = x @ q.dequantize().t()
    assert torch.allclose(dense.forward(x), want, rtol=1e-4, atol=1e-5)
    monkeypatch.setenv("CANDLE_DEQUANTIZE_ALL", "0")
    monkeypatch.setenv("CANDLE_DEQUANTIZE_ALL_F16", "yes")
    f16 = QMatMul.from_arc(q)
    assert f16.arm == "TensorF16" and f16.dense.dtype == torch.float16
    assert torch.equal(f16.dequantize_f16(), q.dequantize().half())          # quantized_tests.rs:229-234
    assert torch.allclose(f16.forward(x), want, rtol=2e-2, atol=2e-2) and f16.forward(x).dtype == torch.float32
    monkeypatch.delenv("CANDLE_DEQUANTIZE_ALL_F16")
    monkeypatch.delenv("CANDLE_DEQUANTIZE_ALL")
    assert QMatMul.from_arc(q).arm == "QTensor"
    assert torch.allclose(base.forward_via_f16(x), want, rtol=2e-2, atol=2e-2)
    # the quantized arm differs from the dense ones only by the activation quantization
    assert (base.forward(x) - want).norm() <= 2e-2 * want.norm()
