"""The model steps fused in front of the matmul (rms_norm, silu(x) * x2) through the C ABI.

What is checked, and against what:
  * silu * mul: the fused quantizer gives the bytes of the two-step device sequence (same
    expression, same exp), whose elementwise result is compared with the oracle to 2 ulp.
  * rms_norm: the kernels add the squares in a fixed order of their own (groups of 8, a binary
    tree per 256-element chunk, chunks in sequence) and multiply by scale = 1 / sqrt(mean + eps);
    for Q8K activations the scale goes into the block scales (or, for one row, into the result)
    instead of the elements.  The helpers below restate exactly that in numpy float32 and the
    oracle's quantizer, and the device bytes must equal it.  Against the reference's CPU code
    (squares added one by one, every element divided by the root: oracle.rms_norm) the quants may
    differ by one unit in rare positions; the matmul results stay within the f32 bars.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from oracle import cpu_oracle as orc  # noqa: E402  (checker only)
from test_gpu_parity import WEIGHT_DTYPES, check_f32, dev, make_inputs  # noqa: E402


@pytest.fixture(scope="module")
def qh():
    from candle_amd import qhip
    qhip.load()
    assert qhip.load().cq_device_count() >= 1, "no HIP device visible"
    return qhip


def staged(qh, m: int) -> int:
    """Flag for the plain call a fused call is compared with bit for bit: with two to four rows the plain
    call would take the one-launch kernel, which adds up a row's products in another order than the
    quantizer + matmul launches the fused call goes through."""
    return qh.FLAG_STAGED_ACT if 2 <= m <= 4 else 0


def canonical_scale(x: np.ndarray, eps: float) -> np.ndarray:
    """1 / sqrt(mean(x^2) + eps) per row in float32, the squares added in the kernels' order."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    m, k = x.shape
    chunks = (k + 255) // 256
    sq = np.zeros((m, chunks * 256), np.float32)
    sq[:, :k] = x * x
    s = sq.reshape(m, chunks, 32, 2, 4)
    four = ((s[..., 0] + s[..., 1]) + s[..., 2]) + s[..., 3]          # sequential sums of 4
    g = four[..., 0] + four[..., 1]                                    # groups of 8
    while g.shape[-1] > 1:                                             # j with j^1, then ^2, ...
        g = g[..., 0::2] + g[..., 1::2]
    p = g[..., 0]                                                      # [m, chunks]
    total = p[:, 0].copy()
    for c in range(1, chunks):
        total = total + p[:, c]
    return np.float32(1.0) / np.sqrt(total / np.float32(k) + np.float32(eps), dtype=np.float32)


def canonical_rms_norm(x: np.ndarray, alpha: np.ndarray, eps: float) -> np.ndarray:
    """scale * x * alpha in float32: what the kernels quantize for Q8_0 / Q8_1 activations."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    return (canonical_scale(x, eps)[:, None] * x * alpha.astype(np.float32)[None, :]).astype(np.float32)


def canonical_rms_blocks(act: int, x: np.ndarray, alpha: np.ndarray, eps: float) -> np.ndarray:
    """The activation blocks the kernels produce for rms_norm(x): for Q8K the blocks of z = x * alpha
    with their scale multiplied by the row's scale, else the blocks of scale * x * alpha."""
    if act != orc.Q8K:
        return np.concatenate([orc.quantize(act, r) for r in canonical_rms_norm(x, alpha, eps)])
    scale = canonical_scale(x, eps)
    z = (np.ascontiguousarray(x, dtype=np.float32) * alpha.astype(np.float32)[None, :]).astype(np.float32)
    rows = []
    for r in range(x.shape[0]):
        b = orc.quantize(orc.Q8K, z[r]).reshape(-1, 292).copy()
        d = b[:, :4].copy().view(np.float32)
        b[:, :4] = (d * scale[r]).astype(np.float32).view(np.uint8)
        rows.append(b.ravel())
    return np.concatenate(rows)


def act_quants(act: int, blocks: np.ndarray) -> np.ndarray:
    """The int8 quants of a run of Q8_0 / Q8_1 / Q8K blocks (k_quants.rs:78-93, :148-155)."""
    ts, lo, n = {orc.Q8_0: (34, 2, 32), orc.Q8_1: (36, 4, 32), orc.Q8K: (292, 4, 256)}[act]
    return blocks.reshape(-1, ts)[:, lo:lo + n].copy().view(np.int8)


def rms_inputs(seed, m, k):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((m, k)) * rng.uniform(0.2, 5.0, (m, 1))).astype(np.float32)
    alpha = (1.0 + 0.2 * rng.standard_normal(k)).astype(np.float32)
    return x, alpha


@pytest.mark.parametrize("act", [orc.Q8K, orc.Q8_0, orc.Q8_1])
@pytest.mark.parametrize("m,k", [(1, 256), (1, 4096), (3, 1024), (5, 11008), (2, 14336)])
def test_rms_norm_quantizer_bytes(qh, act, m, k):
    x, alpha = rms_inputs(k + m, m, k)
    eps = 1e-5
    got = qh.quantize_act(act, dev(x), qh.PRE_RMS_NORM, dev(alpha), eps).cpu().numpy()
    want = canonical_rms_blocks(act, x, alpha, eps)
    assert np.array_equal(got, want), np.flatnonzero(got != want)[:10]
    # the reference's CPU sequence: at most a unit of difference in the quants, in few places, and
    # the same dequantized values to rounding
    ref = np.concatenate([orc.quantize(act, r) for r in orc.rms_norm(x, alpha, eps)])
    dq = act_quants(act, got).astype(np.int32) - act_quants(act, ref).astype(np.int32)
    assert np.abs(dq).max() <= 1 and np.count_nonzero(dq) <= 3e-3 * dq.size + 1
    if act != orc.Q8_1:   # the reference has no to_float for Q8_1 (k_quants.rs:693-695)
        back, back_ref = orc.dequantize(act, got), orc.dequantize(act, ref)
        assert np.abs(back - back_ref).max() <= 1.01 * np.abs(back_ref).max() / 127
        assert np.linalg.norm(back - back_ref) <= 2e-3 * np.linalg.norm(back_ref)
    canon = canonical_rms_norm(x, alpha, eps)
    assert np.abs(canon - orc.rms_norm(x, alpha, eps)).max() <= 1e-5 * np.abs(canon).max()


def test_rms_norm_quantizer_ragged_row_and_eps(qh):
    # Q8_0 activations allow rows that are not whole 256-element chunks; eps must count
    x, alpha = rms_inputs(3, 4, 32 * 37)
    x *= 1e-3
    for eps in (1e-5, 0.25):
        got = qh.quantize_act(orc.Q8_0, dev(x), qh.PRE_RMS_NORM, dev(alpha), eps).cpu().numpy()
        assert np.array_equal(got, canonical_rms_blocks(orc.Q8_0, x, alpha, eps))
    # an all-zero row: m = sqrt(eps), every quant zero, d = 0
    z = np.zeros((1, 512), np.float32)
    got = qh.quantize_act(orc.Q8K, dev(z), qh.PRE_RMS_NORM, dev(np.ones(512, np.float32)), 1e-6).cpu().numpy()
    assert not got.any()


@pytest.mark.parametrize("act", [orc.Q8K, orc.Q8_0, orc.Q8_1])
@pytest.mark.parametrize("m,k", [(1, 4096), (4, 11008), (3, 512)])
def test_silu_mul_quantizer_equals_two_steps(qh, act, m, k):
    rng = np.random.default_rng(k + m)
    a = (rng.standard_normal((m, k)) * 3).astype(np.float32)
    b = rng.standard_normal((m, k)).astype(np.float32)
    a[0, :8] = [0.0, -0.0, 40.0, -40.0, 88.0, -88.0, -100.0, 1e-30]
    h = qh.silu_mul(dev(a), dev(b))
    got = qh.quantize_act(act, dev(a), qh.PRE_SILU_MUL, dev(b))
    assert torch.equal(got, qh.quantize_act(act, h))
    # the device's silu * mul against the oracle's: a few units in the last place (exp differs)
    want = orc.silu_mul(a, b)
    err = np.abs(h.cpu().numpy().astype(np.float64) - want.astype(np.float64))
    assert (err <= 4 * np.spacing(np.abs(want)).astype(np.float64) + 1e-37).all()


@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
@pytest.mark.parametrize("m,k,n", [(1, 4096, 512), (1, 11008, 130), (1, 256, 40), (2, 4096, 64), (7, 1024, 96),
                                   (40, 512, 64)])
def test_matmul_with_rms_norm(qh, dt, m, k, n):
    w, _ = make_inputs(k + n, m, k, n)
    x, alpha = rms_inputs(n + m, m, k)
    eps = 1e-5
    wq = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, wq, n, k)
    got = qh.qmatmul(qw, dev(x), pre=qh.PRE_RMS_NORM, aux=dev(alpha), eps=eps)
    # the same kernels on host-prepared input, in the kernels' order of operations: same bits
    if dt in (orc.Q4_0, orc.Q4_1, orc.Q5_0, orc.Q5_1, orc.Q8_0):   # the types with 32-element activation blocks
        assert torch.equal(got, qh.qmatmul(qw, dev(canonical_rms_norm(x, alpha, eps)), staged(qh, m)))
    elif m == 1 and dt != orc.Q2K:   # one row: x * alpha through the matmul, the result times the row's scale
        # (Q2K: two sums, the scale inside each: equal to rounding only, covered by the oracle comparison below)
        plain = qh.qmatmul(qw, dev((x * alpha[None, :]).astype(np.float32))).cpu().numpy()
        assert np.array_equal(got.cpu().numpy(), plain * canonical_scale(x, eps)[:, None])
    # the reference sequence rms_norm -> QMatMul::forward
    check_f32(got.cpu().numpy(), orc.matmul(dt, orc.rms_norm(x, alpha, eps), wq, n))


@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
@pytest.mark.parametrize("m,k,n", [(1, 11008, 256), (1, 4096, 77), (3, 2048, 64), (16, 1024, 48), (33, 512, 64)])
def test_matmul_with_silu_mul(qh, dt, m, k, n):
    w, a = make_inputs(k + n + 1, m, k, n)
    b = np.random.default_rng(n).standard_normal((m, k)).astype(np.float32)
    wq = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, wq, n, k)
    got = qh.qmatmul(qw, dev(a), pre=qh.PRE_SILU_MUL, aux=dev(b))
    assert torch.equal(got, qh.qmatmul(qw, qh.silu_mul(dev(a), dev(b)), staged(qh, m)))
    check_f32(got.cpu().numpy(), orc.matmul(dt, orc.silu_mul(a, b), wq, n))


def test_host_mirror_methods(qh):
    from candle_amd.quantized import GgmlDType, QMatMul, QTensor
    w, x = make_inputs(5, 3, 512, 64)
    alpha = np.linspace(0.5, 1.5, 512, dtype=np.float32)
    mm = QMatMul.from_qtensor(QTensor.quantize(dev(w), GgmlDType.Q4K))
    wq = mm.qtensor.data()
    got = mm.forward_rms_norm(dev(x), dev(alpha), 1e-6)
    check_f32(got.cpu().numpy(), orc.matmul(orc.Q4K, orc.rms_norm(x, alpha, 1e-6), wq, 64))
    got = mm.forward_silu_mul(dev(x), dev(x[::-1].copy()))
    check_f32(got.cpu().numpy(), orc.matmul(orc.Q4K, orc.silu_mul(x, x[::-1].copy()), wq, 64))
    # rank-3 inputs keep their leading dimensions
    x3 = dev(np.stack([x, x]))
    assert mm.forward_rms_norm(x3, dev(alpha), 1e-6).shape == (2, 3, 64)


@pytest.mark.parametrize("pre_name", ["silu", "rms"])
def test_grouped_with_fused_step(qh, pre_name):
    rng = np.random.default_rng(11)
    n_e, k, n, tokens = 4, 512, 96, 20
    ws = [orc.quantize(orc.Q4K, (rng.standard_normal((n, k)) * 0.05).astype(np.float32)) for _ in range(n_e)]
    experts = [qh.QWeight.from_ggml(orc.Q4K, b, n, k) for b in ws]
    counts = [11, 0, 20, 3]
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    row_ids = np.concatenate([rng.permutation(tokens)[:c] for c in counts]).astype(np.int32)
    x = rng.standard_normal((tokens, k)).astype(np.float32)
    if pre_name == "silu":
        aux = rng.standard_normal((tokens, k)).astype(np.float32)
        got = qh.qmatmul_grouped(experts, dev(x), dev(row_ids), offsets, pre=qh.PRE_SILU_MUL, aux=dev(aux))
        staged = qh.silu_mul(dev(x), dev(aux))
        inp = orc.silu_mul(x, aux)
    else:
        aux = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
        got = qh.qmatmul_grouped(experts, dev(x), dev(row_ids), offsets, pre=qh.PRE_RMS_NORM, aux=dev(aux), eps=1e-5)
        staged = None   # K-quant experts: the row scale goes into the block scales, covered by the byte test above
        inp = orc.rms_norm(x, aux, 1e-5)
    if staged is not None:
        assert torch.equal(got, qh.qmatmul_grouped(experts, staged, dev(row_ids), offsets))
    for e in range(n_e):
        rows = row_ids[offsets[e]:offsets[e + 1]]
        if rows.size:
            check_f32(got[offsets[e]:offsets[e + 1]].cpu().numpy(), orc.matmul(orc.Q4K, inp[rows], ws[e], n))


def test_fused_argument_errors(qh):
    w, x = make_inputs(1, 2, 256, 16)
    qw = qh.QWeight.from_ggml(orc.Q8_0, orc.quantize(orc.Q8_0, w), 16, 256)
    xd = dev(x)
    with pytest.raises(qh.QHipError, match="rms-norm"):
        qh.qmatmul(qw, xd, pre=qh.PRE_RMS_NORM, aux=dev(np.ones(255, np.float32)), eps=1e-5)
    with pytest.raises(qh.QHipError, match="silu-mul"):
        qh.qmatmul(qw, xd, pre=qh.PRE_SILU_MUL, aux=dev(np.ones((1, 256), np.float32)))
    with pytest.raises(qh.QHipError):
        qh.qmatmul(qw, xd, pre=7, aux=xd)
    # straight at the C ABI: null aux, unknown step, misaligned aux, a reused workspace
    import ctypes as C
    L = qh.load()
    ws = torch.empty(L.cq_workspace_bytes(qw.handle, 2, 0), dtype=torch.uint8, device="cuda")
    y = torch.empty((2, 16), dtype=torch.float32, device="cuda")
    call = lambda pre, aux, flags=0: L.cq_qmatmul_fused(qw.handle, pre, C.c_void_p(xd.data_ptr()), aux, 1e-5, 2,
                                                        C.c_void_p(y.data_ptr()), flags, C.c_void_p(ws.data_ptr()),
                                                        ws.numel(), None)
    assert call(qh.PRE_RMS_NORM, None) == -1 and b"null" in L.cq_last_error()
    assert call(9, C.c_void_p(xd.data_ptr())) == -1 and b"unknown fused step" in L.cq_last_error()
    assert call(qh.PRE_SILU_MUL, C.c_void_p(xd.data_ptr() + 4)) == -1 and b"aligned" in L.cq_last_error()
    assert call(qh.PRE_SILU_MUL, C.c_void_p(xd.data_ptr()), qh.FLAG_REUSE_ACT) == -1
    assert call(qh.PRE_NONE, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(y, qh.qmatmul(qw, xd))


@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
@pytest.mark.parametrize("m", [1, 3, 9])
def test_rms_norm_rows_without_a_finite_scale(qh, dt, m):
    """A row with a NaN, with an infinity, or whose squares overflow has no finite non-zero scale: the reference's
    normalised row is then all NaN or all zero, quantizes to zero blocks and gives zeros.  The fused calls (Q8K
    activations keep the scale out of the quantized elements) give the same, and the other rows their usual values."""
    rng = np.random.default_rng(31 * int(dt) + m)
    k, n, eps = 1024, 40, 1e-5
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    alpha = rng.standard_normal(k).astype(np.float32)
    x[0, 5] = np.nan
    if m > 2:
        x[1, 700] = np.inf
        x[2, :] *= np.float32(1e25)          # squares overflow: scale 0
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    with np.errstate(all="ignore"):
        normed = orc.rms_norm(x, alpha, eps)
        ref = orc.matmul(dt, normed, blocks, n)
    bad_rows = [0] + ([1, 2] if m > 2 else [])
    assert not ref[bad_rows].any()                      # the reference's own answer for such rows: zeros
    for flags in (0, qh.FLAG_STAGED_ACT):
        got = qh.qmatmul(qw, dev(x), flags, pre=qh.PRE_RMS_NORM, aux=dev(alpha), eps=eps).cpu().numpy()
        assert not got[bad_rows].any(), flags
        good = [r for r in range(m) if r not in bad_rows]
        if good:
            check_f32(got[good], ref[good])
    acts = qh.quantize_act(orc.VEC_DOT_TYPE[dt], dev(x), pre=qh.PRE_RMS_NORM, aux=dev(alpha), eps=eps).cpu().numpy()
    rowb = acts.size // m
    for r in bad_rows:
        assert not acts.reshape(m, rowb)[r].any()       # zero blocks, as the reference's quantizer writes for them
