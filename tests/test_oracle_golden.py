"""Pins the CPU oracle against every golden vector the reference's own tests hold
for the quantized matmul path (candle-core/tests/quantized_tests.rs) and against
what the mathematics fixes.  No GPU needed."""
import numpy as np
import pytest

from oracle import cpu_oracle as orc

DT = {"q4_0": orc.Q4_0, "q4_1": orc.Q4_1, "q5_0": orc.Q5_0, "q5_1": orc.Q5_1, "q8_0": orc.Q8_0, "q2k": orc.Q2K, "q3k": orc.Q3K, "q4k": orc.Q4K, "q5k": orc.Q5K, "q6k": orc.Q6K, "q8k": orc.Q8K}


# ---------------------------------------------------------------- f16 ----
def test_f16_to_f32_exhaustive():
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([orc.f16_to_f32(int(v)) for v in h], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()


def test_f32_to_f16_matches_ieee_rne():
    rng = np.random.default_rng(1)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 6e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 3e-8,
                  6.1e-5, 6.103515625e-5, 1.0009765625, 1.00048828125, 1.00146484375, np.inf, -np.inf],
                 dtype=np.float32),
        # every f16 value, and the exact midpoints between neighbours (tie cases)
        np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32),
        ((np.arange(0, 0x7bff, dtype=np.uint16).view(np.float16).astype(np.float64)
          + np.arange(1, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float64)) / 2).astype(np.float32),
    ])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([orc.f32_to_f16(float(v)) for v in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


# --------------------------------------------------- G1/G2: Q4_0 matmul ----
def test_q4_0_matmul_golden(goldens):
    g = goldens["q4_0_matmul_m3_k64_n4"]
    m, k, n = 3, 64, 4
    lhs = np.arange(m * k, dtype=np.float32).reshape(m, k)
    rhs = np.arange(k * n, dtype=np.float32).reshape(n, k)
    w = orc.quantize(orc.Q4_0, rhs)
    assert w.size == 8 * 18
    dst = orc.matmul(orc.Q4_0, lhs, w, n)
    assert np.round(dst).ravel().tolist() == g["rounded"]
    assert (lhs @ rhs.T).tolist() == g["f32_matmul"]


def test_q4_0_matmul_neg_golden(goldens):
    g = goldens["q4_0_matmul_neg_m3_k64_n4"]
    m, k, n = 3, 64, 4
    lhs = (np.arange(m * k, dtype=np.float32) - np.float32(m * k) / np.float32(2.0)).reshape(m, k)
    rhs = (np.arange(k * n, dtype=np.float32) - np.float32(k * n) / np.float32(3.0)).reshape(n, k)
    dst = orc.matmul(orc.Q4_0, lhs, orc.quantize(orc.Q4_0, rhs), n)
    # Rust's f32::round is half-away-from-zero; no output is near a tie here.
    assert np.round(dst).ravel().tolist() == g["rounded"]
    # batch invariance (quantized_tests.rs:169-177): stacking rows leaves each row's result unchanged
    dst2 = orc.matmul(orc.Q4_0, np.concatenate([lhs, lhs]), orc.quantize(orc.Q4_0, rhs), n)
    assert np.array_equal(dst2[3:], dst) and np.array_equal(dst2[:3], dst)


# ------------------------------------------------ G3: Q4_0 round trip ----
def test_q4_0_roundtrip_golden(goldens):
    g = goldens["q4_0_roundtrip_ramp128"]
    src = np.arange(128, dtype=np.float32)
    dst = orc.dequantize(orc.Q4_0, orc.quantize(orc.Q4_0, src))
    want = np.array(g["dst"], dtype=np.float32)
    assert np.array_equal(dst.view(np.uint32), want.view(np.uint32))  # includes the sign of -0.0


def test_q5_0_roundtrip_golden(goldens):
    """quantize_q5_0 (quantized_tests.rs:289-319): ramp 0..127 through Q5_0 and back, 3 decimals."""
    g = goldens["q5_0_roundtrip_ramp128"]
    src = np.arange(128, dtype=np.float32)
    dst = orc.dequantize(orc.Q5_0, orc.quantize(orc.Q5_0, src))
    # round_vector: (1000 * x).round() / 1000 in f32, half away from zero
    t = np.float32(1000.0) * dst
    rounded = (np.copysign(np.floor(np.abs(t) + np.float32(0.5)), t)).astype(np.float32) / np.float32(1000.0)
    want = np.array(g["dst"], dtype=np.float32)
    assert np.array_equal(rounded.view(np.uint32), want.view(np.uint32)), (rounded, want)   # includes the sign of -0.0


def test_q5_1_roundtrip_golden(goldens):
    """quantize_q5_1 (quantized_tests.rs:321-351): the ramp 0..127 comes back exactly."""
    g = goldens["q5_1_roundtrip_ramp128"]
    src = np.arange(128, dtype=np.float32)
    blocks = orc.quantize(orc.Q5_1, src)
    assert blocks.size == 4 * 24
    dst = orc.dequantize(orc.Q5_1, blocks)
    t = np.float32(1000.0) * dst
    rounded = (np.copysign(np.floor(np.abs(t) + np.float32(0.5)), t)).astype(np.float32) / np.float32(1000.0)
    assert rounded.tolist() == g["dst"]


# ------------------------------------------- G4: K-quant round trips ----
def _test_vector2(bound, size=1024):
    v = np.arange(size, dtype=np.float32)
    return (v - np.float32(size) / np.float32(2.0)) * np.float32(bound) / (np.float32(size) / np.float32(2.0))


@pytest.mark.parametrize("name", ["q2k", "q3k", "q4k", "q5k", "q6k", "q8k"])
def test_kquant_roundtrip_golden(goldens, name):
    g = goldens["kquant_roundtrip_test_vector2"]
    idx = g["indices"]
    src = _test_vector2(0.5)
    assert [float(src[i]) for i in idx] == [float(np.float32(v)) for v in g["src_spot"]]
    dst = orc.dequantize(DT[name], orc.quantize(DT[name], src))
    assert np.abs(dst - src).max() < g[name]["tol_bound_0p5"]
    rounded = np.round(np.float32(1000.0) * dst) / np.float32(1000.0)
    got = [float(rounded[i]) for i in idx]
    want = [float(np.float32(v)) for v in g[name]["spot"]]
    assert got == want, (got, want)
    big = _test_vector2(128.0)
    dbig = orc.dequantize(DT[name], orc.quantize(DT[name], big))
    assert np.abs(dbig - big).max() < g[name]["tol_bound_128"]


# --------------------------------------------- G5: total quantization error ----
def _ggml_like(offset):
    i = np.arange(4096, dtype=np.float32)
    return (np.float32(0.1) + np.float32(2.0) * np.cos(i + np.float32(offset), dtype=np.float32)).astype(np.float32)


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "q2k", "q3k", "q4k", "q5k", "q6k", "q8k", "q8_0"])
def test_quantization_total_error(goldens, name):
    src = _ggml_like(0.0)
    dst = orc.dequantize(DT[name], orc.quantize(DT[name], src))
    rmse = np.sqrt(np.sum((src - dst) ** 2, dtype=np.float32)) / np.float32(src.size)
    g = goldens["quantization_total_error"]
    assert rmse <= g[{"q3k": "max_rmse_over_n_3bits", "q2k": "max_rmse_over_n_2bits"}.get(name, "max_rmse_over_n")]


# ------------------------------------------------- G6: dot product error ----
@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q2k", "q3k", "q4k", "q5k", "q6k", "q8k"])
def test_dot_product_error(goldens, name):
    g = goldens["dot_product_error"]
    ramp = (np.arange(4096, dtype=np.float32) / np.float32(4096))
    for a, b, err_m in ((_ggml_like(0.0), _ggml_like(1.0), 1.0), (ramp, ramp, 2.0)):
        dt = DT[name]
        aq = orc.quantize(dt, a)
        bq = orc.quantize(orc.VEC_DOT_TYPE[dt], b)
        res = orc.vec_dot(dt, a.size, aq, bq)
        ref = float(np.sum(a * b, dtype=np.float32))
        err = abs(res - ref) / a.size
        assert np.isfinite(err) and err <= g["max_dot_product_error"]
        assert err - g["leniency"] <= g["ggml_error"][name] * err_m, (name, err)


# ------------------------------------- G7: seeded full path m=11,k=512,n=21 ----
@pytest.mark.parametrize("name", ["q2k", "q3k", "q4k", "q5k", "q6k", "q8k"])
def test_seeded_matmul_golden(goldens, seeded_inputs, name):
    g = goldens["seeded_matmul_m11_k512_n21"]
    lhs, rhs = seeded_inputs
    m, k, n = 11, 512, 21
    dst = orc.matmul(DT[name], lhs, orc.quantize(DT[name], rhs), n).ravel()
    got = [float(np.round(np.float32(1000.0) * dst[i]) / np.float32(1000.0)) for i in g["flat_indices"]]
    want = [float(np.float32(v)) for v in g[name]]
    assert got == want, (got, want)


# ------------------------------------------------ G8: batch invariance ----
@pytest.mark.parametrize("name", ["q4_0", "q8_0", "q4k", "q5k", "q6k"])
def test_batch_invariance(seeded_inputs, name):
    lhs, rhs = seeded_inputs
    lhs, rhs = lhs[:2, :256], rhs[:6, :256]
    w = orc.quantize(DT[name], rhs)
    mm = orc.matmul(DT[name], lhs, w, 6)
    for reps in (2, 3, 6):
        mmr = orc.matmul(DT[name], np.concatenate([lhs] * reps), w, 6)
        for r in range(reps):
            assert np.array_equal(mmr[2 * r:2 * r + 2], mm)


# --------------------------------------------- G9: generic matmul error ----
@pytest.mark.parametrize("name", ["q4_0", "q8_0", "q4k", "q5k", "q6k"])
def test_generic_matmul_error(goldens, name):
    m, n, k = goldens["generic_matmul_error"]["mnk"]
    lhs = (np.arange(m * k, dtype=np.float32) / np.float32(m * k)).reshape(m, k)
    rhs_kn = (np.arange(k * n, dtype=np.float32) / np.float32(n * k)).reshape(k, n)
    mm = lhs @ rhs_kn
    res = orc.matmul(DT[name], lhs, orc.quantize(DT[name], np.ascontiguousarray(rhs_kn.T)), n)
    err = float(np.sum(np.abs(mm - res) / np.abs(mm))) / (m * n)
    assert err <= goldens["generic_matmul_error"]["max_mean_rel_error"]


# ---------------------- what the mathematics fixes (independent restatements) ----
def _unpack_q4k(blocks):
    b = blocks.reshape(-1, 144)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32)[:, 0]
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float32)[:, 0]
    s = b[:, 4:16].astype(np.int32)
    sc = np.zeros((b.shape[0], 8), np.int32)
    mn = np.zeros((b.shape[0], 8), np.int32)
    for j in range(8):
        if j < 4:
            sc[:, j] = s[:, j] & 63
            mn[:, j] = s[:, j + 4] & 63
        else:
            sc[:, j] = (s[:, j + 4] & 0xF) | ((s[:, j - 4] >> 6) << 4)
            mn[:, j] = (s[:, j + 4] >> 4) | ((s[:, j] >> 6) << 4)
    qs = b[:, 16:].astype(np.int32).reshape(-1, 4, 32)
    q = np.stack([qs & 0xF, qs >> 4], axis=2).reshape(-1, 8, 32)  # [block, sub-block, 32]
    return d, dmin, sc, mn, q


def _unpack_q5k(blocks):
    """Q5K blocks (k_quants.rs:119-127: d, dmin, scales[12], qh[32], qs[128]) unpacked with numpy;
    sub-block j takes bit j of qh[l] as the fifth bit of its element l."""
    b = blocks.reshape(-1, 176)
    as_q4k = np.concatenate([b[:, :16], b[:, 48:]], axis=1)     # same header, scales and nibbles as Q4K
    d, dmin, sc, mn, q = _unpack_q4k(as_q4k)
    qh = b[:, 16:48].astype(np.int32)                            # [block, 32]
    hi = np.stack([(qh >> j) & 1 for j in range(8)], axis=1)     # [block, sub-block, 32]
    return d, dmin, sc, mn, q + 16 * hi


def _unpack_q6k(blocks):
    b = blocks.reshape(-1, 210)
    ql = b[:, :128].astype(np.int32).reshape(-1, 2, 2, 32)   # [blk, half, t, l]
    qh = b[:, 128:192].astype(np.int32).reshape(-1, 2, 32)
    sc = b[:, 192:208].copy().view(np.int8).astype(np.int32)
    d = b[:, 208:210].copy().view(np.float16).astype(np.float32)[:, 0]
    q = np.zeros((b.shape[0], 2, 4, 32), np.int32)
    q[:, :, 0] = (ql[:, :, 0] & 0xF) | ((qh & 3) << 4)
    q[:, :, 1] = (ql[:, :, 1] & 0xF) | (((qh >> 2) & 3) << 4)
    q[:, :, 2] = (ql[:, :, 0] >> 4) | (((qh >> 4) & 3) << 4)
    q[:, :, 3] = (ql[:, :, 1] >> 4) | (((qh >> 6) & 3) << 4)
    return d, sc, (q - 32).reshape(-1, 256)


def _unpack_q8k(blocks):
    b = blocks.reshape(-1, 292)
    d = b[:, 0:4].copy().view(np.float32)[:, 0]
    qs = b[:, 4:260].copy().view(np.int8).astype(np.int32)
    bsums = b[:, 260:292].copy().view(np.int16).astype(np.int32)
    return d, qs, bsums


def test_q8k_bsums_invariant_and_extreme_value():
    rng = np.random.default_rng(5)
    x = rng.standard_normal(2048).astype(np.float32)
    d, qs, bsums = _unpack_q8k(orc.quantize(orc.Q8K, x))
    assert np.array_equal(bsums, qs.reshape(-1, 16, 16).sum(-1))
    # the element with the largest |x| maps to -128 exactly, and d = 1/iscale = max / -128
    xb = x.reshape(-1, 256)
    am = np.abs(xb).argmax(1)
    assert (qs[np.arange(8), am] == -128).all()
    iscale = np.float32(-128.0) / xb[np.arange(8), am]
    assert np.array_equal(d, (np.float32(1.0) / iscale).astype(np.float32))
    # all-zero block: d = 0, qs = 0, bsums = 0
    dz, qz, bz = _unpack_q8k(orc.quantize(orc.Q8K, np.zeros(256, np.float32)))
    assert dz[0] == 0 and not qz.any() and not bz.any()
    # tie on |x| with opposite signs: the first occurrence decides the sign of iscale
    t = np.zeros(256, np.float32); t[3] = 2.0; t[7] = -2.0
    _, qt, _ = _unpack_q8k(orc.quantize(orc.Q8K, t))
    assert qt[0, 3] == -128 and qt[0, 7] == 127  # +128 saturates to 127
    t[3], t[7] = -2.0, 2.0
    _, qt, _ = _unpack_q8k(orc.quantize(orc.Q8K, t))
    assert qt[0, 3] == -128 and qt[0, 7] == 127


def test_q8_0_closed_form():
    rng = np.random.default_rng(6)
    x = rng.standard_normal(1024).astype(np.float32)
    b = orc.quantize(orc.Q8_0, x).reshape(-1, 34)
    d16 = b[:, :2].copy().view(np.float16)[:, 0]
    qs = b[:, 2:].copy().view(np.int8)
    xb = x.reshape(-1, 32)
    d = np.abs(xb).max(1) / np.float32(127.0)
    assert np.array_equal(d16, d.astype(np.float16))
    idv = (np.float32(1.0) / d).astype(np.float32)
    v = xb * idv[:, None]
    want = np.where(v >= 0, np.floor(v + np.float32(0.5)), np.ceil(v - np.float32(0.5)))  # half away
    # |v| <= 127 so v +- 0.5 is exact in f32 except at huge exponents; cross-check with float64
    want64 = np.sign(v.astype(np.float64)) * np.floor(np.abs(v.astype(np.float64)) + 0.5)
    assert np.array_equal(want.astype(np.int32), want64.astype(np.int32))
    assert np.array_equal(qs.astype(np.int32), want64.astype(np.int32))


def test_q8_1_is_q8_0_plus_s():
    """BlockQ8_1::from_float (k_quants.rs:665-691): d and qs are BlockQ8_0::from_float's (pinned by the Q4_0 /
    Q8_0 goldens); `s` against the closed form f16(f16(sum q) * d) and the looser invariant that it is d * sum(q)
    to within one f16 unit in the last place.  What pins `s` independently of this reading is the reference's
    Q4_1 x Q8_1 dot-product test below."""
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(4096) * 3).astype(np.float32)
    b0 = orc.quantize(orc.Q8_0, x).reshape(-1, 34)
    b1 = orc.quantize(orc.Q8_1, x).reshape(-1, 36)
    assert np.array_equal(b0[:, :2], b1[:, :2]) and np.array_equal(b0[:, 2:], b1[:, 4:])
    qs = b1[:, 4:].copy().view(np.int8).astype(np.int32)
    d = b1[:, :2].copy().view(np.float16)[:, 0]
    s = b1[:, 2:4].copy().view(np.float16)[:, 0]
    want = (qs.sum(1).astype(np.float32).astype(np.float16).astype(np.float32) * d.astype(np.float32)).astype(np.float16)
    assert np.array_equal(s.view(np.uint16), want.view(np.uint16))
    exact = d.astype(np.float64) * qs.sum(1)
    ulp = np.spacing(np.abs(s).astype(np.float16)).astype(np.float64)
    assert (np.abs(s.astype(np.float64) - exact) <= ulp).all()


# ---- Q4_1: the reference vectors that depend on the `s` field of Q8_1 blocks ----
def test_q4_1_roundtrip_golden(goldens):
    """quantize_q4_1 (quantized_tests.rs:256-287): ramp 0..127 through Q4_1 and back, 3 decimals."""
    g = goldens["q4_1_roundtrip_ramp128"]
    src = np.arange(128, dtype=np.float32)
    blocks = orc.quantize(orc.Q4_1, src)
    assert blocks.size == 4 * 20
    dst = orc.dequantize(orc.Q4_1, blocks)
    # round_vector: (1000 * x).round() / 1000 in f32, half away from zero (no value is near a tie)
    t = np.float32(1000.0) * dst
    rounded = (np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))).astype(np.float32) / np.float32(1000.0)
    assert rounded.tolist() == [float(np.float32(v)) for v in g["dst_rounded_3"]]


def _seq_dot_f32(a, b):
    """vec_dot_reference (quantized_tests.rs:781-783): f32 products added one by one."""
    acc = np.float32(0.0)
    for p in (a * b).astype(np.float32):
        acc = np.float32(acc + p)
    return float(acc)


def _q4_1_cases():
    ramp = (np.arange(4096, dtype=np.float32) / np.float32(4096))
    return ((_ggml_like(0.0), _ggml_like(1.0), 1.0), (ramp, ramp, 2.0))


def _q4_1_dot_error(a, b, mutate=None):
    aq = orc.quantize(orc.Q4_1, a)
    bq = orc.quantize(orc.Q8_1, b).reshape(-1, 36).copy()
    if mutate is not None:
        d = bq[:, :2].copy().view(np.float16)[:, 0].astype(np.float32)
        s = bq[:, 2:4].copy().view(np.float16)[:, 0].astype(np.float32)
        sumq = bq[:, 4:].copy().view(np.int8).astype(np.int32).sum(1).astype(np.float32)
        with np.errstate(over="ignore"):
            bq[:, 2:4] = mutate(d, s, sumq).astype(np.float16).reshape(-1, 1).view(np.uint8)
    res = orc.vec_dot(orc.Q4_1, a.size, aq, bq.ravel())
    return abs(res - _seq_dot_f32(a, b)) / a.size


def test_q4_1_dot_product_error_pins_q8_1_s(goldens):
    """ggml_matmul_error_test::<BlockQ4_1> (quantized_tests.rs:795, :866): Q4_1 weights against Q8_1 activations
    on the cos vectors (bound 0.008) and the ramps (x2).  The result is sum_i * d * d8 + m * s per block, so this
    is the reference-held check of BlockQ8_1::from_float's `s`."""
    g = goldens["dot_product_error"]
    for a, b, err_m in _q4_1_cases():
        err = _q4_1_dot_error(a, b)
        assert np.isfinite(err) and err <= g["max_dot_product_error"]
        assert err - g["leniency"] <= g["ggml_error"]["q4_1"] * err_m, err


@pytest.mark.parametrize("mutant", ["dropped", "negated", "unscaled_sum", "scale_only", "halved", "one_percent_low"])
def test_q4_1_dot_product_bound_rejects_wrong_s(goldens, mutant):
    """The bound above is sharp enough: each plausible mistake in `s` fails it on at least one of the two inputs."""
    g = goldens["dot_product_error"]
    mutate = {
        "dropped": lambda d, s, sumq: np.zeros_like(s),
        "negated": lambda d, s, sumq: -s,
        "unscaled_sum": lambda d, s, sumq: sumq,
        "scale_only": lambda d, s, sumq: d,
        "halved": lambda d, s, sumq: s * np.float32(0.5),
        # the reference's bound sits 1.1 % above the correct result on the cos vectors, so even this fails it
        "one_percent_low": lambda d, s, sumq: s * np.float32(0.99),
    }[mutant]
    failed = False
    for a, b, err_m in _q4_1_cases():
        err = _q4_1_dot_error(a, b, mutate)
        if not np.isfinite(err) or err > g["max_dot_product_error"] or err - g["leniency"] > g["ggml_error"]["q4_1"] * err_m:
            failed = True
    assert failed, mutant


def test_q4_1_closed_form_and_matmul_driver():
    """Q4_1 from_float / to_float / dot against an independent numpy evaluation (float64 for the combine), and the
    matmul driver with Q8_1 as the VecDotType (k_quants.rs:260, :1842-1883)."""
    rng = np.random.default_rng(21)
    m, k, n = 3, 256, 5
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = (rng.standard_normal((n, k)) * 0.02 + 0.01).astype(np.float32)
    w = orc.quantize(orc.Q4_1, rhs).reshape(n, k // 32, 20)
    d = w[..., :2].copy().view(np.float16)[..., 0]
    mn = w[..., 2:4].copy().view(np.float16)[..., 0]
    q = np.concatenate([w[..., 4:] & 15, w[..., 4:] >> 4], axis=-1).astype(np.int64)   # elements j, then j + 16
    xb = rhs.reshape(n, k // 32, 32)
    assert np.array_equal(mn, xb.min(-1).astype(np.float16))
    assert np.array_equal(d, ((xb.max(-1) - xb.min(-1)) / np.float32(15.0)).astype(np.float16))
    deq = orc.dequantize(orc.Q4_1, w.ravel()).reshape(n, k // 32, 32)
    assert np.array_equal(deq, q.astype(np.float32) * d.astype(np.float32)[..., None] + mn.astype(np.float32)[..., None])
    assert np.abs(deq - xb).max() <= (xb.max(-1) - xb.min(-1)).max() / 15 * 0.5 + 1e-4
    a = np.stack([orc.quantize(orc.Q8_1, lhs[r]) for r in range(m)]).reshape(m, k // 32, 36)
    d8 = a[..., :2].copy().view(np.float16)[..., 0].astype(np.float64)
    s8 = a[..., 2:4].copy().view(np.float16)[..., 0].astype(np.float64)
    q8 = a[..., 4:].copy().view(np.int8).astype(np.int64)
    sumi = np.einsum("nbl,mbl->mnb", q, q8)
    ref = (sumi * d.astype(np.float64)[None] * d8[:, None] + mn.astype(np.float64)[None] * s8[:, None]).sum(-1)
    out = orc.matmul(orc.Q4_1, lhs, w.ravel(), n)
    assert np.abs(out - ref).max() <= 1e-5 * np.abs(ref).max() + 1e-6
    # odd block counts are refused like the reference (k_quants.rs:274-276)
    with pytest.raises(ValueError):
        orc.vec_dot(orc.Q4_1, 32, w.ravel()[:20], a.ravel()[:36])


def _unpack_q2k(w):
    """Independent unpacking of Q2K blocks (k_quants.rs:96-103, :841-872): d, dmin, the sixteen 4-bit scales and mins,
    the 256 two-bit quants."""
    b = w.reshape(-1, 84)
    scb, qs = b[:, :16].astype(np.int64), b[:, 16:80].astype(np.int64)
    d = b[:, 80:82].copy().view(np.float16)[:, 0]
    dmin = b[:, 82:84].copy().view(np.float16)[:, 0]
    q = np.zeros((b.shape[0], 256), np.int64)
    for e in range(256):
        q[:, e] = (qs[:, 32 * (e // 128) + e % 32] >> (2 * ((e % 128) // 32))) & 3
    return d, dmin, scb & 0xF, scb >> 4, q


def _unpack_q3k(w):
    """Independent unpacking of Q3K blocks (k_quants.rs:107-114, :1094-1146): d, the sixteen 6-bit scales minus 32,
    and the 256 signed quants (two low bits from qs, minus 4 unless the element's hmask bit is set)."""
    b = w.reshape(-1, 110)
    hmask, qs, scb = b[:, :32].astype(np.int64), b[:, 32:96].astype(np.int64), b[:, 96:108].astype(np.int64)
    d = b[:, 108:110].copy().view(np.float16)[:, 0]
    sc = np.zeros((b.shape[0], 16), np.int64)
    for j in range(16):
        low = (scb[:, j] & 0xF) if j < 8 else (scb[:, j - 8] >> 4)
        sc[:, j] = (low | (((scb[:, 8 + j % 4] >> (2 * (j // 4))) & 3) << 4)) - 32
    q = np.zeros((b.shape[0], 256), np.int64)
    for e in range(256):
        low = (qs[:, 32 * (e // 128) + e % 32] >> (2 * ((e % 128) // 32))) & 3
        q[:, e] = low - 4 * (1 - ((hmask[:, e % 32] >> (e // 32)) & 1))
    return d, sc, q


@pytest.mark.parametrize("name", ["q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q2k", "q3k", "q4k", "q5k", "q6k", "q8k"])
def test_int_dots_and_matmul_bruteforce(name):
    """Integer block dots recomputed by int64 numpy from independently unpacked blocks,
    and the f32 result against a float64 evaluation of the same formula."""
    rng = np.random.default_rng(11)
    dt = DT[name]
    m, k, n = 3, 1024, 5
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    w = orc.quantize(dt, rhs)
    a = np.concatenate([orc.quantize(orc.VEC_DOT_TYPE[dt], lhs[r]) for r in range(m)])
    oi, om = orc.block_int_dots(dt, a, m, w, n, k)
    out = orc.matmul(dt, lhs, w, n)
    if name in ("q2k", "q3k", "q4k", "q5k", "q6k", "q8k"):
        d8, q8, bs = _unpack_q8k(a)
        d8, q8, bs = d8.reshape(m, -1), q8.reshape(m, -1, 256), bs.reshape(m, -1, 16)
        if name in ("q4k", "q5k"):
            d, dmin, sc, mn, q = _unpack_q4k(w) if name == "q4k" else _unpack_q5k(w)
            kb = k // 256
            d, dmin = d.reshape(n, kb), dmin.reshape(n, kb)
            sc, mn, q = sc.reshape(n, kb, 8), mn.reshape(n, kb, 8), q.reshape(n, kb, 8, 32)
            sub = np.einsum("nbjl,mbjl->mnbj", q.astype(np.int64), q8.reshape(m, kb, 8, 32).astype(np.int64))
            I = (sub * sc[None]).sum(-1)
            Mn = np.einsum("mbj,nbj->mnb", bs.reshape(m, kb, 8, 2).sum(-1).astype(np.int64), mn.astype(np.int64))
            assert np.array_equal(oi, I) and np.array_equal(om, Mn)
            ref = (d[None].astype(np.float64) * d8[:, None] * I - dmin[None].astype(np.float64) * d8[:, None] * Mn).sum(-1)
        elif name == "q2k":
            d, dmin, sc, mn, q = _unpack_q2k(w)
            kb = k // 256
            d, dmin = d.reshape(n, kb), dmin.reshape(n, kb)
            sc, mn, q = sc.reshape(n, kb, 16), mn.reshape(n, kb, 16), q.reshape(n, kb, 16, 16)
            sub = np.einsum("nbjl,mbjl->mnbj", q, q8.reshape(m, kb, 16, 16).astype(np.int64))
            I = (sub * sc[None]).sum(-1)
            Mn = np.einsum("mbj,nbj->mnb", bs.astype(np.int64), mn)
            assert np.array_equal(oi, I) and np.array_equal(om, Mn)
            ref = (d[None].astype(np.float64) * d8[:, None] * I - dmin[None].astype(np.float64) * d8[:, None] * Mn).sum(-1)
        elif name in ("q6k", "q3k"):
            d, sc, q = _unpack_q6k(w) if name == "q6k" else _unpack_q3k(w)
            kb = k // 256
            d, sc, q = d.reshape(n, kb), sc.reshape(n, kb, 16), q.reshape(n, kb, 16, 16)
            sub = np.einsum("nbjl,mbjl->mnbj", q.astype(np.int64), q8.reshape(m, kb, 16, 16).astype(np.int64))
            I = (sub * sc[None]).sum(-1)
            assert np.array_equal(oi, I)
            ref = (d[None].astype(np.float64) * d8[:, None] * I).sum(-1)
        else:
            dw, qw, _ = _unpack_q8k(w)
            kb = k // 256
            I = np.einsum("nbl,mbl->mnb", qw.reshape(n, kb, 256).astype(np.int64), q8.astype(np.int64))
            assert np.array_equal(oi, I)
            ref = (dw.reshape(n, kb)[None].astype(np.float64) * d8[:, None] * I).sum(-1)
    elif name in ("q4_1", "q5_1"):
        ab = a.reshape(m, -1, 36)
        da = ab[:, :, :2].copy().view(np.float16)[..., 0].astype(np.float64)
        sa = ab[:, :, 2:4].copy().view(np.float16)[..., 0].astype(np.float64)
        qa = ab[:, :, 4:].copy().view(np.int8).astype(np.int64)
        wb = w.reshape(n, -1, 20 if name == "q4_1" else 24)
        dw = wb[:, :, :2].copy().view(np.float16)[..., 0].astype(np.float64)
        mw = wb[:, :, 2:4].copy().view(np.float16)[..., 0].astype(np.float64)
        nib = wb[:, :, -16:].astype(np.int64)
        qw = np.concatenate([nib & 0xF, nib >> 4], axis=-1)
        if name == "q5_1":
            qh = wb[:, :, 4:8].copy().view(np.uint32)[..., 0].astype(np.int64)
            qw = qw | (((qh[..., None] >> np.arange(32)) & 1) << 4)
        I = np.einsum("nbl,mbl->mnb", qw, qa)
        assert np.array_equal(oi, I)
        ref = (I * dw[None] * da[:, None] + mw[None] * sa[:, None]).sum(-1)
    else:
        ab = a.reshape(m, -1, 34)
        da = ab[:, :, :2].copy().view(np.float16)[..., 0].astype(np.float64)
        qa = ab[:, :, 2:].copy().view(np.int8).astype(np.int64)
        if name == "q4_0":
            wb = w.reshape(n, -1, 18)
            dw = wb[:, :, :2].copy().view(np.float16)[..., 0].astype(np.float64)
            nib = wb[:, :, 2:].astype(np.int64)
            qw = np.concatenate([nib & 0xF, nib >> 4], axis=-1) - 8
        elif name == "q5_0":
            wb = w.reshape(n, -1, 22)
            dw = wb[:, :, :2].copy().view(np.float16)[..., 0].astype(np.float64)
            qh = wb[:, :, 2:6].copy().view(np.uint32)[..., 0].astype(np.int64)
            nib = wb[:, :, 6:].astype(np.int64)
            fifth = (qh[..., None] >> np.arange(32)) & 1
            qw = (np.concatenate([nib & 0xF, nib >> 4], axis=-1) | (fifth << 4)) - 16
        else:
            wb = w.reshape(n, -1, 34)
            dw = wb[:, :, :2].copy().view(np.float16)[..., 0].astype(np.float64)
            qw = wb[:, :, 2:].copy().view(np.int8).astype(np.int64)
        I = np.einsum("nbl,mbl->mnb", qw, qa)
        assert np.array_equal(oi, I)
        ref = (I * dw[None] * da[:, None]).sum(-1)
    rel = np.linalg.norm(out - ref) / np.linalg.norm(ref)
    assert rel < 2e-6, rel
    # and the quantized product approximates the f32 product within quantization noise
    mm = lhs.astype(np.float64) @ rhs.astype(np.float64).T
    assert np.linalg.norm(out - mm) / np.linalg.norm(mm) < {"q3k": 0.25, "q2k": 0.45}.get(name, 0.12)   # two and three bits are noisier


def q8_1_formula_float64(dt, x, blocks, n, k):
    """The formula in float64 from independently unpacked blocks: every integer exact, no f32 rounding."""
    m = x.shape[0]
    a = np.stack([orc.quantize(orc.Q8_1, x[r]) for r in range(m)]).reshape(m, k // 32, 36)
    d8 = a[..., :2].copy().view(np.float16)[..., 0].astype(np.float64)
    s8 = a[..., 2:4].copy().view(np.float16)[..., 0].astype(np.float64)
    q8 = a[..., 4:].copy().view(np.int8).astype(np.int64)                      # [m, k/32, 32]
    kb = k // 256
    if dt == orc.Q4K:
        w = blocks.reshape(n, kb, 144)
        d = w[..., 0:2].copy().view(np.float16)[..., 0].astype(np.float64)
        dmin = w[..., 2:4].copy().view(np.float16)[..., 0].astype(np.float64)
        sc12 = w[..., 4:16].astype(np.int64)
        sc = np.zeros((n, kb, 8), np.int64)
        mn = np.zeros((n, kb, 8), np.int64)
        for j in range(8):                                                     # get_scale_min_k4, utils.rs:49-59
            if j < 4:
                sc[..., j] = sc12[..., j] & 63
                mn[..., j] = sc12[..., j + 4] & 63
            else:
                sc[..., j] = (sc12[..., j + 4] & 0xF) | ((sc12[..., j - 4] >> 6) << 4)
                mn[..., j] = (sc12[..., j + 4] >> 4) | ((sc12[..., j] >> 6) << 4)
        qs = w[..., 16:].astype(np.int64).reshape(n, kb, 4, 32)
        q = np.stack([qs & 15, qs >> 4], axis=3).reshape(n, kb, 8, 32)       # sub-blocks 2g (low), 2g + 1 (high)
        dots = np.einsum("nbjl,mbjl->mnbj", q, q8.reshape(m, kb, 8, 32))
        sd = (dots * sc[None] * d8.reshape(m, 1, kb, 8)).sum(-1)
        sm = (mn[None] * s8.reshape(m, 1, kb, 8)).sum(-1)
        return (d[None] * sd - dmin[None] * sm).sum(-1)
    w = blocks.reshape(n, kb, 210)
    ql = w[..., :128].astype(np.int64).reshape(n, kb, 2, 64)
    qh = w[..., 128:192].astype(np.int64).reshape(n, kb, 2, 32)
    scl = w[..., 192:208].copy().view(np.int8).astype(np.int64)
    d = w[..., 208:210].copy().view(np.float16)[..., 0].astype(np.float64)
    q = np.zeros((n, kb, 2, 128), np.int64)                                    # k_quants.rs:1716-1746
    for half in range(2):
        l = np.arange(32)
        q[:, :, half, l] = (ql[:, :, half, l] & 15) | (((qh[:, :, half, l] >> 0) & 3) << 4)
        q[:, :, half, l + 32] = (ql[:, :, half, l + 32] & 15) | (((qh[:, :, half, l] >> 2) & 3) << 4)
        q[:, :, half, l + 64] = (ql[:, :, half, l] >> 4) | (((qh[:, :, half, l] >> 4) & 3) << 4)
        q[:, :, half, l + 96] = (ql[:, :, half, l + 32] >> 4) | (((qh[:, :, half, l] >> 6) & 3) << 4)
    q = (q.reshape(n, kb, 16, 16) - 32)
    dots = np.einsum("nbjl,mbjl->mnbj", q, q8.reshape(m, kb, 16, 16))
    d8g = np.repeat(d8.reshape(m, kb, 8), 2, axis=-1)                          # group j lies in Q8_1 block j // 2
    return (d[None] * (dots * scl[None] * d8g[:, None]).sum(-1)).sum(-1)


@pytest.mark.parametrize("name", ["q4k", "q6k"])
@pytest.mark.parametrize("m,k,n", [(1, 256, 8), (3, 512, 37), (5, 4096, 16)])
def test_q8_1_variant_exact_formula(name, m, k, n):
    """`orc_matmul_q8_1` against the formula of candle-kernels/src/quantized.cu:2141-2166 (Q4_K) / :2258-2281 (Q6_K)
    evaluated in float64 from independently unpacked weight blocks and Q8_1 activation blocks: every integer exact, no
    f32 rounding.  A wrong integer, scale, sign or sub-block index anywhere moves a result by far more than f32
    rounding does (2e-5 of the largest result)."""
    dt = DT[name]
    rng = np.random.default_rng(1000 * m + n)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x.ravel()[rng.choice(x.size, size=max(1, x.size // 100), replace=False)] = 8.0
    blocks = orc.quantize(dt, w)
    got = orc.matmul_q8_1(dt, x, blocks, n).astype(np.float64)
    exact = q8_1_formula_float64(dt, x, blocks, n, k)
    assert np.abs(got - exact).max() <= 2e-5 * np.abs(exact).max()


@pytest.mark.parametrize("name", ["q4k", "q6k"])
def test_q8_1_variant_bruteforce(name):
    """Q4K/Q6K x Q8_1 (CUDA formulation, CPU rounding): no CPU reference exists -> parity
    unpinned; checked by float64 brute force on the dequantized operands."""
    rng = np.random.default_rng(13)
    dt = DT[name]
    m, k, n = 2, 512, 4
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    w = orc.quantize(dt, rhs)
    out = orc.matmul_q8_1(dt, lhs, w, n)
    wd = orc.dequantize(dt, w).reshape(n, k).astype(np.float64)
    a1 = np.stack([orc.quantize(orc.Q8_1, lhs[r]) for r in range(m)]).reshape(m, -1, 36)
    d = a1[:, :, :2].copy().view(np.float16)[..., 0].astype(np.float64)
    qa = a1[:, :, 4:].copy().view(np.int8).astype(np.float64)
    ad = (qa * d[..., None]).reshape(m, k)
    ref = ad @ wd.T
    # the min term uses s = f16(f16(sum q)*d) instead of d*sum q: small f16 rounding differences
    assert np.linalg.norm(out - ref) / np.linalg.norm(ref) < 2e-3


def test_moe_route_and_ffn_match_dense_masked():
    rng = np.random.default_rng(17)
    tokens, hidden, ffn, n_e, top_k = 9, 256, 512, 4, 2
    xs = rng.standard_normal((tokens, hidden)).astype(np.float32)
    logits = rng.standard_normal((tokens, n_e)).astype(np.float32)
    rw = orc.softmax_last_dim(logits)
    e64 = np.exp(logits.astype(np.float64) - logits.max(1, keepdims=True))
    assert np.allclose(rw, e64 / e64.sum(1, keepdims=True), rtol=1e-6)
    offsets, row_ids, weights = orc.moe_route(rw, top_k)
    assert offsets[-1] == tokens * top_k
    # independent routing: numpy stable argsort of -rw
    order = np.argsort(-rw, axis=1, kind="stable")[:, :top_k]
    for e in range(n_e):
        rows = row_ids[offsets[e]:offsets[e + 1]]
        assert rows.tolist() == [t for t in range(tokens) if e in order[t]]
        for p, t in zip(range(offsets[e], offsets[e + 1]), rows):
            s = np.float32(0)
            for ee in order[t]:
                s = np.float32(s + rw[t, ee])
            assert weights[p] == np.float32(rw[t, e] / s)
    w1 = [orc.quantize(orc.Q4K, (rng.standard_normal((ffn, hidden)) * 0.05).astype(np.float32)) for _ in range(n_e)]
    w3 = [orc.quantize(orc.Q4K, (rng.standard_normal((ffn, hidden)) * 0.05).astype(np.float32)) for _ in range(n_e)]
    w2 = [orc.quantize(orc.Q6K, (rng.standard_normal((hidden, ffn)) * 0.05).astype(np.float32)) for _ in range(n_e)]
    ys = orc.moe_ffn(orc.Q4K, orc.Q6K, w1, w2, w3, hidden, ffn, xs, offsets, row_ids, weights)
    # dense-masked evaluation: every expert on every token, masked by the routing weight
    dense = np.zeros((tokens, hidden), np.float64)
    for e in range(n_e):
        h1 = orc.matmul(orc.Q4K, xs, w1[e], ffn)
        h3 = orc.matmul(orc.Q4K, xs, w3[e], ffn)
        act = (h1 / (np.float32(1.0) + np.exp(-h1))) * h3
        out = orc.matmul(orc.Q6K, act.astype(np.float32), w2[e], hidden)
        mask = np.zeros(tokens)
        for p in range(offsets[e], offsets[e + 1]):
            mask[row_ids[p]] = weights[p]
        dense += out.astype(np.float64) * mask[:, None]
    assert np.linalg.norm(ys - dense) / np.linalg.norm(dense) < 1e-5


# ------------------------------------------- neighbours of the matmul: rms_norm, silu * mul ----
def test_rms_norm_golden_and_closed_form(goldens):
    g = goldens["rms_norm_2x2x3"]
    x = np.array(g["x"], dtype=np.float32)
    got = orc.rms_norm(x, np.array(g["alpha"], dtype=np.float32), g["eps"])
    assert np.round(got.astype(np.float64), 4).tolist() == g["rounded4"]
    # closed form in float64 on a long row; a dropped eps, a missing division by the row length or
    # alpha applied before the division by m would all show
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((3, 4096)) * 3).astype(np.float32)
    alpha = (1 + 0.1 * rng.standard_normal(4096)).astype(np.float32)
    want = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 0.5) * alpha
    got = orc.rms_norm(x, alpha, 0.5)
    assert np.abs(got - want).max() <= 2e-6 * np.abs(want).max()
    assert np.abs(orc.rms_norm(x, alpha, 1e-5) - want).max() > 1e-3   # eps matters at this size


def test_silu_mul_closed_form():
    rng = np.random.default_rng(6)
    a = np.concatenate([rng.standard_normal(4000) * 4, [0.0, -0.0, 30.0, -30.0, 88.0, -88.0, -104.0]]).astype(np.float32)
    b = rng.standard_normal(a.size).astype(np.float32)
    got = orc.silu_mul(a, b)
    a64 = a.astype(np.float64)
    want = a64 / (1 + np.exp(-a64)) * b
    assert np.abs(got - want).max() <= 1e-6 * np.abs(want).max()
    assert got[4000] == 0.0 and abs(got[4002] - 30.0 * b[4002]) < 1e-5 and abs(got[4006]) < 1e-30
