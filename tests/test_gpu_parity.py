"""Parity of the HIP path (through the C ABI) against the CPU oracle on identical seeded inputs.

Bars (BASELINE north star): quantized activation blocks and per-block integer dot products
bit-exact; f32 outputs within relative L2 1e-4 and max-abs <= 1e-3 * ||row||_2.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from oracle import cpu_oracle as orc  # noqa: E402  (checker only)

REL_L2_TOL = 1e-4       # north star: relative L2 error of the f32 output
MAX_ABS_FACTOR = 1e-3   # north star: max-abs <= 1e-3 * ||row||_2


@pytest.fixture(scope="module")
def qh():
    from candle_amd import qhip
    qhip.load()
    assert qhip.load().cq_device_count() >= 1, "no HIP device visible"
    return qhip


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def check_f32(got: np.ndarray, want: np.ndarray):
    got = got.astype(np.float64).reshape(want.shape)
    want64 = want.astype(np.float64)
    for r in range(want.shape[0]):
        nrm = np.linalg.norm(want64[r])
        err = np.linalg.norm(got[r] - want64[r])
        assert err <= REL_L2_TOL * max(nrm, 1e-30), (r, err / max(nrm, 1e-30))
        assert np.abs(got[r] - want64[r]).max() <= MAX_ABS_FACTOR * max(nrm, 1e-30), r


def make_inputs(seed, m, k, n, wscale=0.02, outliers=False):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k)) * wscale).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    if outliers:  # 1% of positions at +-8 sigma (BASELINE config 3)
        idx = rng.choice(x.size, size=max(1, x.size // 100), replace=False)
        x.ravel()[idx] = np.where(rng.random(idx.size) < 0.5, -8.0, 8.0).astype(np.float32)
    return w, x


# Q5_0 and Q3K are held on the device in the planes of Q8_0 and Q6K (same values, same arithmetic), Q4_1 and Q5_1 in
# Q8_0 planes plus a plane of minima whose term the one-launch kernels add themselves and a second launch adds elsewhere (Q2K likewise in Q6K planes): every test below takes them through the boundary
# like the others and compares with the oracle's own code for the type
WEIGHT_DTYPES = [orc.Q4_0, orc.Q4_1, orc.Q5_0, orc.Q5_1, orc.Q8_0, orc.Q2K, orc.Q3K, orc.Q4K, orc.Q5K, orc.Q6K]


# ------------------------------------------------------------ activation quantizers ----
def _act_cases(k):
    rng = np.random.default_rng(k)
    x = rng.standard_normal((5, k)).astype(np.float32)
    x[1] *= 1e-3
    x[2] = 0.0                                    # all-zero blocks
    x[3, ::7] = 8.0; x[3, 3::11] = -8.0           # ties on |x| with both signs, outliers
    x[4] = (np.arange(k, dtype=np.float32) - k / 2) / 64.0  # ramp with exact .5 rounding cases
    return x


@pytest.mark.parametrize("act", [orc.Q8_0, orc.Q8_1, orc.Q8K])
@pytest.mark.parametrize("k", [256, 4096, 11008])
def test_quantize_act_bit_exact(qh, act, k):
    x = _act_cases(k)
    got = qh.quantize_act(act, dev(x)).cpu().numpy()
    want = np.concatenate([orc.quantize(act, x[r]) for r in range(x.shape[0])])
    assert got.size == want.size
    assert np.array_equal(got, want), np.flatnonzero(got != want)[:10]


def test_quantize_act_tie_first_index(qh):
    x = np.zeros((2, 256), np.float32)
    x[0, 200] = -3.0; x[0, 13] = 3.0      # first max is +3 at 13 -> iscale < 0
    x[1, 200] = 3.0; x[1, 13] = -3.0
    got = qh.quantize_act(orc.Q8K, dev(x)).cpu().numpy()
    want = np.concatenate([orc.quantize(orc.Q8K, x[r]) for r in range(2)])
    assert np.array_equal(got, want)


def test_quantize_act_rejects_bad_k(qh):
    with pytest.raises(qh.QHipError):
        qh.quantize_act(orc.Q8K, torch.zeros((1, 128), device="cuda"))


# ---------------------------------------------------------------- storage round trips ----
@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
@pytest.mark.parametrize("n,k", [(3, 512), (37, 1024), (5, 11008)])
def test_repack_roundtrip_and_dequantize(qh, dt, n, k):
    w, _ = make_inputs(n * k + dt, 1, k, n)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    assert qw.dtype == dt and qw.shape == (n, k) and qw.size_in_bytes == blocks.size
    assert np.array_equal(qw.to_ggml(), blocks)
    want = orc.dequantize(dt, blocks).reshape(n, k)
    got = qw.dequantize().cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    got16 = qw.dequantize_f16().cpu().numpy()
    assert np.array_equal(got16.view(np.uint16), want.astype(np.float16).view(np.uint16))


def test_repack_roundtrip_random_bytes(qh):
    # the re-pack is a byte permutation: any byte pattern must survive, not only valid quantizations
    rng = np.random.default_rng(3)
    for dt in WEIGHT_DTYPES:
        n, k = 4, 768
        blocks = rng.integers(0, 256, size=n * k // orc.BLOCK_SIZE[dt] * orc.TYPE_SIZE[dt], dtype=np.uint8)
        qw = qh.QWeight.from_ggml(dt, blocks, n, k)
        assert np.array_equal(qw.to_ggml(), blocks)


@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
def test_weight_quantize_on_device_bit_exact(qh, dt):
    rng = np.random.default_rng(dt)
    n, k = 24, 1024
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    w[0] = 0.0                          # all-zero blocks
    w[1, :256] = 0.5                    # constant sub-blocks (max == min)
    w[2] = np.linspace(-1, 1, k)        # ramp
    w[3, ::2] = -w[3, 1::2]             # |x| ties
    qw = qh.QWeight.zeros(dt, n, k)
    qw.quantize_(dev(w))
    assert np.array_equal(qw.to_ggml(), orc.quantize(dt, w))


def test_weight_create_rejects_bad_shapes(qh):
    with pytest.raises(qh.QHipError):
        qh.QWeight.from_ggml(orc.Q4K, np.zeros(144, np.uint8), 1, 128)      # k not a block multiple
    with pytest.raises(qh.QHipError):
        qh.QWeight.from_ggml(orc.Q4K, np.zeros(100, np.uint8), 1, 256)      # byte size mismatch
    with pytest.raises(qh.QHipError):
        qh.QWeight.from_ggml(5, np.zeros(144, np.uint8), 1, 256)            # unknown dtype


# ------------------------------------------------------------- integer block dots ----
@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
@pytest.mark.parametrize("m,k,n", [(3, 512, 37), (1, 11008, 9), (2, 4096, 16)])
def test_int_dots_bit_exact(qh, dt, m, k, n):
    w, x = make_inputs(1000 + dt + k, m, k, n, outliers=True)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    oi, om = qh.qmatmul_int_dots(qw, dev(x))
    acts = np.concatenate([orc.quantize(orc.VEC_DOT_TYPE[dt], x[r]) for r in range(m)])
    wi, wm = orc.block_int_dots(dt, acts, m, blocks, n, k)
    assert np.array_equal(oi.cpu().numpy(), wi)
    if dt in (orc.Q4K, orc.Q5K):
        assert np.array_equal(om.cpu().numpy(), wm)


# ----------------------------------------------------------------- f32 results ----
@pytest.mark.parametrize("dt,m,k,n", [
    (orc.Q4_0, 1, 4096, 4096),     # config 0
    (orc.Q4K, 1, 4096, 4096),      # config 1: q/k/v/o
    (orc.Q4K, 1, 4096, 11008),     # config 1: gate/up (headline matvec)
    (orc.Q6K, 1, 11008, 4096),     # config 1: down
    (orc.Q6K, 1, 4096, 2048),      # config 1: lm_head rows (a 2048-row slice of the 32000)
    (orc.Q8_0, 1, 4096, 4096),
    (orc.Q4_0, 3, 64, 4),          # smallest shapes of the reference's tests
    (orc.Q4K, 5, 256, 3),
    (orc.Q5K, 1, 4096, 4096),
    (orc.Q5K, 1, 11008, 512),
    (orc.Q5K, 6, 512, 40),
    (orc.Q5K, 20, 1024, 24),       # more rows than one pass of the dot-product kernel takes
])
def test_matvec_matches_oracle(qh, dt, m, k, n):
    w, x = make_inputs(7 * dt + k + n, m, k, n)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    got = qh.qmatmul(qw, dev(x), qh.FLAG_FORCE_MATVEC).cpu().numpy()
    check_f32(got, orc.matmul(dt, x, blocks, n))


@pytest.mark.parametrize("dt,k,n", [(orc.Q6K, 4096, 32000), (orc.Q6K, 11008, 4096), (orc.Q4K, 4096, 11008),
                                     (orc.Q4K, 14336, 4096)])
def test_decode_full_size_row_samples(qh, dt, k, n):
    """The largest decode shapes of the configurations at their full size (lm_head, down and gate/up
    projections, an expert's w2-shaped tensor).  Weights are quantized on the device (bit-exact with
    the oracle's quantizer, checked above); the oracle then recomputes blocks of rows taken from the
    start, the middle and the end of the result out of the very same GGML bytes, and every row of the
    one-launch path must equal the two-launch path bit for bit."""
    rng = np.random.default_rng(dt * 7 + k)
    w = torch.randn((n, k), device="cuda", generator=torch.Generator(device="cuda").manual_seed(dt + n)) * 0.02
    qw = qh.QWeight.zeros(dt, n, k).quantize_(w)
    del w
    x = rng.standard_normal((1, k)).astype(np.float32)
    xd = dev(x)
    y = qh.qmatmul(qw, xd)
    assert torch.equal(y, qh.qmatmul(qw, xd, qh.FLAG_STAGED_ACT))
    got = y.cpu().numpy()
    blocks = qw.to_ggml().reshape(n, -1)
    for r0 in (0, n // 2 - 32, n - 64):
        rows = blocks[r0:r0 + 64].reshape(-1)
        check_f32(got[:, r0:r0 + 64], orc.matmul(dt, x, rows, 64))


@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
@pytest.mark.parametrize("k,n", [(256, 7), (512, 300), (4096, 1000), (11008, 129), (14336, 65)])
def test_fused_decode_equals_two_launch_path(qh, dt, k, n):
    """m = 1 runs as one launch with the activation quantizer in the kernel prologue.  Its result
    must equal, bit for bit, the stand-alone quantizer (checked bit-exact above) followed by the
    plain matvec: same quantized activations, same accumulation order."""
    w, x = make_inputs(31 * dt + k, 1, k, n, outliers=True)
    big = np.float32(np.abs(x).max() + 1.0)          # |x| tie with opposite signs inside the first block
    x[0, 5], x[0, 9] = big, -big
    qw = qh.QWeight.from_ggml(dt, orc.quantize(dt, w), n, k)
    xd = dev(x)
    fused = qh.qmatmul(qw, xd)
    staged = qh.qmatmul(qw, xd, qh.FLAG_STAGED_ACT)
    assert torch.equal(fused, staged)
    x[:] = 0.0
    assert torch.equal(qh.qmatmul(qw, dev(x)), torch.zeros((1, n), device="cuda"))


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q5K, orc.Q6K])
def test_fused_decode_sign_of_scale_cases(qh, dt):
    """The Q8K scale takes the sign of the FIRST element with the largest magnitude.  Blocks where
    that magnitude occurs with both signs (negative first, positive first, in the same eight
    elements, in either half of a wave's pair of blocks), with one sign only, all-zero blocks beside
    non-zero ones, and values that round at a tie: the one-launch decode path must still equal the
    stand-alone quantizer plus matvec bit for bit, and that quantizer the oracle."""
    k, n = 2048, 64
    w, x = make_inputs(77 + dt, 1, k, n)
    x[0] = np.round(x[0] * 8) / 8                       # many products land on exact .5 ties
    big = np.float32(9.5)
    x[0, 0 * 256 + 200], x[0, 0 * 256 + 17] = big, -big          # block 0: negative first
    x[0, 1 * 256 + 3], x[0, 1 * 256 + 250] = big, -big           # block 1 (upper half-wave): positive first
    x[0, 2 * 256 + 8], x[0, 2 * 256 + 9] = -big, big             # block 2: both inside one lane's eight
    x[0, 3 * 256 + 100] = -big                                   # block 3: negative only
    x[0, 4 * 256:5 * 256] = 0.0                                  # block 4: all zero, block 5 not
    x[0, 6 * 256:7 * 256] = -0.0                                 # block 6: all minus zero
    x[0, 7 * 256 + 255] = big                                    # block 7: positive only, last element
    xd = dev(x)
    got = qh.quantize_act(orc.Q8K, xd).cpu().numpy()
    want = orc.quantize(orc.Q8K, x[0])
    assert got.size == want.size and np.array_equal(got, want)
    qw = qh.QWeight.from_ggml(dt, orc.quantize(dt, w), n, k)
    fused = qh.qmatmul(qw, xd)
    assert torch.equal(fused, qh.qmatmul(qw, xd, qh.FLAG_STAGED_ACT))
    check_f32(fused.cpu().numpy(), orc.matmul(dt, x, orc.quantize(dt, w), n))


def test_rounding_instruction_selfcheck(qh):
    """Every f32 in [-130, 130]: the device's one-instruction rounding equals round-half-away."""
    import ctypes as C
    bad = C.c_uint64(123)
    qh.check(qh.load().cq_selfcheck_round(0, C.byref(bad)))
    assert bad.value == 0


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q8_0])
@pytest.mark.parametrize("m", [2, 4, 8, 16])
@pytest.mark.parametrize("k,n", [(4096, 4096), (4096, 11008)])
def test_small_batch_matches_oracle(qh, dt, m, k, n):
    """BASELINE config 2: M in {2,4,8,16} on the decode shapes."""
    w, x = make_inputs(dt + m + n, m, k, n)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    got = qh.qmatmul(qw, dev(x)).cpu().numpy()
    check_f32(got, orc.matmul(dt, x, blocks, n))


@pytest.mark.parametrize("dt,m,n", [(orc.Q4K, 9, 11008), (orc.Q4K, 16, 14336), (orc.Q4K, 13, 16 * 1100), (orc.Q4K, 8, 16 * 800),
                                     (orc.Q4K, 16, 16 * 1025), (orc.Q5K, 5, 16 * 800), (orc.Q5K, 16, 11008), (orc.Q6K, 16, 11008),
                                     (orc.Q8_0, 16, 11008), (orc.Q8_0, 6, 16 * 1100), (orc.Q8_0, 12, 16 * 1025), (orc.Q4_0, 16, 11008),
                                     (orc.Q4_0, 7, 16 * 1100), (orc.Q4_0, 9, 16 * 1025), (orc.Q5_0, 16, 11008), (orc.Q4_1, 11, 11008)])
def test_small_batch_many_tiles_match_oracle(qh, dt, m, n):
    """5-16 rows against more 16-row weight tiles than compute units at K = 4096: two to five tiles per workgroup
    (rounds of four with one meeting each, a second round of a single tile), and the cases next to them that the
    per-block kernel takes."""
    check_many_tiles(qh, dt, m, 4096, n)


@pytest.mark.parametrize("dt,m,k,n", [(orc.Q4K, 16, 2560, 16 * 300), (orc.Q8_0, 9, 3840, 16 * 520), (orc.Q4_0, 16, 2304, 16 * 1030),
                                       (orc.Q4K, 12, 3328, 16 * 1100)])
def test_small_batch_many_tiles_fewer_k_blocks_than_waves(qh, dt, m, k, n):
    """The same with 9-15 K blocks: some of the sixteen waves own no block and only meet the others."""
    check_many_tiles(qh, dt, m, k, n)


def check_many_tiles(qh, dt, m, k, n):
    w, x = make_inputs(3 * dt + m + n + k, m, k, n, outliers=True)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    got = qh.qmatmul(qw, dev(x)).cpu().numpy()
    check_f32(got, orc.matmul(dt, x, blocks, n))
    # run-to-run: the partial tiles are summed in wave order
    again = qh.qmatmul(qw, dev(x)).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))


@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
@pytest.mark.parametrize("m,k,n", [(3, 512, 37), (5, 1024, 64), (7, 2048, 9), (9, 256, 130), (12, 11008, 24),
                                   (2, 256, 8), (8, 14336, 16), (70, 512, 48), (133, 256, 32)])
def test_ragged_batches_match_oracle(qh, dt, m, k, n):
    """Row counts that do not fill the 4- and 8-row batches of the dot-product kernels, weight row
    counts that are not a multiple of the waves per workgroup, the shortest rows (one K block) and
    rows longer than the single-launch decode path takes."""
    w, x = make_inputs(11 * dt + m + k + n, m, k, n, outliers=True)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    got = qh.qmatmul(qw, dev(x), qh.FLAG_FORCE_MATVEC).cpu().numpy()
    check_f32(got, orc.matmul(dt, x, blocks, n))
    # the same rows one at a time (decode kernel) give the same values: batch invariance
    one = np.concatenate([qh.qmatmul(qw, dev(x[r:r + 1])).cpu().numpy() for r in range(m)])
    check_f32(got, one)


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q5K, orc.Q6K])
@pytest.mark.parametrize("m,k,n", [(2, 256, 16), (3, 512, 48), (8, 4096, 64), (9, 1024, 32), (16, 2048, 80),
                                   (17, 768, 16), (24, 11008, 32), (32, 4096, 16), (33, 2304, 48), (5, 14336, 16)])
def test_skinny_matches_oracle(qh, dt, m, k, n):
    """The split-K MFMA kernel for few rows: every row-group count (1-4 groups of eight rows), more
    than 32 rows (two launches), fewer K blocks than waves, K blocks not a multiple of the waves."""
    w, x = make_inputs(17 * dt + m + k + n, m, k, n, outliers=True)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    got = qh.qmatmul(qw, dev(x), qh.FLAG_FORCE_SKINNY)
    check_f32(got.cpu().numpy(), orc.matmul(dt, x, blocks, n))
    assert torch.equal(got, qh.qmatmul(qw, dev(x), qh.FLAG_FORCE_SKINNY))   # deterministic: no atomics


@pytest.mark.parametrize("m,k,n", [(2, 256, 16), (3, 512, 48), (8, 4096, 64), (9, 1024, 32), (16, 2048, 80),
                                   (17, 768, 16), (24, 11008, 32), (32, 4096, 16), (33, 2304, 48), (5, 14336, 16)])
@pytest.mark.parametrize("dt", [orc.Q8_0, orc.Q4_0])
def test_skinny_q8_0_matches_oracle(qh, dt, m, k, n):
    """The split-K MFMA kernel for Q8_0 / Q4_0 weights and Q8_0 activations (one MFMA per 32-element
    block), on the same shapes; rows of whole 256-element groups only."""
    w, x = make_inputs(19 * dt + m + k + n, m, k, n, outliers=True)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    got = qh.qmatmul(qw, dev(x), qh.FLAG_FORCE_SKINNY)
    check_f32(got.cpu().numpy(), orc.matmul(dt, x, blocks, n))
    assert torch.equal(got, qh.qmatmul(qw, dev(x), qh.FLAG_FORCE_SKINNY))
    # from five to sixteen rows this kernel is the default choice (beyond, where n is no multiple of 32 and the tile
    # kernel does not take the weight); it agrees with the dot-product one
    if m >= 5 and (m <= 16 or n % 32):
        assert torch.equal(got, qh.qmatmul(qw, dev(x)))
    else:
        check_f32(got.cpu().numpy(), qh.qmatmul(qw, dev(x)).cpu().numpy())
    check_f32(got.cpu().numpy(), qh.qmatmul(qw, dev(x), qh.FLAG_FORCE_MATVEC).cpu().numpy())


def test_skinny_unsupported_shapes_are_refused(qh):
    """Q8_0 / Q4_0 rows that are not whole 256-element groups, n not a multiple of 16."""
    for dt, k, n in ((orc.Q8_0, 288, 16), (orc.Q4_0, 96, 16), (orc.Q4K, 256, 24)):
        w, x = make_inputs(5, 4, k, n)
        qw = qh.QWeight.from_ggml(dt, orc.quantize(dt, w), n, k)
        with pytest.raises(qh.QHipError):
            qh.qmatmul(qw, dev(x), qh.FLAG_FORCE_SKINNY)
        check_f32(qh.qmatmul(qw, dev(x)).cpu().numpy(), orc.matmul(dt, x, orc.quantize(dt, w), n))


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q5K, orc.Q6K])
def test_gemm_ragged_rows_large(qh, dt):
    """M = 300 (not a multiple of the 128-row workgroup tile) on a K-split shape: every output row
    of the tile kernel equals the dot-product kernels' result for that row within tolerance."""
    m, k, n = 300, 4096, 512
    w, x = make_inputs(13 * dt + 2, m, k, n, outliers=True)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    got = qh.qmatmul(qw, dev(x)).cpu().numpy()
    rows = [0, 1, 127, 128, 255, 256, 298, 299]
    want = orc.matmul(dt, x[rows], blocks, n)
    check_f32(got[rows], want)
    ref = qh.qmatmul(qw, dev(x), qh.FLAG_FORCE_MATVEC).cpu().numpy()
    check_f32(got, ref)


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q5K, orc.Q6K])
@pytest.mark.parametrize("m,k,n", [(9, 256, 32), (33, 512, 96), (64, 1024, 160), (130, 768, 288), (11, 512, 64),
                                   (1, 256, 32), (129, 2048, 416)])
def test_gemm_matches_oracle_small(qh, dt, m, k, n):
    """The int8-MFMA tile kernel on ragged shapes (m any, n a multiple of 32 but not of the
    128-row workgroup tile; from one K block up)."""
    w, x = make_inputs(3 * dt + m + k + n, m, k, n, outliers=True)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    got = qh.qmatmul(qw, dev(x), qh.FLAG_FORCE_GEMM).cpu().numpy()
    check_f32(got, orc.matmul(dt, x, blocks, n))


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q5K, orc.Q6K])
def test_gemm_needs_32_row_multiple(qh, dt):
    """Weight row counts that are not a multiple of 32 take the dot-product kernels: forcing the
    tile kernel is an error, the automatic choice still matches the oracle."""
    m, k, n = 33, 512, 70
    w, x = make_inputs(5 * dt + 1, m, k, n)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    with pytest.raises(qh.QHipError):
        qh.qmatmul(qw, dev(x), qh.FLAG_FORCE_GEMM)
    check_f32(qh.qmatmul(qw, dev(x)).cpu().numpy(), orc.matmul(dt, x, blocks, n))


@pytest.mark.parametrize("dt,m,k,n", [(orc.Q3K, 1, 4096, 32000), (orc.Q3K, 512, 4096, 14336), (orc.Q2K, 1, 11008, 4096),
                                      (orc.Q2K, 512, 14336, 4096), (orc.Q5_0, 16, 4096, 11008), (orc.Q5_0, 512, 4096, 14336),
                                      (orc.Q4_1, 1, 4096, 11008), (orc.Q5_1, 512, 4096, 4096), (orc.Q8K, 3, 4096, 4096)])
def test_other_weight_types_at_model_shapes(qh, dt, m, k, n):
    """The types that are held in another type's planes (and Q8K weights) at the shapes of the BASELINE configurations:
    weights quantized on the device, sampled weight rows (first, last, tile edges, random) over all activation rows
    against the oracle's own code for the type, and the bytes of the sampled rows against the oracle's quantizer."""
    rng = np.random.default_rng(k + n + int(dt))
    gen = torch.Generator(device="cuda").manual_seed(k + int(dt))
    wt = torch.randn((n, k), generator=gen, device="cuda") * 0.02
    qw = qh.QWeight.zeros(dt, n, k).quantize_(wt)
    x = rng.standard_normal((m, k)).astype(np.float32)
    idx = rng.choice(x.size, size=max(1, x.size // 100), replace=False)
    x.ravel()[idx] = np.where(rng.random(idx.size) < 0.5, -8.0, 8.0).astype(np.float32)
    got = qh.qmatmul(qw, dev(x)).cpu().numpy()
    rows = np.unique(np.concatenate([[0, 31, 32, 255, 256, n // 2, n - 257, n - 256, n - 33, n - 32, n - 1],
                                     rng.choice(n, size=21, replace=False)]))
    row_bytes = k // orc.BLOCK_SIZE[dt] * orc.TYPE_SIZE[dt]
    blocks = qw.to_ggml().reshape(n, row_bytes)[rows]
    assert np.array_equal(blocks.ravel(), orc.quantize(dt, wt[torch.from_numpy(rows).cuda()].cpu().numpy()))
    del wt
    ms = np.arange(m) if m <= 16 else np.unique(np.concatenate([[0, 31, 32, 127, 128, m - 1], rng.choice(m, size=10, replace=False)]))
    want = orc.matmul(dt, x[ms], blocks.ravel(), len(rows))
    g = got[np.ix_(ms, rows)].astype(np.float64)
    assert np.linalg.norm(g - want) <= REL_L2_TOL * np.linalg.norm(want)
    for i in range(len(ms)):
        nrm = np.linalg.norm(want[i])
        assert np.linalg.norm(g[i] - want[i]) <= REL_L2_TOL * nrm, (int(ms[i]), np.linalg.norm(g[i] - want[i]) / nrm)


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q5K, orc.Q6K])
@pytest.mark.parametrize("m,k,n", [(512, 4096, 14336), (512, 14336, 4096)])
def test_prefill_gemm_config3(qh, dt, m, k, n):
    """BASELINE config 3 at full size: M = 512 tokens on the Mistral FFN shapes, activations N(0,1)
    with 1% outliers at +-8 sigma.  Weights are quantized on the device (bit-identical to the CPU
    quantizer, checked above).  The oracle evaluates, over all 512 tokens, 96 weight rows: the first and the last
    row of the first, a middle and the last workgroup tile (256 weight rows each), of a wave's 32-row tile inside
    them, and random rows for the rest.  The whole 512 x n output is compared with the dot-product kernels
    (oracle-checked row by row above), so that no tile of the launch goes unseen."""
    rng = np.random.default_rng(k + dt)
    gen = torch.Generator(device="cuda").manual_seed(k + dt)
    wt = torch.randn((n, k), generator=gen, device="cuda") * 0.02
    qw = qh.QWeight.zeros(dt, n, k).quantize_(wt)
    del wt
    x = rng.standard_normal((m, k)).astype(np.float32)
    idx = rng.choice(x.size, size=x.size // 100, replace=False)
    x.ravel()[idx] = np.where(rng.random(idx.size) < 0.5, -8.0, 8.0).astype(np.float32)
    xd = dev(x)
    got_d = qh.qmatmul(qw, xd)                                  # m > 32: the tile kernel
    got = got_d.cpu().numpy()
    tiles = n // 256
    edge = []
    for t in (0, tiles // 2, tiles - 1):
        edge += [256 * t, 256 * t + 31, 256 * t + 32, 256 * t + 224, 256 * t + 255]
    rest = rng.choice(n, size=96 - len(edge), replace=False)
    rows = np.unique(np.concatenate([np.array(edge), rest]))
    row_bytes = k // 256 * orc.TYPE_SIZE[dt]
    blocks = qw.to_ggml().reshape(n, row_bytes)[rows].ravel()
    want = orc.matmul(dt, x, blocks, len(rows))
    g = got[:, rows].astype(np.float64)
    err = np.linalg.norm(g - want) / np.linalg.norm(want)
    assert err <= REL_L2_TOL, err
    for r in list(range(0, m, 37)) + [127, 128, m - 1]:          # with the edges of the 128-row activation tiles
        # max-abs bar, with ||row||_2 scaled from the sampled columns to the full row
        nrm = np.linalg.norm(want[r]) * np.sqrt(n / len(rows))
        assert np.abs(g[r] - want[r]).max() <= MAX_ABS_FACTOR * nrm
    # every element against the dot-product kernels: same integers, f32 sums in another order
    mv = qh.qmatmul(qw, xd, qh.FLAG_FORCE_MATVEC)
    diff = (got_d - mv).double()
    row_norm = mv.double().norm(dim=1)
    assert float((diff.norm(dim=1) / row_norm).max()) <= 1e-5
    assert float((diff.abs().amax(dim=1) / row_norm).max()) <= 1e-5


def test_reference_goldens_through_hip(qh, goldens, seeded_inputs):
    # quantized_tests.rs:49-64 and :109-129 (Q4_0, m=3, k=64, n=4)
    m, k, n = 3, 64, 4
    lhs = np.arange(m * k, dtype=np.float32).reshape(m, k)
    rhs = np.arange(k * n, dtype=np.float32).reshape(n, k)
    qw = qh.QWeight.from_ggml(orc.Q4_0, orc.quantize(orc.Q4_0, rhs), n, k)
    got = qh.qmatmul(qw, dev(lhs)).cpu().numpy()
    assert np.round(got).ravel().tolist() == goldens["q4_0_matmul_m3_k64_n4"]["rounded"]
    lhs = (np.arange(m * k, dtype=np.float32) - np.float32(m * k) / 2).reshape(m, k)
    rhs = (np.arange(k * n, dtype=np.float32) - np.float32(k * n) / np.float32(3.0)).reshape(n, k)
    qw = qh.QWeight.from_ggml(orc.Q4_0, orc.quantize(orc.Q4_0, rhs), n, k)
    got = qh.qmatmul(qw, dev(lhs)).cpu().numpy()
    assert np.round(got).ravel().tolist() == goldens["q4_0_matmul_neg_m3_k64_n4"]["rounded"]
    # quantized_tests.rs:998-1151 (seeded m=11, k=512, n=21), weights quantized on the device
    g = goldens["seeded_matmul_m11_k512_n21"]
    lhs, rhs = seeded_inputs
    for name, dt in (("q2k", orc.Q2K), ("q3k", orc.Q3K), ("q4k", orc.Q4K), ("q5k", orc.Q5K), ("q6k", orc.Q6K)):
        qw = qh.QWeight.zeros(dt, 21, 512).quantize_(dev(rhs))
        out = qh.qmatmul(qw, dev(lhs)).cpu().numpy().ravel()
        spot = [float(np.round(np.float32(1000.0) * out[i]) / np.float32(1000.0)) for i in g["flat_indices"]]
        assert spot == [float(np.float32(v)) for v in g[name]], (name, spot)


@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
def test_batch_invariance(qh, dt, seeded_inputs):
    """quantized_tests.rs:181-216: a row's result does not depend on how many rows are stacked."""
    lhs, rhs = seeded_inputs
    lhs, rhs = lhs[:2, :256], rhs[:6, :256]
    qw = qh.QWeight.from_ggml(dt, orc.quantize(dt, rhs), 6, 256)
    mm = qh.qmatmul(qw, dev(lhs), qh.FLAG_FORCE_MATVEC).cpu().numpy()
    for reps in (2, 3, 6):
        mmr = qh.qmatmul(qw, dev(np.concatenate([lhs] * reps)), qh.FLAG_FORCE_MATVEC).cpu().numpy()
        for r in range(reps):
            assert np.array_equal(mmr[2 * r:2 * r + 2], mm)


def test_forward_shape_and_errors(qh):
    w, x = make_inputs(5, 6, 256, 8)
    qw = qh.QWeight.from_ggml(orc.Q4K, orc.quantize(orc.Q4K, w), 8, 256)
    x3 = dev(x.reshape(2, 3, 256))
    y = qh.qmatmul(qw, x3)
    assert tuple(y.shape) == (2, 3, 8)                       # last dim replaced by n (mod.rs:483-489)
    assert torch.equal(y.reshape(6, 8), qh.qmatmul(qw, dev(x)))
    with pytest.raises(qh.QHipError):                        # mod.rs:485-487
        qh.qmatmul(qw, torch.zeros((2, 512), device="cuda"))
    with pytest.raises(qh.QHipError):                        # mod.rs:480-482
        qh.qmatmul(qw, torch.zeros((256,), device="cuda"))
    with pytest.raises(qh.QHipError):                        # mod.rs:474-476
        qh.qmatmul(qw, torch.zeros((256, 4), device="cuda").t())
    assert tuple(qh.qmatmul(qw, torch.zeros((0, 256), device="cuda")).shape) == (0, 8)


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q5K, orc.Q6K])
@pytest.mark.parametrize("m,k,n", [(300, 256 * 7, 1056), (512, 4096, 4096), (130, 256 * 3, 160), (65, 256 * 2, 128),
                                   (200, 256 * 9, 2048 + 96), (96, 256 * 16, 512)])
def test_prefill_few_weight_rows_long_k(qh, dt, m, k, n):
    """Few column tiles and a long K: the launches that halve K between the waves of a workgroup (odd block counts:
    unequal halves; 2 and 3 blocks; weight row counts that leave waves of the last workgroup without rows; ragged
    activation rows) - against the oracle, and bit for bit the same on a second call."""
    w, x = make_inputs(17 * dt + m + k + n, m, k, n, outliers=True)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    got = qh.qmatmul(qw, dev(x)).cpu().numpy()
    check_f32(got, orc.matmul(dt, x, blocks, n))
    again = qh.qmatmul(qw, dev(x), qh.FLAG_DETERMINISTIC).cpu().numpy()
    check_f32(again, got)
    third = qh.qmatmul(qw, dev(x), qh.FLAG_DETERMINISTIC).cpu().numpy()
    assert np.array_equal(again.view(np.uint32), third.view(np.uint32))


@pytest.mark.parametrize("dt,m,k,n", [(orc.Q4K, 17, 4096, 14336), (orc.Q4K, 24, 4096, 14304), (orc.Q6K, 32, 4096, 12288),
                                       (orc.Q5K, 25, 4096, 12256), (orc.Q4K, 48, 8192, 4096), (orc.Q6K, 64, 6144, 4096),
                                       (orc.Q8_0, 17, 4096, 12288), (orc.Q4_0, 32, 4096, 12288), (orc.Q8_0, 24, 2048, 24576),
                                       (orc.Q4_0, 21, 4096, 12256), (orc.Q4_0, 29, 4096, 20480), (orc.Q8_0, 3, 11008, 4096), (orc.Q4_0, 4, 11008, 512),
                                       (orc.Q8_0, 2, 256 * 400, 64)])
def test_kernel_choice_at_its_row_count_limits(qh, dt, m, k, n):
    """Shapes either side of the limits at which a call goes to the split-K kernel, a tile kernel or a dot-product
    kernel (17-32 rows against many weight rows; 33-64 rows against few weight rows with a long K; 2-4 rows of
    Q8_0 / Q4_0 whose weight rows are too long for the one-launch kernel): the call's own choice against 40 sampled
    weight rows of the oracle and against every kernel that can be forced on the same shape."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7 * dt + m + n)
    w = torch.randn((n, k), generator=gen, device="cuda", dtype=torch.float32) * 0.02
    x = torch.randn((m, k), generator=gen, device="cuda", dtype=torch.float32)
    qw = qh.QWeight.zeros(dt, n, k).quantize_(w)
    got = qh.qmatmul(qw, x)
    rows = np.random.default_rng(n + m).choice(n, 40, replace=False)
    blocks = qw.to_ggml().reshape(n, -1)
    want = orc.matmul(dt, x.cpu().numpy(), np.ascontiguousarray(blocks[rows]).ravel(), len(rows))
    check_f32(got.cpu().numpy()[:, rows], want)
    forced = 0
    for flag in (qh.FLAG_FORCE_SKINNY, qh.FLAG_FORCE_GEMM, qh.FLAG_FORCE_MATVEC):
        try:
            other = qh.qmatmul(qw, x, flag)
        except qh.QHipError:
            continue   # that kernel does not take the shape
        forced += 1
        assert torch.allclose(got, other, rtol=3e-5, atol=3e-5), flag
    assert forced >= 2


# ------------------------------------------------------------------------- MoE ----
@pytest.mark.parametrize("tokens,starve", [(24, False), (64, True)])
def test_moe_ffn_matches_oracle(qh, tokens, starve):
    """Mixtral-shaped expert FFN at reduced width: routed top-2, per-expert gathered QMatMul,
    silu(w1 x) * w3 x, w2, scaled scatter-add (quantized_llama.rs:75-143).  24 tokens keep every
    expert on the dot-product kernels (at most 8 rows each); 64 tokens (BASELINE config 4's count)
    with one expert that no token picks give experts on the tile kernel and an empty slice."""
    rng = np.random.default_rng(23 + tokens)
    hidden, ffn, n_e, top_k = 512, 1024, 8, 2
    xs = rng.standard_normal((tokens, hidden)).astype(np.float32)
    logits = rng.standard_normal((tokens, n_e)).astype(np.float32)
    if starve:
        logits[:, 5] = -30.0
    offsets, row_ids, weights = orc.moe_route(orc.softmax_last_dim(logits), top_k)
    if starve:
        assert offsets[6] == offsets[5] and max(np.diff(offsets)) > 8
    w1 = [orc.quantize(orc.Q4K, (rng.standard_normal((ffn, hidden)) * 0.05).astype(np.float32)) for _ in range(n_e)]
    w3 = [orc.quantize(orc.Q4K, (rng.standard_normal((ffn, hidden)) * 0.05).astype(np.float32)) for _ in range(n_e)]
    w2 = [orc.quantize(orc.Q6K, (rng.standard_normal((hidden, ffn)) * 0.05).astype(np.float32)) for _ in range(n_e)]
    want = orc.moe_ffn(orc.Q4K, orc.Q6K, w1, w2, w3, hidden, ffn, xs, offsets, row_ids, weights)
    q1 = [qh.QWeight.from_ggml(orc.Q4K, b, ffn, hidden) for b in w1]
    q3 = [qh.QWeight.from_ggml(orc.Q4K, b, ffn, hidden) for b in w3]
    q2 = [qh.QWeight.from_ggml(orc.Q6K, b, hidden, ffn) for b in w2]
    x_d, rid_d, wt_d = dev(xs), dev(row_ids), dev(weights)
    h1 = qh.qmatmul_grouped(q1, x_d, rid_d, offsets)
    h3 = qh.qmatmul_grouped(q3, x_d, rid_d, offsets)
    # w3 on the rows the workspace already holds (quantized for w1 / w3 just now): no second quantizer launch
    assert torch.allclose(h3, qh.qmatmul_grouped(q3, x_d, rid_d, offsets, flags=qh.FLAG_REUSE_ACT), rtol=1e-5, atol=1e-5)
    h = qh.silu_mul(h1, h3)
    y = qh.qmatmul_grouped(q2, h, None, offsets)
    ys = qh.moe_scatter_add(y, rid_d, wt_d, tokens).cpu().numpy()
    # Stage by stage against the oracle.  The second matmul re-quantizes h; a 1-ulp difference
    # between the device expf and libm's can move one int8 activation across a rounding boundary
    # (an error of ~1e-3 of that row), so stage 3 feeds the oracle the device's own h.
    h1n, h3n, hn, yn = (t.cpu().numpy() for t in (h1, h3, h, y))
    for e in range(n_e):
        sl = slice(offsets[e], offsets[e + 1])
        if sl.start == sl.stop:
            continue
        cur = xs[row_ids[sl]]
        check_f32(h1n[sl], orc.matmul(orc.Q4K, cur, w1[e], ffn))
        check_f32(h3n[sl], orc.matmul(orc.Q4K, cur, w3[e], ffn))
        check_f32(yn[sl], orc.matmul(orc.Q6K, hn[sl], w2[e], hidden))
    silu = h1n.astype(np.float64) / (1.0 + np.exp(-h1n.astype(np.float64))) * h3n
    assert np.abs(hn - silu).max() <= 1e-6 * np.abs(silu).max()
    acc = np.zeros((tokens, hidden), np.float32)
    for p in range(offsets[-1]):               # sequential index_add in expert order
        acc[row_ids[p]] += yn[p] * weights[p]
    assert np.array_equal(ys, acc)
    # end to end: only as loose as the re-quantization effect described above
    assert np.linalg.norm(ys - want) / np.linalg.norm(want) < 5e-3


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_grouped_random_shapes_match_oracle(qh, seed):
    """The grouped launch over random expert slices (empty ones, more than one 32-row tile, a single row), 1-9 K blocks
    (fewer blocks than the copies run ahead, odd counts, K split over workgroups or not) and weight row counts that
    leave waves of the last workgroup without rows: every slice against the oracle's matmul with its expert."""
    rng = np.random.default_rng(100 + seed)
    dt = [orc.Q4K, orc.Q5K, orc.Q6K][seed % 3]
    k = 256 * int(rng.integers(1, 10))
    n = 32 * int(rng.integers(1, 14))
    n_e = int(rng.integers(1, 7))
    rows = [int(rng.choice([0, 1, 5, 16, 17, 31, 32, 33, 45])) for _ in range(n_e)]
    offsets = np.concatenate([[0], np.cumsum(rows)]).astype(np.int32)
    total = int(offsets[-1])
    if total == 0:
        rows[0] = 7
        offsets = np.concatenate([[0], np.cumsum(rows)]).astype(np.int32)
        total = int(offsets[-1])
    blocks = [orc.quantize(dt, (rng.standard_normal((n, k)) * 0.03).astype(np.float32)) for _ in range(n_e)]
    experts = [qh.QWeight.from_ggml(dt, b, n, k) for b in blocks]
    tokens = 19
    x = rng.standard_normal((tokens, k)).astype(np.float32)
    rid = rng.integers(0, tokens, size=total).astype(np.int32)
    y = qh.qmatmul_grouped(experts, dev(x), torch.from_numpy(rid).cuda(), offsets).cpu().numpy()
    for e in range(n_e):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if lo < hi:
            check_f32(y[lo:hi], orc.matmul(dt, x[rid[lo:hi]], blocks[e], n))


@pytest.mark.parametrize("tokens,total,hidden", [(5, 9, 6), (7, 200, 8), (64, 128, 4096), (3, 70, 1028), (4, 0, 16)])
def test_moe_scatter_add_order_and_shapes(qh, tokens, total, hidden):
    """ys[row_ids[p]] += weights[p] * y[p] for p in increasing order (cpu_backend/mod.rs:619-653): both
    kernels (hidden a multiple of 4 or not), more rows than one 64-row search step, tokens that
    receive nothing, no rows at all.  Sums are compared bit for bit with the same sequential loop."""
    rng = np.random.default_rng(tokens * 1000 + total)
    y = rng.standard_normal((total, hidden)).astype(np.float32)
    rid = rng.integers(0, max(tokens - 1, 1), size=total).astype(np.int32)     # the last token gets no row
    wt = rng.random(total).astype(np.float32)
    want = np.zeros((tokens, hidden), np.float32)
    for p in range(total):
        want[rid[p]] = want[rid[p]] + y[p] * wt[p]
    y_d = dev(y) if total else torch.zeros((0, hidden), device="cuda")
    rid_d = dev(rid) if total else torch.zeros((0,), dtype=torch.int32, device="cuda")
    wt_d = dev(wt) if total else torch.zeros((0,), device="cuda")
    got = qh.moe_scatter_add(y_d, rid_d, wt_d, tokens).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_moe_config4_full_size(qh):
    """BASELINE config 4 at its real shape: 8 experts of w1/w3 [14336 x 4096] Q4K and w2 [4096 x 14336]
    Q6K, 64 tokens routed top-2.  The oracle would need minutes for all of it, so: every expert's
    slice of each grouped launch is compared with the plain tile kernel on the same rows (the same
    workgroup body without the tile table), a sample of weight rows of every expert with the
    oracle, and the combine with the sequential index_add."""
    hidden, ffn, n_e, tokens, top_k = 4096, 14336, 8, 64, 2
    rng = np.random.default_rng(4)
    gen = torch.Generator(device="cuda")
    xs = rng.standard_normal((tokens, hidden)).astype(np.float32)
    logits = rng.standard_normal((tokens, n_e)).astype(np.float32)
    offsets, row_ids, weights = orc.moe_route(orc.softmax_last_dim(logits), top_k)
    assert offsets[-1] == tokens * top_k

    def make(dt, n, k, seed):
        gen.manual_seed(seed)
        w = torch.randn((n, k), generator=gen, device="cuda", dtype=torch.float32) * 0.02
        return qh.QWeight.zeros(dt, n, k).quantize_(w)

    q1 = [make(orc.Q4K, ffn, hidden, 100 + e) for e in range(n_e)]
    q3 = [make(orc.Q4K, ffn, hidden, 200 + e) for e in range(n_e)]
    q2 = [make(orc.Q6K, hidden, ffn, 300 + e) for e in range(n_e)]
    x_d, rid_d, wt_d = dev(xs), dev(row_ids), dev(weights)
    h1 = qh.qmatmul_grouped(q1, x_d, rid_d, offsets)
    h3 = qh.qmatmul_grouped(q3, x_d, rid_d, offsets)
    assert torch.equal(h3, qh.qmatmul_grouped(q3, x_d, rid_d, offsets, flags=qh.FLAG_REUSE_ACT))   # (no K split at 14336 rows)
    with pytest.raises(qh.QHipError, match="exclude each other"):
        qh.qmatmul_grouped(q2, h1, None, offsets, flags=qh.FLAG_REUSE_ACT, pre=qh.PRE_SILU_MUL, aux=h3)
    h = qh.silu_mul(h1, h3)
    y = qh.qmatmul_grouped(q2, h, None, offsets)
    y_fused = qh.qmatmul_grouped(q2, h1, None, offsets, pre=qh.PRE_SILU_MUL, aux=h3)
    assert torch.allclose(y, y_fused, rtol=1e-5, atol=1e-5)   # w2 splits K: partial sums are added in any order
    ys = qh.moe_scatter_add(y, rid_d, wt_d, tokens)
    hn, yn = h.cpu().numpy(), y.cpu().numpy()
    sample13 = rng.choice(ffn, 24, replace=False)
    sample2 = rng.choice(hidden, 24, replace=False)
    for e in range(n_e):
        sl = slice(int(offsets[e]), int(offsets[e + 1]))
        if sl.start == sl.stop:
            continue
        cur = xs[row_ids[sl]]
        cur_d = dev(cur)
        # grouped launch == plain tile kernel on the expert's rows, up to the order in which the partial
        # sums of a split K are added (a lone expert's launch splits K to fill the machine)
        for got, qs, inp in ((h1, q1, cur_d), (h3, q3, cur_d), (y, q2, h[sl].contiguous())):
            assert torch.allclose(got[sl], qh.qmatmul(qs[e], inp, qh.FLAG_FORCE_GEMM), rtol=1e-5, atol=1e-5), e
        # sampled weight rows against the oracle (GGML rows are independent: a row's blocks are a matrix of one row)
        for qs, inp, got, k, rows in ((q1, cur, h1, hidden, sample13), (q3, cur, h3, hidden, sample13),
                                      (q2, hn[sl], y, ffn, sample2)):
            blocks = qs[e].to_ggml().reshape(qs[e].shape[0], -1)
            sub = np.ascontiguousarray(blocks[rows]).ravel()
            want = orc.matmul(qs[e].dtype, inp, sub, len(rows))
            have = got[sl].cpu().numpy()[:, rows]
            assert np.linalg.norm(have - want) <= REL_L2_TOL * np.linalg.norm(want), e
    acc = np.zeros((tokens, hidden), np.float32)
    for p in range(offsets[-1]):               # sequential index_add in expert order
        acc[row_ids[p]] += yn[p] * weights[p]
    assert np.array_equal(ys.cpu().numpy(), acc)


# ------------------------------------- tile kernel of the 32-element-block types (Q8_0, Q4_0) ----
@pytest.mark.parametrize("dt", [orc.Q8_0, orc.Q4_0])
@pytest.mark.parametrize("m,k,n", [(17, 512, 32), (32, 4096, 96), (33, 256, 32), (64, 512, 64), (70, 1024, 96), (130, 768, 288),
                                   (200, 2048, 32), (129, 4096, 64)])
def test_gemm_blk32_matches_oracle(qh, dt, m, k, n):
    """More than 16 rows of Q8_0 / Q4_0 weights go to their own int8-MFMA tile kernel (one MFMA result per
    32-element block, scaled by the two block scales): ragged row counts, one and several K steps,
    split K (few workgroups), against the oracle and against the split-K kernel on the same workspace."""
    w, x = make_inputs(3 * dt + m + k, m, k, n, outliers=True)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    got = qh.qmatmul(qw, dev(x))
    check_f32(got.cpu().numpy(), orc.matmul(dt, x, blocks, n))
    other = qh.qmatmul(qw, dev(x), qh.FLAG_FORCE_SKINNY)
    assert torch.allclose(got, other, rtol=2e-5, atol=1e-5)


@pytest.mark.parametrize("dt", [orc.Q8_0, orc.Q4_0])
def test_gemm_blk32_full_size(qh, dt):
    """M = 512 on 4096 x 4096: every output against the split-K kernel (a different kernel, the same
    integers), 48 sampled weight rows against the oracle, and batch invariance against the decode kernel."""
    m, k, n = 512, 4096, 4096
    gen = torch.Generator(device="cuda")
    gen.manual_seed(31 + dt)
    w = torch.randn((n, k), generator=gen, device="cuda", dtype=torch.float32) * 0.02
    x = torch.randn((m, k), generator=gen, device="cuda", dtype=torch.float32)
    qw = qh.QWeight.zeros(dt, n, k).quantize_(w)
    got = qh.qmatmul(qw, x)
    other = qh.qmatmul(qw, x, qh.FLAG_FORCE_SKINNY)
    assert torch.allclose(got, other, rtol=2e-5, atol=2e-5)
    rows = np.random.default_rng(5).choice(n, 48, replace=False)
    blocks = qw.to_ggml().reshape(n, -1)
    want = orc.matmul(dt, x.cpu().numpy(), np.ascontiguousarray(blocks[rows]).ravel(), len(rows))
    check_f32(got.cpu().numpy()[:, rows], want)
    one = qh.qmatmul(qw, x[7:8].contiguous())
    assert torch.allclose(got[7:8], one, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q6K, orc.Q8_0, orc.Q4_0])
def test_split_k_output_is_cleared_wherever_it_lives(qh, dt):
    """Launches that split K add into a zeroed output.  The activation quantizer clears it on its way
    when the output does not overlap the input and takes 16-byte stores; otherwise a fill launch does.
    All three ways give the oracle's result on an output that held NaNs: a fresh buffer, one that is
    not 16-byte aligned, and the input's own memory (n == k, computed in place)."""
    m, k, n = 48, 2048, 2048            # 8 x 1 tiles on 256 CUs: K is split
    w, x = make_inputs(40 + dt, m, k, n)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    want = orc.matmul(dt, x, blocks, n)
    flags = qh.FLAG_FORCE_GEMM if dt in (orc.Q4K, orc.Q6K) else 0
    xd = dev(x)
    y = torch.full((m, n), float("nan"), device="cuda")
    qh.qmatmul(qw, xd, flags, out=y)
    check_f32(y.cpu().numpy(), want)
    buf = torch.full((m * n + 4,), float("nan"), device="cuda")
    y1 = buf[1:1 + m * n].view(m, n)    # 4 bytes past a 16-byte boundary
    qh.qmatmul(qw, xd, flags, out=y1)
    assert torch.allclose(y1, y, rtol=1e-5, atol=1e-6)
    assert torch.isnan(buf[0]) and torch.isnan(buf[1 + m * n:]).all()
    xin = xd.clone()
    qh.qmatmul(qw, xin, flags, out=xin)  # in place
    assert torch.allclose(xin, y, rtol=1e-5, atol=1e-6)
    # the rows reused from the workspace: nothing is quantized, so the fill launch clears
    y2 = torch.full((m, n), float("nan"), device="cuda")
    qh.qmatmul(qw, xd, flags, out=y)
    qh.qmatmul(qw, xd, flags | qh.FLAG_REUSE_ACT, out=y2)
    assert torch.allclose(y2, y, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q6K, orc.Q8_0, orc.Q4_0])
@pytest.mark.parametrize("m,k,n", [(40, 1024, 1024), (100, 2048, 4096), (300, 1024, 4096), (520, 1024, 2048),
                                   (130, 4096, 11008), (1000, 512, 8192), (4100, 1024, 1024), (48, 512, 40000)])
def test_tile_plans_agree_with_dot_product_kernels(qh, dt, m, k, n):
    """The tile kernels pick tile height and K split per shape; whatever they pick, the result equals the
    dot-product kernels' (which the tests above hold against the oracle) to rounding, and a sample of
    weight rows is held against the oracle directly."""
    rng = np.random.default_rng(m + k + n + dt)
    gen = torch.Generator(device="cuda").manual_seed(m + k + n + dt)
    wt = torch.randn((n, k), generator=gen, device="cuda") * 0.02
    qw = qh.QWeight.zeros(dt, n, k).quantize_(wt)
    del wt
    x = rng.standard_normal((m, k)).astype(np.float32)
    xd = dev(x)
    got = qh.qmatmul(qw, xd)
    ref = qh.qmatmul(qw, xd, qh.FLAG_FORCE_MATVEC)
    err = (torch.linalg.norm(got - ref) / torch.linalg.norm(ref)).item()
    assert err <= 2e-6, err
    rows = np.sort(rng.choice(n, size=16, replace=False))
    row_bytes = k // orc.BLOCK_SIZE[dt] * orc.TYPE_SIZE[dt]
    blocks = qw.to_ggml().reshape(n, row_bytes)[rows].ravel()
    want = orc.matmul(dt, x, blocks, len(rows))
    g = got.cpu().numpy()[:, rows].astype(np.float64)
    assert np.linalg.norm(g - want) / np.linalg.norm(want) <= REL_L2_TOL


@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
@pytest.mark.parametrize("m,k,n", [(2, 4096, 264), (3, 2048, 77), (4, 1024, 4096), (2, 8192, 64), (3, 8192, 40), (2, 11008, 72),
                                   (3, 11008, 72)])
def test_few_rows_one_launch_equals_single_rows(qh, dt, m, k, n):
    """Two to four activation rows on short enough weight rows go through the one-launch decode kernel:
    every output row has the bits of its own one-row call (same order of operations per row), and the
    two-launch path (quantizer + matmul kernel) agrees to rounding; longer rows stay on the two-launch path
    and still match."""
    w, x = make_inputs(7 * dt + m + k + n, m, k, n, outliers=True)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    xd = dev(x)
    got = qh.qmatmul(qw, xd)
    elems = {orc.Q4_0: 32, orc.Q4_1: 16, orc.Q5_0: 16, orc.Q5_1: 16, orc.Q8_0: 16, orc.Q2K: 32, orc.Q3K: 32, orc.Q4K: 64, orc.Q5K: 64, orc.Q6K: 32}[dt]   # weights per 16-byte lane unit
    units = k // elems
    per_lane = -(-units // 64) * elems
    if units <= (384 if m == 2 else 256) and (per_lane <= 64 or (per_lane <= 128 and m <= 3) or m <= 2):   # the library's rule
        for r in range(m):
            assert torch.equal(got[r:r + 1], qh.qmatmul(qw, xd[r:r + 1].contiguous())), r
    two = qh.qmatmul(qw, xd, qh.FLAG_STAGED_ACT)
    assert (torch.linalg.norm(got - two) / torch.linalg.norm(two)).item() <= 2e-6
    check_f32(got.cpu().numpy(), orc.matmul(dt, x, blocks, n))


@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("dt,k,n", [(dt, k, n) for dt in (orc.Q4_1, orc.Q5_1, orc.Q2K)
                                    for k, n in [(256, 8), (512, 40), (2048, 64), (4096, 300), (11008, 24), (14336, 16),
                                                 (64, 16), (192, 33), (1088, 64), (4160, 48)]
                                    if dt != orc.Q2K or k % 256 == 0])
def test_offset_types_one_launch_equals_workspace_path(qh, dt, m, k, n):
    """Q4_1 / Q5_1 / Q2K: the one-launch kernels add the offset term (block minima times the activation blocks' scaled
    sums) themselves; the other paths add it in a second launch over the quantized rows in the workspace.  Same
    operations in the same order: equal bits at one row.  Row lengths with whole and partial groups of eight 32-element blocks,
    one and several passes of 64 lanes over the blocks (an even number of blocks: the reference takes no other)."""
    w, x = make_inputs(23 * dt + m + k + n, m, k, n, outliers=True)
    w = w + 0.5 * np.abs(w).mean()          # offsets that matter
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    xd = dev(x)
    got = qh.qmatmul(qw, xd)
    two = qh.qmatmul(qw, xd, qh.FLAG_STAGED_ACT)
    if m == 1:
        assert torch.equal(got, two)
    else:   # several rows: the kernels behind the workspace add up the main term in another order
        assert (torch.linalg.norm(got - two) / torch.linalg.norm(two)).item() <= 2e-6
    check_f32(got.cpu().numpy(), orc.matmul(dt, x, blocks, n))


# ------------------------------------------------------------- seeded random shapes ----
def _random_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(count):
        dt = int(rng.choice(WEIGHT_DTYPES))
        blk = 32 if dt in (orc.Q4_0, orc.Q4_1, orc.Q5_0, orc.Q5_1, orc.Q8_0) else 256
        k = blk * int(rng.integers(1, (2048 // blk) + 1))
        m = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 32, 33, 40, 64, 65, 70]))
        n = int(rng.choice([1, 2, 7, 8, 15, 16, 17, 31, 32, 33, 48, 63, 64, 96, 100, 128, 255, 256, 257, 300]))
        cases.append((dt, m, k, n))
    return cases


@pytest.mark.parametrize("dt,m,k,n", _random_cases(96, 20240611))
def test_random_shapes_match_oracle(qh, dt, m, k, n):
    """Whatever kernel the automatic choice lands on for a shape (one-launch decode, several rows in one launch,
    split-K, tile, dot-product fallbacks for ragged n and k): every row against the oracle at the usual bars."""
    w, x = make_inputs(dt * 1000003 + m * 10007 + k * 101 + n, m, k, n, outliers=True)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    if dt in (orc.Q4_1, orc.Q5_0, orc.Q5_1) and (k // 32) % 2:
        # the reference's vec_dot of these types refuses an odd number of blocks (k_quants.rs:273, 363, 469)
        with pytest.raises(ValueError):
            orc.matmul(dt, x, blocks, n)
        with pytest.raises(qh.QHipError, match="not divisible by 2"):
            qh.qmatmul(qw, dev(x))
        return
    check_f32(qh.qmatmul(qw, dev(x)).cpu().numpy(), orc.matmul(dt, x, blocks, n))


def _pattern_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        dt = int(rng.choice(WEIGHT_DTYPES + [orc.Q8K]))
        blk = 32 if dt in (orc.Q4_0, orc.Q4_1, orc.Q5_0, orc.Q5_1, orc.Q8_0) else 256
        k = blk * (2 * int(rng.integers(1, 33)) if blk == 32 else int(rng.choice([1, 2, 3, 5, 8, 16, 43])))
        m = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 16, 17, 33, 64, 65, 129]))
        n = int(rng.choice([1, 7, 8, 16, 31, 32, 33, 64, 100, 128, 257]))
        cases.append((dt, m, k, n, i % 4))
    return cases


@pytest.mark.parametrize("dt,m,k,n,kind", _pattern_cases(64, 20250117))
def test_input_patterns_match_oracle(qh, dt, m, k, n, kind):
    """Inputs that exercise the quantizers' special cases rather than their typical ones, through whatever kernel the
    automatic choice and the forced dot-product path land on: all-zero rows, blocks and weight rows and a row with a
    single non-zero (scale 0 / one live quant); equal magnitudes with both signs (the first-index rules of the
    maximum searches) and constant blocks; positive weights with large minima against a ramp; scales 0.01 - 100."""
    rng = np.random.default_rng(dt * 7919 + m * 131 + k + n + kind)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    if kind == 0:
        x[rng.integers(0, m)] = 0
        x[:, :min(k, 256)] = 0
        r = rng.integers(0, m)
        x[r] = 0
        x[r, rng.integers(0, k)] = -3.0
        w[rng.integers(0, n)] = 0
    elif kind == 1:
        x = np.where(rng.random((m, k)) < 0.5, -1.5, 1.5).astype(np.float32)
        w = np.where(rng.random((n, k)) < 0.5, -0.25, 0.25).astype(np.float32) + np.float32(0.125 * (n % 2))
    elif kind == 2:
        w = np.abs(w) + np.float32(0.05)
        x = ((np.arange(m * k, dtype=np.float32).reshape(m, k) % 97) - 48) / 16
    else:
        x *= np.float32(10.0 ** int(rng.integers(-2, 3)))
        w *= np.float32(10.0 ** int(rng.integers(-2, 2)))
    blocks = orc.quantize(dt, w)
    ref = orc.matmul(dt, x, blocks, n)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    assert np.array_equal(qh.QWeight.zeros(dt, n, k).quantize_(dev(w)).to_ggml(), blocks)   # device quantizer: same bytes
    ref64 = ref.astype(np.float64)
    for flags in (0, qh.FLAG_FORCE_MATVEC):
        got = qh.qmatmul(qw, dev(x), flags).cpu().numpy()
        if n >= 32:
            check_f32(got, ref)
        else:   # a handful of outputs per row, some of them sums that nearly cancel: the bar over the whole result
            assert np.isfinite(got).all()
            assert np.linalg.norm(got - ref64) <= REL_L2_TOL * np.linalg.norm(ref64)
        assert not got[~x.any(axis=1)].any()          # a row of zeros gives zeros, offsets or not


@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
@pytest.mark.parametrize("m", [1, 3, 9])
def test_nan_activations_follow_the_reference(qh, dt, m):
    """The reference's maximum searches skip NaN (comparisons with it are false) and its casts turn NaN into 0, so
    activations with NaN give numbers, not NaN - unless a scale becomes infinite.  Isolated NaN, a run of NaN that fills
    whole lanes of the quantizers (eight, sixteen, thirty-two in a row), a block of NaN and a row of NaN, through the
    one-launch kernels (one and three rows) and the workspace path: finite where the oracle is finite, the same
    values."""
    rng = np.random.default_rng(100 * int(dt) + m)
    k, n = 1024, 40
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[0, [3, 77, 500]] = np.nan
    x[0, 256:264] = np.nan
    x[0, 320:336] = np.nan
    x[0, 512:544] = np.nan
    x[0, 768:1024] = np.nan
    if m > 1:
        x[1, :] = np.nan
    blocks = orc.quantize(dt, w)
    ref = orc.matmul(dt, x, blocks, n)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    for flags in (0, qh.FLAG_STAGED_ACT, qh.FLAG_FORCE_MATVEC):
        got = qh.qmatmul(qw, dev(x), flags).cpu().numpy()
        fin = np.isfinite(ref)
        assert np.array_equal(np.isfinite(got), fin), flags
        assert np.linalg.norm((got - ref)[fin]) <= REL_L2_TOL * np.linalg.norm(ref[fin]), flags


# byte offsets of the f16 fields of a block (k_quants.rs:42-155)
_F16_FIELDS = {orc.Q4_0: [0], orc.Q4_1: [0, 2], orc.Q5_0: [0], orc.Q5_1: [0, 2], orc.Q8_0: [0], orc.Q2K: [80, 82],
               orc.Q3K: [108], orc.Q4K: [0, 2], orc.Q5K: [0, 2], orc.Q6K: [208]}


def _byte_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        dt = WEIGHT_DTYPES[i % len(WEIGHT_DTYPES)]
        kb = int(rng.choice([16, 32, 64])) if orc.BLOCK_SIZE[dt] == 32 else int(rng.choice([1, 2, 3, 8]))
        cases.append((dt, int(rng.choice([1, 3, 8, 17, 40, 130])), kb * orc.BLOCK_SIZE[dt], int(rng.choice([16, 48, 100])), i % 3))
    return cases


@pytest.mark.parametrize("dt,m,k,n,mode", _byte_cases(60, 77))
def test_weights_from_arbitrary_bytes(qh, dt, m, k, n, mode):
    """Blocks no quantizer would write: every integer field random, all ones, or at the corners 0x00 / 0x7f / 0x80 / 0xff
    (six-bit scales of 63, Q6K scales of -128, Q8_0 quants of -128 ...), the f16 fields finite; activations that quantize
    to +-127 / -128.  Bytes back, dequantize and every kernel choice against the oracle: the integer ranges the
    matrix-core kernels' digit splits assume hold for any block."""
    rng = np.random.default_rng(dt * 131 + m + k + n + mode)
    ts, kb = orc.TYPE_SIZE[dt], k // orc.BLOCK_SIZE[dt]
    raw = rng.integers(0, 256, size=(n * kb, ts), dtype=np.uint8)
    if mode == 1:
        raw[:] = 0xff
    if mode == 2:
        raw[:] = rng.choice([0x00, 0x80, 0x7f, 0xff], size=raw.shape).astype(np.uint8)
    for off in _F16_FIELDS[dt]:
        vals = (rng.uniform(1e-3, 1.0, size=n * kb) * rng.choice([-1.0, 1.0], size=n * kb)).astype(np.float16)
        raw[:, off:off + 2] = vals.view(np.uint8).reshape(-1, 2)
    blocks = raw.ravel()
    x = np.where(rng.random((m, k)) < 0.5, -3.0, 3.0).astype(np.float32) if mode else rng.standard_normal((m, k)).astype(np.float32)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    assert np.array_equal(qw.to_ggml(), blocks)
    assert np.array_equal(qw.dequantize().cpu().numpy().ravel(), orc.dequantize(dt, blocks).ravel()[:n * k])
    ref = orc.matmul(dt, x, blocks, n).astype(np.float64)
    for flags in (0, qh.FLAG_STAGED_ACT, qh.FLAG_FORCE_MATVEC, qh.FLAG_FORCE_SKINNY, qh.FLAG_FORCE_GEMM):
        try:
            got = qh.qmatmul(qw, dev(x), flags).cpu().numpy().astype(np.float64)
        except qh.QHipError:
            assert flags in (qh.FLAG_FORCE_SKINNY, qh.FLAG_FORCE_GEMM)   # a forced kernel that does not take the shape
            continue
        assert np.isfinite(got).all()
        assert np.linalg.norm(got - ref) <= REL_L2_TOL * np.linalg.norm(ref), flags


@pytest.mark.parametrize("dt,m", [(orc.Q4_0, 33), (orc.Q8_0, 33), (orc.Q4K, 130), (orc.Q6K, 130), (orc.Q5K, 130)])
def test_deterministic_flag_repeats_bit_for_bit(qh, dt, m):
    """quantized_tests.rs:181-216 (`qmm_batch`): the CPU QMatMul gives the same bits on every run.  The tile kernels split K
    over workgroups that add their partial sums atomically when a weight has few row tiles (4096 x 4096 at these row
    counts); with CQ_FLAG_DETERMINISTIC they do not, and twenty calls give the same bits - which also match the oracle
    to the f32 bars on sampled rows."""
    n = k = 4096
    gen = torch.Generator(device="cuda").manual_seed(int(dt) * 100 + m)
    qw = qh.QWeight.zeros(dt, n, k).quantize_(torch.randn((n, k), device="cuda", generator=gen) * 0.02)
    x = torch.randn((m, k), device="cuda", generator=gen)
    first = qh.qmatmul(qw, x, qh.FLAG_DETERMINISTIC)
    for _ in range(19):
        assert torch.equal(qh.qmatmul(qw, x, qh.FLAG_DETERMINISTIC), first)
    blocks = qw.to_ggml().reshape(n, -1)
    rows = np.ascontiguousarray(blocks[1000:1016]).reshape(-1)
    xs = x[[0, m // 2, m - 1]].cpu().numpy()
    check_f32(first[[0, m // 2, m - 1]][:, 1000:1016].cpu().numpy(), orc.matmul(dt, xs, rows, 16))
    # the default launch of the same call agrees to rounding
    plain = qh.qmatmul(qw, x)
    assert float((plain - first).norm() / first.norm()) < 1e-6


def test_deterministic_flag_grouped_experts(qh):
    """The grouped launch of an expert's w2-shaped projection (few row tiles, long rows) splits K by default."""
    n, k, n_e = 512, 4096, 4
    rng = np.random.default_rng(5)
    experts = []
    for e in range(n_e):
        w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
        experts.append(qh.QWeight.from_ggml(orc.Q6K, orc.quantize(orc.Q6K, w), n, k))
    offsets = np.array([0, 12, 30, 41, 64], dtype=np.int32)
    x = dev(rng.standard_normal((64, k)).astype(np.float32))
    first = qh.qmatmul_grouped(experts, x, None, offsets, flags=qh.FLAG_DETERMINISTIC)
    for _ in range(10):
        assert torch.equal(qh.qmatmul_grouped(experts, x, None, offsets, flags=qh.FLAG_DETERMINISTIC), first)
    plain = qh.qmatmul_grouped(experts, x, None, offsets)
    assert float((plain - first).norm() / first.norm()) < 1e-6
