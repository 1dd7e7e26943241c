"""The per-block integer dot products out of the matrix-core kernels (the small-batch split-K kernels and the prefill
tile kernels), bit for bit against the oracle's `block_int_dots` (k_quants.rs:1221-1241 for Q4K, :1418-1438 for Q5K,
:1615-1633 for Q6K, :245-250 / :640-645 for Q4_0 / Q8_0) and, at the BASELINE configs[3] shape, against the
dot-product kernels' integers over the whole launch.  The Q4K / Q5K min term is not an integer in these kernels: it
is contracted on the f16 matrix core from operands split in two f16 pieces; its distance to the integer form is
bounded here."""
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


def make_inputs(seed, m, k, n, x_scale=1.0):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = (rng.standard_normal((m, k)) * x_scale).astype(np.float32)
    idx = rng.choice(x.size, size=max(1, x.size // 100), replace=False)
    x.ravel()[idx] = np.where(rng.random(idx.size) < 0.5, -8.0, 8.0).astype(np.float32) * np.float32(x_scale)
    return w, x


def k4_scales_mins(hdr12):
    """get_scale_min_k4 (utils.rs:49-59) over [..., 12] bytes -> (sc[..., 8], mn[..., 8])."""
    b = hdr12.astype(np.int64)
    sc = np.zeros(b.shape[:-1] + (8,), np.int64)
    mn = np.zeros(b.shape[:-1] + (8,), np.int64)
    for j in range(8):
        if j < 4:
            sc[..., j] = b[..., j] & 63
            mn[..., j] = b[..., j + 4] & 63
        else:
            sc[..., j] = (b[..., j + 4] & 0xF) | ((b[..., j - 4] >> 6) << 4)
            mn[..., j] = (b[..., j + 4] >> 4) | ((b[..., j] >> 6) << 4)
    return sc, mn


def min_term_reference(dt, acts, m, blocks, n, k, with_d8):
    """(-s * sum_j min_j*bsum32_j, |s| * sum_j min_j*|bsum32_j|) in float64, [m, n, k/256], s = dmin * d8 (tile kernel)
    or s = dmin (small-batch kernels: the activation block's scale multiplies afterwards, with the main term)."""
    kb = k // 256
    w = blocks.reshape(n, kb, orc.TYPE_SIZE[dt])
    dmin = w[..., 2:4].copy().view(np.float16)[..., 0].astype(np.float64)          # [n, kb]
    _, mn = k4_scales_mins(w[..., 4:16])                                            # [n, kb, 8]
    a = acts.reshape(m, kb, 292)
    d8 = a[..., :4].copy().view(np.float32)[..., 0].astype(np.float64)              # [m, kb]
    bs16 = a[..., 260:292].copy().view(np.int16).astype(np.int64)                   # [m, kb, 16]
    bs32 = bs16[..., 0::2] + bs16[..., 1::2]                                        # [m, kb, 8]
    s = np.einsum("nbj,mbj->mnb", mn, bs32)
    sabs = np.einsum("nbj,mbj->mnb", mn, np.abs(bs32))
    scale = dmin[None] * (d8 if with_d8 else np.ones_like(d8))[:, None]
    return -scale * s, np.abs(scale) * sabs


KQ = [orc.Q4K, orc.Q5K, orc.Q6K]
B32 = [orc.Q8_0, orc.Q4_0]


def check_dump(qh, dt, kernel, m, k, n, seed, x_scale=1.0):
    w, x = make_inputs(seed, m, k, n, x_scale)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    oi, om = qh.qmatmul_int_dots_mfma(qw, dev(x), kernel)
    acts = np.concatenate([orc.quantize(orc.VEC_DOT_TYPE[dt], x[r]) for r in range(m)])
    wi, wm = orc.block_int_dots(dt, acts, m, blocks, n, k)
    assert np.array_equal(oi.cpu().numpy(), wi)                  # every (row, weight row, block), bit for bit
    if dt in (orc.Q4K, orc.Q5K):
        tile = kernel == qh.MFMA_TILE
        ref, mag = min_term_reference(dt, acts, m, blocks, n, k, with_d8=tile)
        got = om.cpu().numpy().astype(np.float64)
        # the sums exact in f16, -dmin*min_j in two f16 pieces: every product exact, the f32 sum of the 32 terms rounds
        # (tile kernel: stored times d8, one more rounding; its 128-row tiles add the terms to I * dw, which the dump
        # leaves out)
        bound = 2.0 ** -20 if tile else 2.0 ** -21
        assert np.all(np.abs(got - ref) <= bound * mag + 1e-30), float((np.abs(got - ref) / (mag + 1e-30)).max())
        # the same launch with the minima themselves as the weight operand of that contraction: the integer Mn_b of
        # k_quants.rs:1221-1241, bit for bit (same instructions, same sums; at most 16 * 2048 * 63: exact in f32)
        oi2, om2 = qh.qmatmul_int_dots_mfma(qw, dev(x), kernel | qh.MFMA_INT_MIN)
        assert np.array_equal(oi2.cpu().numpy(), wi)
        assert np.array_equal(om2.cpu().numpy().astype(np.int64), wm.astype(np.int64))
    return x, blocks, qw


@pytest.mark.parametrize("dt", KQ + B32)
@pytest.mark.parametrize("m,k,n", [(2, 256, 16), (5, 512, 64), (13, 1024, 48), (19, 768, 96), (32, 2304, 32), (27, 4096, 80),
                                   (45, 512, 64)])
def test_skinny_kernel_integers(qh, dt, m, k, n):
    """The split-K small-batch kernels: one workgroup tile per CU (activations resident in LDS) for these n."""
    check_dump(qh, dt, qh.MFMA_SKINNY, m, k, n, 11 * dt + m + k + n)


@pytest.mark.parametrize("dt", KQ + B32)
def test_skinny_kernel_integers_many_tiles(qh, dt):
    """More 16-row weight tiles than compute units: the kernel that copies activations per block."""
    check_dump(qh, dt, qh.MFMA_SKINNY, 16, 512, 16 * 300, 77 + dt)


@pytest.mark.parametrize("dt,m,n", [(orc.Q4K, 16, 16 * 300), (orc.Q4K, 11, 16 * 700), (orc.Q4K, 16, 16 * 1100),
                                     (orc.Q4K, 7, 16 * 800), (orc.Q5K, 8, 16 * 800), (orc.Q5K, 16, 16 * 300),
                                     (orc.Q8_0, 16, 16 * 300), (orc.Q8_0, 5, 16 * 1100), (orc.Q4_0, 16, 16 * 700),
                                     (orc.Q4_0, 8, 16 * 1030)])
def test_skinny_kernel_integers_rounds_of_tiles(qh, dt, m, n):
    """K = 4096 and more 16-row tiles than compute units: a workgroup walks its tiles in rounds of up to four with one
    meeting per round (Q4K / Q5K / Q8_0 / Q4_0 where the slots fit the LDS; the other cases take the per-block kernel):
    one tile more for some workgroups than for others, two rounds, a round of one."""
    check_dump(qh, dt, qh.MFMA_SKINNY, m, 4096, n, 5 * dt + m + n)


@pytest.mark.parametrize("dt", KQ + B32)
@pytest.mark.parametrize("m,k,n", [(9, 256, 32), (17, 1024, 352), (32, 512, 64), (33, 512, 96), (64, 1024, 160), (130, 768, 288),
                                   (129, 2048, 416)])
def test_tile_kernel_integers(qh, dt, m, k, n):
    """The prefill tile kernels on ragged shapes: tile heights of 32, 64 and 128 rows, with and without K split."""
    if dt in B32 and m <= 16:
        pytest.skip("the Q8_0 / Q4_0 tile kernel is taken above 16 rows only")
    check_dump(qh, dt, qh.MFMA_TILE, m, k, n, 13 * dt + m + k + n)


@pytest.mark.parametrize("x_scale", [1e-30, 1e-8, 1e-2, 1.0, 500.0, 1e6, 1e30])
@pytest.mark.parametrize("kernel", ["skinny", "tile64", "tile"])
def test_min_term_error_bound_across_magnitudes(qh, kernel, x_scale):
    """The min term's matrix-core operands are the integer sums of the block and -dmin*min_j; the activation block's
    scale multiplies afterwards in f32: the bound holds for activations of any magnitude, in the small-batch kernels,
    in tiles of up to 64 rows (an accumulator of their own) and in the 128-row tiles (the scaled integers as the
    accumulator)."""
    kid = qh.MFMA_SKINNY if kernel == "skinny" else qh.MFMA_TILE
    m, n = {"skinny": (16, 64), "tile64": (56, 64), "tile": (300, 2048)}[kernel]
    check_dump(qh, orc.Q4K, kid, m, 1024, n, 5, x_scale)


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q5K, orc.Q6K])
@pytest.mark.parametrize("m,k,n", [(16, 2048, 64), (60, 1024, 96), (70, 1024, 96), (512, 512, 64), (300, 1024, 2048)])
def test_rows_of_different_magnitudes(qh, dt, m, k, n):
    """One batch whose rows span forty orders of magnitude (1e-20 .. 1e20), one row with a block a thousand times the
    others and one all-zero row: every row against the oracle at the usual bars, on both matrix-core kernels."""
    rng = np.random.default_rng(m + k + n + int(dt))
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    x0 = x
    for flags, lo, hi in ((qh.FLAG_FORCE_SKINNY, -20, 21), (qh.FLAG_FORCE_GEMM, -20, 21)):
        scales = np.float32(10.0) ** rng.integers(lo, hi, size=m).astype(np.float32)
        scales[2] = 1.0
        x = x0 * scales[:, None]
        x[1] = 0.0
        x[2, 256:512] *= np.float32(1e3)          # one block dwarfs the others of its row
        want = orc.matmul(dt, x, blocks, n).astype(np.float64)
        got = qh.qmatmul(qw, dev(x), flags).cpu().numpy().astype(np.float64)
        assert np.all(np.isfinite(got))
        for r in range(m):
            nrm = np.linalg.norm(want[r])
            assert np.linalg.norm(got[r] - want[r]) <= 1e-4 * nrm + 1e-38, (flags, r, float(scales[r]))
            assert np.abs(got[r] - want[r]).max() <= 1e-3 * nrm + 1e-38, (flags, r)


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q5K])
def test_tall_tiles_rows_of_different_magnitudes(qh, dt):
    """A launch of 128-row tiles (512 rows on 16 384 weight rows: more 32-row tiles than four rounds of compute units) with
    rows forty orders of magnitude apart: every row against the dot-product kernels, which hold the min term as an
    integer, and sampled weight rows against the oracle."""
    rng = np.random.default_rng(9 + int(dt))
    m, k, n = 512, 512, 16384
    gen = torch.Generator(device="cuda").manual_seed(int(dt))
    qw = qh.QWeight.zeros(dt, n, k).quantize_(torch.randn((n, k), generator=gen, device="cuda") * 0.02)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x *= (np.float32(10.0) ** rng.integers(-20, 21, size=m).astype(np.float32))[:, None]
    x[7] = 0.0
    xd = dev(x)
    got = qh.qmatmul(qw, xd, qh.FLAG_FORCE_GEMM)
    ref = qh.qmatmul(qw, xd, qh.FLAG_FORCE_MATVEC)
    assert bool(torch.isfinite(got).all())
    err = (got.double() - ref.double()).norm(dim=1)
    nrm = ref.double().norm(dim=1)
    assert bool((err <= 1e-5 * nrm + 1e-38).all()), float((err / (nrm + 1e-38)).max())
    cols = np.unique(np.concatenate([[0, 255, 256, n - 1], rng.choice(n, size=20, replace=False)]))
    blocks = qw.to_ggml().reshape(n, -1)[cols].ravel()
    want = orc.matmul(dt, x, blocks, len(cols)).astype(np.float64)
    sub = got[:, torch.from_numpy(cols).cuda()].cpu().numpy().astype(np.float64)
    for r in range(m):
        assert np.linalg.norm(sub[r] - want[r]) <= 1e-4 * np.linalg.norm(want[r]) + 1e-38, r


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q5K])
def test_grouped_rows_of_different_magnitudes(qh, dt):
    """The grouped launch of the expert FFN (32-row tiles) with token rows forty orders of magnitude apart: every row
    against the oracle's matmul with its expert."""
    rng = np.random.default_rng(int(dt))
    k, n, tokens = 1024, 96, 24
    ws = [(rng.standard_normal((n, k)) * 0.02).astype(np.float32) for _ in range(3)]
    blocks = [orc.quantize(dt, w) for w in ws]
    experts = [qh.QWeight.from_ggml(dt, b, n, k) for b in blocks]
    x = rng.standard_normal((tokens, k)).astype(np.float32)
    x *= (np.float32(10.0) ** rng.integers(-20, 21, size=tokens).astype(np.float32))[:, None]
    offsets = np.array([0, 17, 17 + 40, 17 + 40 + 5], np.int32)
    rid = rng.integers(0, tokens, size=int(offsets[-1])).astype(np.int32)
    y = qh.qmatmul_grouped(experts, dev(x), torch.from_numpy(rid).cuda(), offsets).cpu().numpy().astype(np.float64)
    assert np.all(np.isfinite(y))
    for e in range(3):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        want = orc.matmul(dt, x[rid[lo:hi]], blocks[e], n).astype(np.float64)
        for r in range(hi - lo):
            nrm = np.linalg.norm(want[r])
            assert np.linalg.norm(y[lo + r] - want[r]) <= 1e-4 * nrm + 1e-38, (e, r)


@pytest.mark.parametrize("dt,k,n", [(orc.Q4K, 4096, 14336), (orc.Q6K, 14336, 4096)])
def test_tile_kernel_integers_config3(qh, dt, k, n):
    """BASELINE configs[3] at full size (M = 512, 1 % outliers at +-8 sigma): every block integer of the launch equals
    the dot-product kernels' (compared on the device), and sampled rows equal the oracle's."""
    m = 512
    rng = np.random.default_rng(n + int(dt))
    gen = torch.Generator(device="cuda").manual_seed(n + int(dt))
    wt = torch.randn((n, k), generator=gen, device="cuda") * 0.02
    qw = qh.QWeight.zeros(dt, n, k).quantize_(wt)
    del wt
    x = rng.standard_normal((m, k)).astype(np.float32)
    idx = rng.choice(x.size, size=x.size // 100, replace=False)
    x.ravel()[idx] = np.where(rng.random(idx.size) < 0.5, -8.0, 8.0).astype(np.float32)
    xd = dev(x)
    oi, om = qh.qmatmul_int_dots_mfma(qw, xd, qh.MFMA_TILE)
    ri, rm = qh.qmatmul_int_dots(qw, xd)
    assert bool(torch.equal(oi, ri))
    del ri
    ms = np.unique(np.concatenate([[0, 31, 32, 127, 128, m - 1], rng.choice(m, size=6, replace=False)]))
    tiles = n // 256
    cols = np.unique(np.concatenate([[0, 31, 32, 255, 256 * (tiles // 2), 256 * (tiles // 2) + 255, n - 256, n - 1],
                                     rng.choice(n, size=24, replace=False)]))
    blocks = qw.to_ggml().reshape(n, -1)[cols].ravel()
    acts = np.concatenate([orc.quantize(orc.Q8K, x[r]) for r in ms])
    wi, wm = orc.block_int_dots(dt, acts, len(ms), blocks, len(cols), k)
    sub = oi[torch.from_numpy(ms).cuda()][:, torch.from_numpy(cols).cuda()].cpu().numpy()
    assert np.array_equal(sub, wi)
    if dt == orc.Q4K:
        ref, mag = min_term_reference(dt, acts, len(ms), blocks, len(cols), k, with_d8=True)
        got = om[torch.from_numpy(ms).cuda()][:, torch.from_numpy(cols).cuda()].cpu().numpy().astype(np.float64)
        assert np.all(np.abs(got - ref) <= 2.0 ** -19 * mag + 1e-30)
        # the integer Mn_b of every (row, weight row, block) of the launch against the dot-product kernels' (on the
        # device) and, on the sampled rows, the oracle's
        del oi, om
        _, om2 = qh.qmatmul_int_dots_mfma(qw, xd, qh.MFMA_TILE | qh.MFMA_INT_MIN)
        assert bool(torch.equal(om2.to(torch.int32), rm))
        sub = om2[torch.from_numpy(ms).cuda()][:, torch.from_numpy(cols).cuda()].cpu().numpy()
        assert np.array_equal(sub.astype(np.int64), wm.astype(np.int64))
        # whole launch: the float min term against the dot-product kernels' integer through the scales is covered by
        # the f32 comparison of the results in test_prefill_gemm_config3


def test_mfma_dump_errors(qh):
    rng = np.random.default_rng(1)
    w = (rng.standard_normal((24, 256)) * 0.02).astype(np.float32)
    qw = qh.QWeight.from_ggml(orc.Q4K, orc.quantize(orc.Q4K, w), 24, 256)       # 24 rows: neither kernel takes it
    x = dev(rng.standard_normal((4, 256)).astype(np.float32))
    with pytest.raises(qh.QHipError, match="does not take this weight"):
        qh.qmatmul_int_dots_mfma(qw, x, qh.MFMA_SKINNY)
    with pytest.raises(qh.QHipError, match="does not take this weight"):
        qh.qmatmul_int_dots_mfma(qw, x, qh.MFMA_TILE)
    with pytest.raises(qh.QHipError, match="CQ_MFMA_SKINNY or CQ_MFMA_TILE"):
        qh.qmatmul_int_dots_mfma(qw, x, 7)
