"""K-quant weights x Q8_1 activations (CQ_FLAG_ACT_Q8_1): the formulation of the reference's CUDA arm
(`mul_mat_via_q8_1`, candle-core/src/quantized/cuda.rs:298-365; dot bodies candle-kernels/src/quantized.cu:2141-2166
for Q4_K, :2258-2281 for Q6_K) with the activations quantized by the CPU rule of `BlockQ8_1::from_float`
(k_quants.rs:665-691), against the oracle's `orc_matmul_q8_1` and against an exact evaluation of the same formula."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from oracle import cpu_oracle as orc  # noqa: E402  (checker only)

REL_L2_TOL = 1e-4
MAX_ABS_FACTOR = 1e-3


@pytest.fixture(scope="module")
def qh():
    from candle_amd import qhip
    qhip.load()
    assert qhip.load().cq_device_count() >= 1, "no HIP device visible"
    return qhip


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def check_f32(got, want):
    got = got.astype(np.float64)
    want = want.astype(np.float64)
    for r in range(want.shape[0]):
        nrm = max(np.linalg.norm(want[r]), 1e-30)
        assert np.linalg.norm(got[r] - want[r]) <= REL_L2_TOL * nrm, (r, np.linalg.norm(got[r] - want[r]) / nrm)
        assert np.abs(got[r] - want[r]).max() <= MAX_ABS_FACTOR * nrm, r


from test_oracle_golden import q8_1_formula_float64 as _exact  # noqa: E402  (the exact evaluation, also held against the oracle on the CPU)


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q6K])
@pytest.mark.parametrize("m,k,n", [(1, 256, 8), (3, 512, 37), (11, 1024, 64), (9, 4096, 48),
                                   # more than 32 rows and n % 32 == 0: the matrix-core kernel (one, two and four
                                   # 32-row tiles per workgroup, a last tile and a last workgroup that are not full)
                                   (33, 512, 64), (70, 1024, 96), (130, 256, 32), (200, 768, 288), (300, 512, 8192)])
def test_q8_1_variant_matches_oracle_and_exact_formula(qh, dt, m, k, n):
    rng = np.random.default_rng(1000 * m + n)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x.ravel()[rng.choice(x.size, size=max(1, x.size // 100), replace=False)] = 8.0
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    got = qh.qmatmul(qw, dev(x), flags=qh.FLAG_ACT_Q8_1).cpu().numpy()
    check_f32(got, orc.matmul_q8_1(dt, x, blocks, n))
    exact = _exact(dt, x, blocks, n, k)
    # a wrong integer anywhere moves a result by far more than f32 rounding does
    assert np.abs(got - exact).max() <= 2e-5 * np.abs(exact).max() + 1e-6
    # batch invariance: a row's result does not depend on the rows beside it (quantized_tests.rs:181-216)
    if 1 < m <= 32:
        one = qh.qmatmul(qw, dev(x[1:2]), flags=qh.FLAG_ACT_Q8_1).cpu().numpy()
        assert np.array_equal(one[0], got[1])
    if m > 32:
        # the same within the matrix-core kernel (another tile height, other neighbours), and to rounding against
        # the dot-product kernel that takes up to 32 rows
        part = qh.qmatmul(qw, dev(x[m - 33:]), flags=qh.FLAG_ACT_Q8_1).cpu().numpy()
        assert np.array_equal(part, got[m - 33:])
        few = qh.qmatmul(qw, dev(x[:5]), flags=qh.FLAG_ACT_Q8_1).cpu().numpy()
        check_f32(got[:5], few)


@pytest.mark.parametrize("dt", [orc.Q4K, orc.Q6K])
@pytest.mark.parametrize("k,n", [(4096, 14336), (14336, 4096)])
def test_q8_1_variant_config3_shapes(qh, dt, k, n):
    """configs[3]: M = 512 with 1 % outliers at +-8 sigma; sampled weight rows against the oracle (the whole
    product would take the scalar oracle minutes) and the whole output against the Q8K formulation, from which it may
    differ by the two activation quantizers' noise only."""
    rng = np.random.default_rng(n)
    m = 512
    gen = torch.Generator(device="cuda")
    gen.manual_seed(n + int(dt))
    wt = torch.randn((n, k), generator=gen, device="cuda") * 0.02
    qw = qh.QWeight.zeros(dt, n, k).quantize_(wt)
    del wt
    x = rng.standard_normal((m, k)).astype(np.float32)
    idx = rng.choice(x.size, size=x.size // 100, replace=False)
    x.ravel()[idx] = np.where(rng.random(idx.size) < 0.5, -8.0, 8.0).astype(np.float32)
    xd = dev(x)
    got = qh.qmatmul(qw, xd, flags=qh.FLAG_ACT_Q8_1)
    blocks = qw.to_ggml().reshape(n, -1)
    rows = np.unique(np.concatenate([[0, 1, n // 2, n - 2, n - 1], rng.choice(n, size=19, replace=False)]))
    ms = np.unique(np.concatenate([[0, 7, 8, m - 1], rng.choice(m, size=12, replace=False)]))
    ref = orc.matmul_q8_1(dt, x[ms], blocks[rows].ravel(), rows.size)
    check_f32(got.cpu().numpy()[np.ix_(ms, rows)], ref)
    q8k = qh.qmatmul(qw, xd)
    dist = float((got - q8k).norm() / q8k.norm())
    assert dist < 2e-2, dist   # two 8-bit activation quantizers apart


def test_q8_1_variant_errors(qh):
    rng = np.random.default_rng(3)
    n, k = 32, 512
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = dev(rng.standard_normal((2, k)).astype(np.float32))
    q8 = qh.QWeight.from_ggml(orc.Q8_0, orc.quantize(orc.Q8_0, w), n, k)
    with pytest.raises(qh.QHipError, match="Q8_1 activations are for Q4K and Q6K"):
        qh.qmatmul(q8, x, flags=qh.FLAG_ACT_Q8_1)
    q4 = qh.QWeight.from_ggml(orc.Q4K, orc.quantize(orc.Q4K, w), n, k)
    with pytest.raises(qh.QHipError, match="combines with"):
        qh.qmatmul(q4, x, flags=qh.FLAG_ACT_Q8_1 | qh.FLAG_FORCE_GEMM)
    # the quantized rows can be shared by a second weight, like the other formulation's
    ws = qh.Workspace()
    a = qh.qmatmul(q4, x, flags=qh.FLAG_ACT_Q8_1, workspace=ws)
    b = qh.qmatmul(q4, x, flags=qh.FLAG_ACT_Q8_1 | qh.FLAG_REUSE_ACT, workspace=ws)
    assert torch.equal(a, b)
