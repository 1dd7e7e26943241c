"""Several weights on the same activations (cq_qmatmul_multi) through the C ABI.

One activation row: a single launch over the rows of all weights; every output must equal, bit for bit,
what the weight's own call gives (same kernel arithmetic per row), which the parity tests hold against
the oracle.  More rows: the rows are quantized once and shared; again equal to the separate calls (to
rounding where a launch splits K and adds atomically)."""
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


def _weights(qh, dt, k, ns, seed):
    out = []
    for i, n in enumerate(ns):
        w, _ = make_inputs(seed + i, 1, k, n)
        blocks = orc.quantize(dt, w)
        out.append((qh.QWeight.from_ggml(dt, blocks, n, k), blocks))
    return out


@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
@pytest.mark.parametrize("k,ns", [(512, (64, 32, 32)), (2048, (256, 40)), (4096, (4096, 1024, 1024)), (1024, (8, 8, 24))])
def test_one_row_one_launch_equals_separate_calls(qh, dt, k, ns):
    if dt == orc.Q8_0 and k > 4096:
        pytest.skip("rows of more than 256 lane units take one call per weight")
    ws = _weights(qh, dt, k, ns, 100 + dt + k)
    rng = np.random.default_rng(k + dt)
    x = rng.standard_normal((1, k)).astype(np.float32)
    xd = dev(x)
    outs = qh.qmatmul_multi([w for w, _ in ws], xd)
    for (w, blocks), y in zip(ws, outs):
        assert torch.equal(y, qh.qmatmul(w, xd))
        check_f32(y.cpu().numpy(), orc.matmul(dt, x, blocks, w.shape[0]))
    # with rms_norm in front
    alpha = dev(rng.standard_normal(k).astype(np.float32))
    outs = qh.qmatmul_multi([w for w, _ in ws], xd, pre=qh.PRE_RMS_NORM, aux=alpha, eps=1e-5)
    for (w, _), y in zip(ws, outs):
        assert torch.equal(y, qh.qmatmul(w, xd, pre=qh.PRE_RMS_NORM, aux=alpha, eps=1e-5))


@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
@pytest.mark.parametrize("m", [2, 7, 40, 130])
def test_more_rows_share_the_quantized_rows(qh, dt, m):
    k, ns = 1024, (256, 96, 96)
    ws = _weights(qh, dt, k, ns, 200 + dt + m)
    rng = np.random.default_rng(m + dt)
    x = rng.standard_normal((m, k)).astype(np.float32)
    xd = dev(x)
    for pre, aux in ((qh.PRE_NONE, None), (qh.PRE_RMS_NORM, dev(rng.standard_normal(k).astype(np.float32))),
                     (qh.PRE_SILU_MUL, dev(rng.standard_normal((m, k)).astype(np.float32)))):
        outs = qh.qmatmul_multi([w for w, _ in ws], xd, pre=pre, aux=aux, eps=1e-5)
        for (w, blocks), y in zip(ws, outs):
            want = qh.qmatmul(w, xd, pre=pre, aux=aux, eps=1e-5)
            assert torch.allclose(y, want, rtol=1e-5, atol=1e-6)
            if pre == qh.PRE_NONE:
                check_f32(y.cpu().numpy(), orc.matmul(dt, x, blocks, w.shape[0]))


@pytest.mark.parametrize("dt", WEIGHT_DTYPES)
@pytest.mark.parametrize("m", [2, 3, 4])
def test_few_rows_one_launch_equals_separate_calls(qh, dt, m):
    """Two to four activation rows of short weight rows: still one launch over all weights, every output
    bit-identical to the weight's own call (which takes the same kernel for one weight)."""
    k, ns = 2048, (264, 40, 96)
    ws = _weights(qh, dt, k, ns, 400 + dt + m)
    x = np.random.default_rng(m * 7 + dt).standard_normal((m, k)).astype(np.float32)
    xd = dev(x)
    outs = qh.qmatmul_multi([w for w, _ in ws], xd)
    for (w, blocks), y in zip(ws, outs):
        assert torch.equal(y, qh.qmatmul(w, xd))
        check_f32(y.cpu().numpy(), orc.matmul(dt, x, blocks, w.shape[0]))


def test_single_weight_four_weights_and_errors(qh):
    dt, k = orc.Q4K, 512
    ws = _weights(qh, dt, k, (32, 32, 64, 32), 300)
    x = dev(np.random.default_rng(3).standard_normal((1, k)).astype(np.float32))
    for count in (1, 4):   # not a two- or three-weight launch: one call per weight, same results
        outs = qh.qmatmul_multi([w for w, _ in ws[:count]], x)
        for (w, _), y in zip(ws, outs):
            assert torch.equal(y, qh.qmatmul(w, x))
    other = _weights(qh, orc.Q6K, k, (32,), 301)[0][0]
    with pytest.raises(qh.QHipError):
        qh.qmatmul_multi([ws[0][0], other], x)            # dtypes differ
    longer = _weights(qh, dt, 2 * k, (32,), 302)[0][0]
    with pytest.raises(qh.QHipError):
        qh.qmatmul_multi([ws[0][0], longer], x)            # row lengths differ
