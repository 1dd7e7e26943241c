"""cq_qmatmul_static (the entry point that allocates nothing: its quantized activations live in a static
device array of the library) against cq_qmatmul, through the C ABI."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from oracle import cpu_oracle as orc  # noqa: E402  (checker only)

SCRATCH_BYTES = 16 << 20


@pytest.fixture(scope="module")
def qh():
    from candle_amd import qhip
    qhip.load()
    assert qhip.load().cq_device_count() >= 1, "no HIP device visible"
    return qhip


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _static(qh, qw, x, flags=0):
    n, k = qw.shape
    m = x.numel() // k
    y = torch.full((m, n), float("nan"), device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    qh.check(qh.load().cq_qmatmul_static(qw.handle, C.c_void_p(x.data_ptr()), m, C.c_void_p(y.data_ptr()), flags, stream))
    return y


# (dtype, n, k, [row counts: each later call is smaller than the one before], bit-exact?)
# The paths that go through the scratch: two-launch decode (forced), split-K MFMA kernel (5..32 rows), tile kernel
# (more rows; with n = 4096 and k = 14336 it splits K and adds partial sums atomically, which is not bit-stable).
CASES = [
    (orc.Q4K, 512, 4096, [16, 5], True),
    (orc.Q6K, 256, 2048, [64, 24, 8], True),
    (orc.Q8_0, 512, 4096, [16, 6], True),
    (orc.Q4_0, 256, 1024, [48, 7], True),
    (orc.Q4K, 1024, 2048, [200, 72], True),
    (orc.Q4K, 256, 14336, [96, 40], False),
]


@pytest.mark.parametrize("dt,n,k,rows,exact", CASES)
def test_static_scratch_equals_workspace_call(qh, dt, n, k, rows, exact):
    rng = np.random.default_rng(n + k)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    blocks = orc.quantize(dt, w)
    qw = qh.QWeight.from_ggml(dt, blocks, n, k)
    for m in rows:   # two (or three) calls in a row on the same scratch, each smaller than the last
        x = dev(rng.standard_normal((m, k)).astype(np.float32))
        assert qh.load().cq_workspace_bytes(qw.handle, m, 0) <= SCRATCH_BYTES
        got = _static(qh, qw, x)
        want = qh.qmatmul(qw, x, workspace=qh.Workspace())
        if exact:
            assert torch.equal(got, want), (dt, m)
        else:
            assert (got - want).norm() <= 1e-5 * want.norm()
        ref = orc.matmul(dt, x[:2].cpu().numpy(), blocks, n)
        assert np.linalg.norm(got[:2].cpu().numpy() - ref) <= 1e-4 * np.linalg.norm(ref)


def test_static_scratch_one_row_paths(qh):
    """One row: the single-launch kernel (no scratch at all) and, forced, the two-launch path through the scratch."""
    rng = np.random.default_rng(1)
    n, k = 1024, 4096
    blocks = orc.quantize(orc.Q4K, (rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    qw = qh.QWeight.from_ggml(orc.Q4K, blocks, n, k)
    for flags in (0, qh.FLAG_STAGED_ACT):
        for _ in range(2):
            x = dev(rng.standard_normal((1, k)).astype(np.float32))
            assert torch.equal(_static(qh, qw, x, flags), qh.qmatmul(qw, x, flags=flags))
    # in place, which always goes through the scratch
    x = dev(rng.standard_normal((1, k)).astype(np.float32))
    sq = qh.QWeight.from_ggml(orc.Q4K, orc.quantize(orc.Q4K, (rng.standard_normal((k, k)) * 0.02).astype(np.float32)), k, k)
    want = qh.qmatmul(sq, x).clone()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    qh.check(qh.load().cq_qmatmul_static(sq.handle, C.c_void_p(x.data_ptr()), 1, C.c_void_p(x.data_ptr()), 0, stream))
    assert torch.equal(x, want)


def test_static_scratch_refuses_what_does_not_fit(qh):
    L = qh.load()
    qw = qh.QWeight.zeros(orc.Q4K, 64, 14336)
    m = 1024
    assert L.cq_workspace_bytes(qw.handle, m, 0) > SCRATCH_BYTES
    x = torch.zeros((m, 14336), device="cuda")
    y = torch.zeros((m, 64), device="cuda")
    rc = L.cq_qmatmul_static(qw.handle, C.c_void_p(x.data_ptr()), m, C.c_void_p(y.data_ptr()), 0, None)
    assert rc == -4 and b"static array holds" in L.cq_last_error()
    assert L.cq_qmatmul_static(None, C.c_void_p(x.data_ptr()), 1, C.c_void_p(y.data_ptr()), 0, None) == -1
    # zero rows: nothing to do, no error
    assert L.cq_qmatmul_static(qw.handle, None, 0, None, 0, None) == 0


def test_static_scratch_allocates_nothing(qh):
    """The device allocator's counters do not move across calls (torch's allocator is not involved either: the
    call gets raw pointers), and the call works inside a stream capture, where allocation is illegal."""
    rng = np.random.default_rng(2)
    n, k, m = 512, 2048, 12
    blocks = orc.quantize(orc.Q4K, (rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    qw = qh.QWeight.from_ggml(orc.Q4K, blocks, n, k)
    x = dev(rng.standard_normal((m, k)).astype(np.float32))
    y = torch.empty((m, n), device="cuda")
    want = qh.qmatmul(qw, x)
    L = qh.load()
    L.cq_qmatmul_static(qw.handle, C.c_void_p(x.data_ptr()), m, C.c_void_p(y.data_ptr()), 0,
                        C.c_void_p(torch.cuda.current_stream().cuda_stream))   # eager once (raises LDS limits)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    s = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        y.fill_(0)
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=s):
            rc = L.cq_qmatmul_static(qw.handle, C.c_void_p(x.data_ptr()), m, C.c_void_p(y.data_ptr()), 0,
                                     C.c_void_p(s.cuda_stream))
        assert rc == 0, L.cq_last_error()
        for _ in range(3):
            y.fill_(0)
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, want)
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after >= free_before - (1 << 20)   # (graph bookkeeping aside: no 16 MiB workspace appeared)
