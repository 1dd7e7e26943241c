"""Re-entrancy of the C ABI (the reference's `QuantizedType: Send + Sync`, mod.rs:250, with
`QMatMul` holding an `Arc<QTensor>`, :395): one weight used from several host threads at once,
each thread on its own stream with its own workspace; errors stay with the thread that caused them."""
import ctypes as C
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from oracle import cpu_oracle as orc  # noqa: E402  (checker only)
from test_gpu_parity import check_f32, make_inputs  # noqa: E402


def test_one_weight_from_four_threads():
    from candle_amd import qhip
    L = qhip.load()
    n, k = 256, 2048
    w, _ = make_inputs(9, 1, k, n)
    blocks = orc.quantize(orc.Q4K, w)
    qw = qhip.QWeight.from_ggml(orc.Q4K, blocks, n, k)
    rows = [1, 3, 16, 40]                      # decode, split-K MFMA, split-K MFMA, tile kernel
    inputs = [np.random.default_rng(100 + i).standard_normal((m, k)).astype(np.float32) for i, m in enumerate(rows)]
    results, errors = [None] * len(rows), [None] * len(rows)

    def work(i):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                x = torch.from_numpy(inputs[i]).cuda()
                ws = qhip.Workspace()
                y = None
                for _ in range(25):
                    y = qhip.qmatmul(qw, x, workspace=ws)
                # an error on this thread: the message is this thread's, the other threads never see it
                bad = torch.zeros((rows[i], k + 256), dtype=torch.float32, device="cuda")
                try:
                    qhip.qmatmul(qw, bad)
                except qhip.QHipError:
                    pass
                rc = L.cq_qmatmul(qw.handle, None, rows[i], C.c_void_p(y.data_ptr()), 0, None, 0, None)
                assert rc == -1 and b"null argument" in L.cq_last_error()
                stream.synchronize()
                results[i] = y.cpu().numpy()
        except Exception as e:   # surfaced in the main thread below
            errors[i] = e

    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(rows))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert all(e is None for e in errors), errors
    for i in range(len(rows)):
        check_f32(results[i], orc.matmul(orc.Q4K, inputs[i], blocks, n))
    assert L.cq_last_error() == b"" or b"null argument" not in L.cq_last_error()   # the main thread made no such call
