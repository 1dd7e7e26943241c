"""The timed CPU baseline (AVX2 + threads) agrees with the scalar oracle to the reference's own
SIMD-vs-scalar criterion: |opt - unopt| / K <= 1e-6 (candle-core/tests/quantized_tests.rs:836)."""
import numpy as np
import pytest

from oracle import cpu_oracle as orc


@pytest.mark.parametrize("dt", [orc.Q4_0, orc.Q8_0, orc.Q4K, orc.Q6K])
@pytest.mark.parametrize("m,k,n", [(1, 4096, 300), (3, 1024, 513), (2, 11008, 64)])
def test_baseline_matches_scalar_oracle(dt, m, k, n):
    rng = np.random.default_rng(dt * 31 + k)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[0, :: 97] = 8.0
    blocks = orc.quantize(dt, w)
    want = orc.matmul(dt, x, blocks, n)
    got = orc.baseline_matmul(dt, x, blocks, n)
    assert np.abs(got - want).max() / k <= 1e-6
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-5
