"""GPU: tg_qgemm_dev_static, the device-resident GEMM entry point that allocates nothing (its scratch, the digit
planes of the activations and the row factors, is a fixed array in the library's device image), against
tg_qgemm_dev on the same operands: same kernels, so the same bits.  Two calls in a row, the second with a
smaller input (the scratch still holds the first call's planes), then a size beyond the stated limit."""
import numpy as np
import pytest

import golden_inputs as gi

pytestmark = pytest.mark.gpu

MAX_ELEMS = 2 * 1024 * 1024   # TG_QGEMM_STATIC_MAX_ELEMS


def _run(tg, w, A, n_out, static):
    m = A.shape[0]
    ad = tg.DeviceBuffer.from_numpy(A)
    cd = tg.DeviceBuffer.from_numpy(np.full((m, n_out), np.nan, np.float32))
    (w.gemm_static if static else w.gemm)(cd, ad, m)
    tg.synchronize()
    return cd.to_numpy(np.float32, (m, n_out))


@pytest.mark.parametrize("i,n", [(1152, 6912), (6912, 1152)])
def test_static_scratch_gemm_equals_the_allocating_entry_point(tg, oracle, i, n):
    print(f"static-scratch GEMM {i}x{n}", flush=True)
    rng = np.random.default_rng(77 + i)
    W = rng.integers(-127, 128, (i, n), dtype=np.int8)
    s = rng.uniform(0.001, 0.02, n).astype(np.float32)
    w = tg.QWeight(W, s)
    m_big = (MAX_ELEMS // i) // 128 * 128          # the largest multiple of 128 rows inside the limit
    assert m_big >= 256
    for m in (m_big - 5, 70):                      # ragged row counts; the second call is the smaller one
        A = rng.standard_normal((m, i)).astype(np.float32)
        want = _run(tg, w, A, n, static=False)
        got = _run(tg, w, A, n, static=True)
        assert not np.isnan(got).any()
        assert np.array_equal(got, want)
        if m == 70:                                # and right, not only equal: against the CPU checker
            ref = oracle.qgemm(A, W, s)
            assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 3e-6
    # beyond the stated maximum: a clear error, nothing launched
    m_over = m_big + 1
    ad = tg.DeviceBuffer.from_numpy(np.zeros((m_over, i), np.float32))
    cd = tg.DeviceBuffer(4 * m_over * n)
    with pytest.raises(tg.TgError) as e:
        w.gemm_static(cd, ad, m_over)
    assert e.value.code == -4 and "TG_QGEMM_STATIC_MAX_ELEMS" in str(e.value)
    w.gemm(cd, ad, m_over)                          # the allocating entry point still takes it
    tg.synchronize()


def test_static_scratch_gemm_in_the_exact_mode(tg):
    """tg_set_gemm_mode(0) needs no scratch at all; the entry point must still work and agree."""
    i, n, m = 640, 1024, 33
    A, W, s = gi.gemm_inputs(m, i, n, 991)
    w = tg.QWeight(W, s)
    tg.lib().tg_set_gemm_mode(0)
    try:
        assert np.array_equal(_run(tg, w, A, n, static=True), _run(tg, w, A, n, static=False))
    finally:
        tg.lib().tg_set_gemm_mode(1)
