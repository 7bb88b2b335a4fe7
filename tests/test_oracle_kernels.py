"""CPU: pins the GEMV/GEMM restatement in oracle/tg_oracle.c.

  * bit for bit against the compiled reference's outputs in tests/golden/golden.npz
    (gemv::launch_qgemv, launch_qgemv_logits, gemm::launch_qgemm; csrc/include/linalg.hpp:176-308)
  * against what the mathematics fixes: an exact integer closed form, float64 brute force,
    column independence, linearity, the accumulate-then-scale order.
"""
import hashlib

import numpy as np
import pytest

import golden_inputs as gi
from conftest import normrel


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


@pytest.mark.parametrize("name", list(gi.GEMV_CASES))
def test_gemv_bit_exact_vs_reference(oracle, golden, name):
    i, n, logits, seed = gi.GEMV_CASES[name]
    x, W, s = gi.gemv_inputs(i, n, seed)
    y = oracle.qgemv(x, W, s, logits)
    assert np.array_equal(y[:2048], golden[f"gemv/{name}/head"])
    assert sha(y) == str(golden[f"gemv/{name}/sha"])


@pytest.mark.parametrize("name", list(gi.GEMM_CASES))
def test_gemm_bit_exact_vs_reference(oracle, golden, name):
    m, i, n, seed = gi.GEMM_CASES[name]
    A, W, s = gi.gemm_inputs(m, i, n, seed)
    Cm = oracle.qgemm(A, W, s)
    assert np.array_equal(Cm.reshape(-1)[:2048], golden[f"gemm/{name}/head"])
    assert sha(Cm) == str(golden[f"gemm/{name}/sha"])


@pytest.mark.parametrize("i,n,logits", [(256, 256, False), (640, 2048, False), (1152, 6912, False), (6912, 1152, False),
                                        (640, 262144, True)])
def test_gemv_integer_closed_form(oracle, i, n, logits):
    """Integer-valued x and power-of-two scales: every product and partial sum is exactly
    representable, so any correct implementation must match the integer result bit for bit."""
    rng = np.random.default_rng(i + n)
    x = rng.integers(-8, 9, i).astype(np.float32)
    W = rng.integers(-127, 128, (i, n), dtype=np.int8)
    s = np.full(n, 2.0 ** -10, np.float32)
    y = oracle.qgemv(x, W, s, logits)
    exact = (x.astype(np.int64) @ W.astype(np.int64)).astype(np.float64) * 2.0 ** -10
    assert np.array_equal(y.astype(np.float64), exact)


def test_gemm_integer_closed_form(oracle):
    rng = np.random.default_rng(5)
    A = rng.integers(-8, 9, (9, 640)).astype(np.float32)
    W = rng.integers(-127, 128, (640, 256), dtype=np.int8)
    s = np.full(256, 2.0 ** -7, np.float32)
    Cm = oracle.qgemm(A, W, s)
    exact = (A.astype(np.int64) @ W.astype(np.int64)).astype(np.float64) * 2.0 ** -7
    assert np.array_equal(Cm.astype(np.float64), exact)


def test_gemv_float64_brute_force(oracle):
    x, W, s = gi.gemv_inputs(256, 256, 77)
    y = oracle.qgemv(x, W, s)
    ref = (x.astype(np.float64) @ W.astype(np.float64)) * s.astype(np.float64)
    assert normrel(y, ref) < 1e-6
    # a transposed operand or a scale applied per row instead of per column fails these
    assert normrel(y, (W.astype(np.float64) @ x.astype(np.float64)) * s) > 0.1
    A, W2, s2 = gi.gemm_inputs(5, 256, 256, 78)
    ref2 = (A.astype(np.float64) @ W2.astype(np.float64)) * s2.astype(np.float64)[None, :]
    assert normrel(oracle.qgemm(A, W2, s2), ref2) < 1e-6


def test_gemv_column_independence_and_linearity(oracle):
    x, W, s = gi.gemv_inputs(640, 256, 79)
    y = oracle.qgemv(x, W, s)
    W2 = W.copy()
    W2[:, 17] = -W2[:, 17]
    y2 = oracle.qgemv(x, W2, s)
    changed = np.nonzero(y != y2)[0]
    assert changed.tolist() == [17] and y2[17] == -y[17]
    assert np.array_equal(oracle.qgemv(2.0 * x, W, s), 2.0 * y)  # scaling by 2 is exact in fp32
    assert np.array_equal(oracle.qgemv(x, W, 2.0 * s), 2.0 * y)


def test_gemv_variants_differ_only_in_rounding(oracle):
    """launch_qgemv (per-row add) and launch_qgemv_logits (4-row fused groups) are different
    roundings of the same sums (linalg.hpp:46-81 vs 119-149)."""
    x, W, s = gi.gemv_inputs(640, 2048, 80)
    a, b = oracle.qgemv(x, W, s, False), oracle.qgemv(x, W, s, True)
    assert not np.array_equal(a, b)
    assert normrel(a, b) < 1e-6


def test_unsupported_shapes(oracle):
    """ROW_SWITCH / COL_SWITCH (static_switch.hpp:7-58) throw on anything else."""
    x, W, s = gi.gemv_inputs(512, 256, 81)
    with pytest.raises(RuntimeError):
        oracle.qgemv(x, W, s)
    x, W, s = gi.gemv_inputs(256, 512, 82)
    with pytest.raises(RuntimeError):
        oracle.qgemv(x, W, s)
    with pytest.raises(RuntimeError):
        oracle.qgemm(np.zeros((2, 256), np.float32), W, s)
    assert oracle.L.tgo_legal_in(262144) == 0 and oracle.L.tgo_legal_out(262144) == 1
