"""CPU: the int8 weight-only quantizer and the weight-file producer.

The rule is three lines of numpy in the reference (py/weight_handlers.py:10-20) and is fully
fixed by its text: scale = max|w| over axis 0 / 127 in fp32, q = rint(w / scale) (ties to even).
Two independent restatements exist here — C in oracle/tg_oracle.c (tgo_quantize) and numpy in
tiny-gemma_amd/weights.py — and are checked against each other and against closed-form invariants.
"""
import hashlib

import numpy as np
import pytest

import __graft_entry__ as ge
import golden_inputs as gi


@pytest.fixture(scope="module")
def tgw():
    ge.load_package()
    from tiny_gemma_amd import weights
    return weights


def test_invariants(oracle):
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((640, 256)) * 0.02).astype(np.float32)
    q, s = oracle.quantize(w)
    assert q.dtype == np.int8 and s.dtype == np.float32
    assert np.array_equal(np.abs(q.astype(np.int32)).max(axis=0), np.full(256, 127))  # every column reaches +-127
    assert np.array_equal(s, (np.abs(w).max(axis=0) / np.float32(127.0)).astype(np.float32))
    assert np.all(np.abs(w - q.astype(np.float32) * s[None, :]) <= s[None, :] * 0.5000001)
    # per column, not per row: a row-wise scale fails this
    assert not np.array_equal(s[:16], (np.abs(w).max(axis=1) / np.float32(127.0))[:16])


def test_ties_to_even(oracle):
    # scale is exactly 1 (column max 127); .5 cases must round to the even neighbour
    w = np.array([[127.0, 127.0, 127.0, 127.0], [0.5, 1.5, 2.5, -0.5], [-1.5, -2.5, 3.5, 4.5]], np.float32)
    q, s = oracle.quantize(w)
    assert np.array_equal(s, np.ones(4, np.float32))
    assert q[1].tolist() == [0, 2, 2, 0] and q[2].tolist() == [-2, -2, 4, 4]


def test_zero_column_rejected(oracle, tgw):
    w = np.ones((8, 4), np.float32)
    w[:, 2] = 0
    with pytest.raises(ZeroDivisionError):
        oracle.quantize(w)
    with pytest.raises(ZeroDivisionError):
        tgw.quantize_weight(w)


@pytest.mark.parametrize("shape", [(640, 1024), (2048, 640), (257, 33)])
def test_c_and_numpy_quantizers_agree(oracle, tgw, shape):
    rng = np.random.default_rng(shape[0])
    w = (rng.standard_normal(shape) * 0.02).astype(np.float32)
    q1, s1 = oracle.quantize(w)
    q2, s2 = tgw.quantize_weight(w)
    assert np.array_equal(q1, q2) and np.array_equal(s1, s2.reshape(-1))
    assert np.allclose(tgw.dequantize(q2, s2), w, atol=float(s2.max()) * 0.51)


def test_file_sizes(oracle, tgw):
    """437,586,944 B (270m) and 1,305,168,896 B (1B): what transformer.hpp:99-165 reads."""
    tg = ge.load_package()
    for name, total in (("270m", 437586944), ("1B", 1305168896)):
        assert oracle.weight_file_bytes(gi.oracle_config(name, None)) == total
        hidden, ffn, layers = {"270m": (640, 2048, 18), "1B": (1152, 6912, 26)}[name]
        cfg = tg.Config(hidden, ffn, layers, 262144, 32768, 512, 256, 4, 1, 1e6, 1e4, 6)
        assert tgw.weight_file_bytes(cfg) == total


def test_generator_is_deterministic_and_matches_fixture(oracle, golden, weight_images):
    img = weight_images("270m", 6, 11)
    assert hashlib.sha256(img.tobytes()).hexdigest() == str(golden["model/small6/weights_sha"])
    # counter based: any element can be recomputed on its own
    assert oracle.normal(11, 0, 12345, 0.02) == oracle.normal(11, 0, 12345, 0.02)
    assert oracle.normal(11, 0, 12345, 0.02) != oracle.normal(11, 0, 12346, 0.02)


def test_generated_file_layout(oracle, weight_images):
    """Block order and tying of the file (py/gemma.py:27-77): the int8 wte block re-quantized
    along the other axis must reproduce the lm_head block."""
    img = weight_images("270m", 6, 11)
    h, V = 640, 262144
    wte_q = img[:V * h].view(np.int8).reshape(V, h)
    wte_s = img[V * h:V * h + 4 * h].view(np.float32)
    lm_off = img.size - (h * V + 4 * V)
    lm_q = img[lm_off:lm_off + h * V].view(np.int8).reshape(h, V)
    lm_s = img[lm_off + h * V:].view(np.float32)
    assert np.abs(wte_q.astype(np.int32)).max(axis=0).min() == 127 and np.abs(lm_q.astype(np.int32)).max(axis=0).min() == 127
    # both blocks dequantize to the same fp32 matrix up to their own half-step errors
    rows = np.arange(0, V, 4099)
    a = wte_q[rows].astype(np.float32) * wte_s[None, :]
    b = (lm_q[:, rows].astype(np.float32) * lm_s[None, rows]).T
    assert np.all(np.abs(a - b) <= 0.5 * (wte_s[None, :] + lm_s[rows][:, None]) * 1.0001)
    # norm weights are fp32 N(0, 0.1), matrices int8: the final-norm block sits right after the wte scales
    rms = img[V * h + 4 * h:V * h + 8 * h].view(np.float32)
    assert 0.05 < rms.std() < 0.2


def test_numpy_generator_writes_the_same_layout(oracle, tgw, orc):
    """An image from tiny-gemma_amd/weights.py loads through the checker's reader and runs."""
    tg = ge.load_package()
    cfg = tg.Config(640, 2048, 1, 262144, 32768, 512, 256, 4, 1, 1e6, 1e4, 6)
    img = tgw.random_weight_image(cfg, 3)
    ocfg = gi.oracle_config("270m", 1)
    assert img.size == oracle.weight_file_bytes(ocfg)
    sess = oracle.model(ocfg, image=img).session()
    tok, logits, _ = sess.prefill(np.array([5, 6, 7], np.int32))
    assert np.isfinite(logits).all() and 0.2 < logits.std() < 2.0 and 0 <= tok < 262144
