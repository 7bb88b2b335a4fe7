"""CPU: pins the non-GEMM ops of oracle/tg_oracle.c against the compiled reference's outputs
(tests/golden/golden.npz) and against textbook float64 forms.

The reference is built with -ffast-math: gcc replaces 1/sqrt and vector divisions by hardware
estimates plus a Newton step and calls vectorised libm routines (powf, expf).  The restatement
uses correctly rounded operations, so these ops agree to a few ULP instead of bit for bit; the
tolerances below say how much.
"""
import numpy as np
import pytest

import golden_inputs as gi
from conftest import normrel


@pytest.mark.parametrize("name", list(gi.RMSNORM_CASES))
def test_rmsnorm(oracle, golden, name):
    rows, dim, seed = gi.RMSNORM_CASES[name]
    x, w = gi.rmsnorm_inputs(rows, dim, seed)
    y = oracle.rmsnorm(x, w)
    assert normrel(y, golden[f"rmsnorm/{name}"]) < 3e-7
    x64 = x.astype(np.float64)
    ref = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6) * (1.0 + w.astype(np.float64))  # ops.hpp:149-176
    assert normrel(y, ref) < 3e-7
    assert normrel(y, x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6) * w) > 0.5  # (1 + w), not w


@pytest.mark.parametrize("theta", [1000000.0, 10000.0])
def test_rope_tables(oracle, golden, theta):
    c, s = oracle.rope_tables(theta, 32768)
    assert np.array_equal(c[:, :128], c[:, 128:]) and np.array_equal(s[:, :128], s[:, 128:])  # decode.hpp:194-198
    p = gi.ROPE_ROWS.astype(np.float64)[:, None]
    freq = theta ** (-(2.0 * np.arange(128)) / 256.0)
    # the reference rounds freq and p*freq to fp32 before cos/sin; at p = 32767 that alone moves the angle by ~1e-3 rad
    assert np.abs(c[gi.ROPE_ROWS, :128] - np.cos(p * freq)).max() < 4e-3
    assert np.abs(c[gi.ROPE_ROWS[:6], :128] - np.cos(p[:6] * freq)).max() < 5e-5
    # vs the compiled reference (vectorised powf gives its frequencies a few ULP of their own)
    assert np.abs(c[gi.ROPE_ROWS] - golden[f"rope/{int(theta)}/cos_rows"]).max() < 8e-3
    assert np.abs(s[gi.ROPE_ROWS[:7]] - golden[f"rope/{int(theta)}/sin_rows"][:7]).max() < 3e-4
    assert np.array_equal(c[0], np.ones(256, np.float32)) and np.array_equal(s[0], np.zeros(256, np.float32))


@pytest.mark.parametrize("theta", [1000000.0, 10000.0])
def test_rope_apply(oracle, golden, theta):
    x = gi.rope_apply_input(7)
    c, s = oracle.rope_tables(theta, 2048)
    y = oracle.rope_apply(x, c, s, 1000)
    assert normrel(y, golden[f"rope/{int(theta)}/apply"]) < 2e-4  # table differences only
    # textbook rotate-half in float64 with the same tables
    c64, s64 = c[1000:1009].astype(np.float64), s[1000:1009].astype(np.float64)
    x64 = x.astype(np.float64)
    rot = np.concatenate([-x64[..., 128:], x64[..., :128]], -1)
    assert normrel(y, x64 * c64[None] + rot * s64[None]) < 2e-7
    wrong = np.concatenate([x64[..., 128:], -x64[..., :128]], -1)  # sign of the rotation swapped
    assert normrel(y, x64 * c64[None] + wrong * s64[None]) > 0.1


@pytest.mark.parametrize("size", [1024, 8192])
def test_gelu_lut(oracle, golden, size):
    t = oracle.gelu_table(-4.0, 4.0, size)
    assert np.array_equal(t, golden[f"gelu/table{size}"])
    x = gi.gelu_input(3)
    y = oracle.gelu(x, t, -4.0, 4.0)
    assert np.array_equal(y, golden[f"gelu/apply{size}"])
    # ops.hpp:41-51: the index is truncated toward zero, so (min - eps, min) still reads table[0];
    # one full step below the table gives 0, at/above the top the identity
    assert y[0] == t[0] and y[1] == 4.0 and y[2] == t[0] and y[3] == t[-1] and y[6] == 10.0 and y[7] == 0.0
    xs = np.linspace(-4, 4, size, endpoint=False)
    ref = 0.5 * xs * (1 + np.tanh(0.7978845608 * (xs + 0.044715 * xs ** 3)))
    assert np.abs(t - ref).max() < 1e-6


def test_embedding(oracle, golden):
    ids, wte, sc = gi.embedding_inputs(5)
    y = oracle.embedding(ids, wte, sc)
    assert np.array_equal(y, golden["embedding"])
    ref = wte[ids].astype(np.float64) * np.sqrt(640.0) * sc.astype(np.float64)
    assert normrel(y, ref) < 2e-7


def dense_attention(q, k, v, key_sets):
    """float64 softmax(q.k/16).v with an explicit list of key indices per query."""
    out = np.zeros(q.shape, np.float64)
    for h in range(q.shape[0]):
        for i, ks in enumerate(key_sets):
            sc = (k[ks].astype(np.float64) @ q[h, i].astype(np.float64)) / 16.0
            p = np.exp(sc - sc.max())
            out[h, i] = (p / p.sum()) @ v[ks].astype(np.float64)
    return out


@pytest.mark.parametrize("name", list(gi.ATTN_PREFILL_CASES))
def test_attention_prefill(oracle, golden, name):
    S, sw, ctx, seed = gi.ATTN_PREFILL_CASES[name]
    q, k, v = gi.attn_prefill_inputs(S, seed)
    o = oracle.attention_prefill(q, k, v, sw, ctx)
    assert normrel(o[:, gi.attn_rows(S), :], golden[f"attn_prefill/{name}"]) < 1e-6
    # local layers attend qs-ctx .. qs inclusive: ctx + 1 keys (ops.hpp:437-443)
    sets = [list(range(max(0, i - ctx) if sw else 0, i + 1)) for i in range(S)]
    assert normrel(o, dense_attention(q, k, v, sets)) < 1e-6
    if sw and S > ctx + 1:
        off_by_one = [list(range(max(0, i - ctx + 1), i + 1)) for i in range(S)]  # a ctx-key window is a different function
        assert normrel(o, dense_attention(q, k, v, off_by_one)) > 1e-3


@pytest.mark.parametrize("name", list(gi.ATTN_DECODE_CASES))
def test_attention_decode(oracle, golden, name):
    max_pos, valid, seed = gi.ATTN_DECODE_CASES[name]
    q, kc, vc = gi.attn_decode_inputs(max_pos, seed)
    o = oracle.attention_decode(q, kc, vc, valid)
    assert normrel(o, golden[f"attn_decode/{name}"]) < 3e-6
    ref = dense_attention(q[:, None, :], kc, vc, [list(range(valid))])[:, 0]
    assert normrel(o, ref) < 3e-6


def test_argmax(oracle, golden):
    lg = gi.argmax_input(9)
    assert oracle.argmax(lg) == int(golden["argmax"]) == int(np.argmax(lg))
    lg[1000] = lg[200000] = lg.max() + 1.0
    assert oracle.argmax(lg) == int(golden["argmax_tie"]) == 1000  # strict '>' scan: lowest index wins (ops.hpp:749-757)
