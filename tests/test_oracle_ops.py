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


# ---- min-p sampler (ops::minp_logits, ops.hpp:762-859) ----
def _minp_float64(lg, minp, temp, randf):
    """Textbook restatement in float64: probabilities over ALL tokens divided by the mass of the tokens at or above
    minp * max probability, then inverse-transform sampling; (index, probs, running sums).  index -1 = never reached."""
    t = lg.astype(np.float32) / np.float32(temp)            # the reference divides and subtracts the maximum in fp32
    p = np.exp((t - t.max()).astype(np.float64))
    denom = p[p >= minp * p.max()].sum()
    q = p / denom
    cum = np.cumsum(q)
    hit = np.nonzero(cum >= randf)[0]
    return (int(hit[0]) if hit.size else -1), q, cum


@pytest.mark.parametrize("name", list(gi.MINP_CASES))
def test_minp_logits_against_reference_fixture(oracle, golden, name):
    seed, scale, peaked, minp, temp, randf = gi.MINP_CASES[name]
    lg = gi.minp_input(seed, scale, peaked)
    idx, probs = oracle.minp_logits(lg, minp, temp, randf)
    assert idx == int(golden[f"minp/{name}/index"])
    ref_head = golden[f"minp/{name}/prob_head"]
    assert np.abs(probs[:256] - ref_head).max() <= 3e-6 * ref_head.max()      # the reference's exp is a vectorised libm one
    assert abs(probs.astype(np.float64).sum() - float(golden[f"minp/{name}/prob_sum"])) <= 3e-6 * float(golden[f"minp/{name}/prob_sum"])


@pytest.mark.parametrize("name", list(gi.MINP_CASES))
def test_minp_logits_against_float64_closed_form(oracle, name):
    """Pins what a plausible mistake would change: a stored mask (probabilities of below-cut tokens zeroed), a cut
    relative to the sum instead of the maximum, '>' instead of '>=' in the draw, a missing temperature."""
    seed, scale, peaked, minp, temp, randf = gi.MINP_CASES[name]
    lg = gi.minp_input(seed, scale, peaked)
    idx, probs = oracle.minp_logits(lg, minp, temp, randf)
    want, q, cum = _minp_float64(lg, minp, temp, randf)
    # fp32 effect, not a mistake: the reference's 32 sequential lane accumulators absorb terms below half an ulp of a
    # lane that holds a dominant probability, so its denominator can be low by ~1e-5 relative ("nomask": 8.8e-6)
    assert np.abs(probs - q).max() <= 2e-5 * q.max()
    seq_total = float(np.cumsum(probs, dtype=np.float32)[-1])   # what the reference's sequential fp32 scan ends at
    if seq_total < randf:
        # the fp32 running sum absorbs small terms and can end below 1 (here below randf) although the probabilities sum
        # to >= 1 in exact arithmetic: the reference then leaves index 0 (ops.hpp:850)
        assert idx == 0
    elif want < 0:
        assert cum[idx] >= randf - 3e-5
    else:
        # identical unless randf sits within fp32 summation error of a boundary of the cumulative distribution
        assert idx == want or min(abs(cum[idx] - randf), abs(cum[max(idx - 1, 0)] - randf)) < 3e-5, (idx, want)
    if name == "masked_mass":
        assert probs.astype(np.float64).sum() > 100.0     # the quirk: below-cut tokens are not removed from the draw
        assert q[idx] < minp * q.max()                    # ... and one of them is what this case draws
    if name == "never_reached":
        assert seq_total < randf and idx == 0             # ops.hpp:850: index stays 0


def test_minp_logits_limits(oracle):
    rng = np.random.default_rng(41)
    lg = rng.standard_normal(262144).astype(np.float32)
    # temperature -> 0 makes the draw the argmax for any randf that the top token's mass covers
    top = int(np.argmax(lg))
    idx, probs = oracle.minp_logits(lg, 0.0, 1e-3, 0.999)
    assert probs[top] > 0.9 and idx <= top                # the running sum crosses at the latest at the dominant token
    # one-hot distribution: every randf in (0, 1] gives that token
    hot = np.full(262144, -1e4, np.float32)
    hot[12345] = 0.0
    for r in (1e-6, 0.5, 1.0):
        assert oracle.minp_logits(hot, 0.1, 1.0, r)[0] == 12345
    # uniform distribution: the draw is floor(randf * n) up to fp32 summation error
    flat = np.zeros(262144, np.float32)
    for r in (0.25, 0.5, 0.75):
        assert abs(oracle.minp_logits(flat, 0.0, 1.0, r)[0] - r * 262144) < 64
