"""GPU: min-p / temperature sampling (ops::minp_logits, ops.hpp:762-859) through the C ABI, and the sampling
branch of gemma::generate chained on the device.

Index parity.  The reference draws the first index whose sequential fp32 running sum of 262144 probabilities
reaches randf; that scan carries ~1e-5 of rounding error of its own (and its 32-lane denominator absorbs terms
next to a dominant probability).  The GPU sums in blocks, so its index equals the checker's unless randf lies
within that fp32 summation error of a boundary of the cumulative distribution; the tests accept exactly that:
identical, or a boundary of the (float64) cumulative distribution within 3e-5 of randf on both sides of the pick.
Where the reference's running sum ends below randf (probability mass lost to absorption) it returns index 0;
the GPU's sum does not lose that mass and returns the token where the exact sum crosses.
"""
import numpy as np
import pytest

import golden_inputs as gi

pytestmark = pytest.mark.gpu

TOL = 3e-5


def near_boundary(cum64, idx, randf):
    """True if idx is the first index reaching randf for some perturbation of the running sums by < TOL."""
    lo = cum64[idx - 1] if idx > 0 else 0.0
    return lo < randf + TOL and cum64[idx] >= randf - TOL


@pytest.mark.parametrize("name", list(gi.MINP_CASES))
def test_minp_logits_matches_checker_and_fixture(tg, oracle, golden, name):
    seed, scale, peaked, minp, temp, randf = gi.MINP_CASES[name]
    lg = gi.minp_input(seed, scale, peaked)
    keep = lg.copy()
    idx = tg.minp_logits(lg, minp, temp, randf)
    assert np.array_equal(lg, keep)                      # the entry point leaves the caller's logits alone
    oidx, probs = oracle.minp_logits(lg, minp, temp, randf)
    assert oidx == int(golden[f"minp/{name}/index"])
    cum64 = np.cumsum(probs.astype(np.float64))
    if float(np.cumsum(probs, dtype=np.float32)[-1]) < randf:
        assert oidx == 0 and (idx == 0 or near_boundary(cum64, idx, randf))   # see the module docstring
    else:
        assert idx == oidx or near_boundary(cum64, idx, randf), (idx, oidx)
    if name in ("peaked", "cold", "masked_mass", "zero_draw"):
        assert idx == oidx                                # boundaries are far apart here: no excuse


def test_minp_many_draws_same_distribution(tg, oracle):
    """64 draws from one peaked distribution: every pick matches the checker's, and the picks follow the mass."""
    lg = gi.minp_input(36, 1.0, True)
    rs = np.random.default_rng(5).uniform(0.0, 1.0, 64).astype(np.float32)
    same = 0
    for r in rs:
        idx = tg.minp_logits(lg, 0.05, 0.8, float(r))
        oidx, probs = oracle.minp_logits(lg, 0.05, 0.8, float(r))
        cum64 = np.cumsum(probs.astype(np.float64))
        assert idx == oidx or near_boundary(cum64, idx, float(r))
        same += idx == oidx
    assert same >= 56                                    # draws that land in the flat tail may move by a token or two


def test_minp_argument_errors(tg):
    lg = np.zeros(262144, np.float32)
    with pytest.raises(tg.TgError):
        tg.minp_logits(lg, 0.1, 0.0, 0.5)                # temperature must be positive
    with pytest.raises(tg.TgError):
        tg.minp_logits(lg[:1000], 0.1, 1.0, 0.5)         # unsupported vocabulary size


def _small_model(tg, oracle, weight_images):
    shape, n_layers, seed, n_prompt, nd, nt, gsize = gi.MODEL_CASES["small6"]
    model = tg.Transformer(tg.named_config(shape, n_layers))
    model.read_weights_mem(weight_images(shape, n_layers, seed))
    return model, gi.prompt_ids(seed, n_prompt)


def test_sampled_generation_chained_equals_stepwise(tg, oracle, weight_images):
    """tg_generate (everything chained on the device) against the reference's loop spelled out on the host:
    forward, copy the logits back, minp_logits with the next uniform number, feed the token."""
    model, prompt = _small_model(tg, oracle, weight_images)
    n = 24
    randf = np.random.default_rng(77).uniform(0.0, 1.0, n + 1).astype(np.float32)
    minp, temp = 0.02, 0.9
    ids, _, _ = model.session().generate(prompt, n, minp, temp, randf)
    sess = model.session()
    _, logits = sess.prefill(prompt)
    step = [tg.minp_logits(logits, minp, temp, float(randf[0]))]
    for i in range(n):
        _, logits = sess.decode(step[-1])
        step.append(tg.minp_logits(logits, minp, temp, float(randf[i + 1])))
    assert ids.tolist() == step
    assert len(set(step)) > n // 2                       # it does sample: a greedy run of this model repeats itself
    # the checker's sampler on the GPU's logits of the last step agrees
    oidx, probs = oracle.minp_logits(logits, minp, temp, float(randf[n]))
    assert step[-1] == oidx or near_boundary(np.cumsum(probs.astype(np.float64)), step[-1], float(randf[n]))


def test_sampled_generation_minp_one_is_greedy(tg, oracle, weight_images):
    model, prompt = _small_model(tg, oracle, weight_images)
    greedy, _, _ = model.session().greedy(prompt, 12)
    ids, _, _ = model.session().generate(prompt, 12, 1.0, 0.7, np.zeros(13, np.float32))   # transformer.hpp:208: minp >= 1 -> argmax
    assert ids.tolist() == greedy.tolist()


def test_sampled_decode_enqueue_continues_a_session(tg, oracle, weight_images):
    """Two sampled batches in a row use their own draws from index 0, and positions advance like greedy steps."""
    model, prompt = _small_model(tg, oracle, weight_images)
    r1 = np.random.default_rng(1).uniform(0, 1, 5).astype(np.float32)
    r2 = np.random.default_rng(2).uniform(0, 1, 7).astype(np.float32)
    a = model.session()
    a.prefill(prompt, want_logits=False)
    a.decode_enqueue_sampled(5, 0.05, 1.0, r1)
    a.decode_enqueue_sampled(7, 0.05, 1.0, r2)
    ids_a = a.read_ids(13)
    b = model.session()
    b.prefill(prompt, want_logits=False)
    b.decode_enqueue_sampled(12, 0.05, 1.0, np.concatenate([r1, r2]))
    assert ids_a.tolist() == b.read_ids(13).tolist()
    assert a.position == prompt.size + 12
