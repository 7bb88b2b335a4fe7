"""GPU: one modules::attention / modules::mlp / modules::lm_head call at a time through the block-level entry points
of the C ABI, against the compiled reference's recorded outputs (tests/golden/golden_blocks.npz, written by
tests/golden/make_golden_blocks.py) on the same seeded residual streams and weights.

This is the granularity of the reference's own unit tests (tests/csrc/test_bench_modules.cpp:13-512, shape lists
tests/scripts/unittests/run_tests.sh:6-32), and their criterion (csrc/include/test_utils.hpp:34,72-76): every
|difference| below an absolute bound AND ||difference|| / ||reference|| <= 1e-3.  Here the relative bound is the one
that binds; it is asserted at 1e-3 for every block and, per kind of block, at about twice what was measured on the
MI355X (printed by each test), so that a numeric regression of 2x fails:

    attention blocks (no table lookup anywhere)      measured 5.4e-7 .. 2.2e-6   asserted 5e-6   (fp32 summation order)
    lm_head blocks                                   measured 2.9e-7 .. 4.0e-7   asserted 1e-6
    mlp blocks, 8192-entry GeLU table                measured 7.6e-7 .. 3.1e-5   asserted 8e-5
    mlp blocks, 1024-entry GeLU table                measured 6.8e-7 .. 5.8e-5   asserted 1.5e-4

The MLP figures are not summation noise: the GeLU is a step-function table lookup (csrc/include/ops.hpp:41-51), and
a last-bit difference of a gate pre-activation that sits on a table boundary selects the neighbouring entry (the
cases at 1e-6 had no such element among their rows x 2048 / 6912 gate values, the others a handful).
"""
import hashlib

import numpy as np
import pytest

import golden_inputs as gi
from conftest import CHECKER_STREAM_MISMATCHES, NEAR_TIE, check_picks, normrel

pytestmark = pytest.mark.gpu

REF_REL = 1e-3   # the reference's own relative tolerance for every block
BOUND = {"attn": 5e-6, "lm_head": 1e-6, ("mlp", 8192): 8e-5, ("mlp", 1024): 1.5e-4}
ABS_TOL = {"attn": 1.0, "mlp": 10.0, "lm_head": 0.1}   # tests/csrc/test_bench_modules.cpp:79,187,266,338,405,485


@pytest.fixture(scope="module")
def blocks():
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_blocks.npz")
    return np.load(path)


@pytest.fixture(scope="module")
def block_models(tg, oracle, blocks):
    """One-layer models of the block cases, built on first use and kept for the module."""
    cache, images = {}, {}

    def get(name):
        if name not in cache:
            cfg_o, seed = gi.block_config(name)
            shape = gi.BLOCK_MODELS[name][0]
            if (shape, seed) not in images:
                images.clear()   # one image at a time (the 1B one is 0.6 GB)
                images[(shape, seed)] = oracle.generate_weights(cfg_o, seed)
            image = images[(shape, seed)]
            assert hashlib.sha256(image.tobytes()).hexdigest() == str(blocks[f"block_model/{name}/weights_sha"])
            cfg = tg.named_config(shape, 1)
            cfg.window_pattern = cfg_o.pattern
            model = tg.Transformer(cfg)
            model.read_weights_mem(image)
            cache[name] = model
        return cache[name]

    yield get
    for m in cache.values():
        m.free()


def _session(model, tables, oracle, gsize):
    return model.session(rope=tables[0], rope_sw=tables[1], gelu_table=oracle.gelu_table(-4.0, 4.0, gsize))


@pytest.fixture(scope="module")
def tables(ref_tables):
    return ref_tables[0], ref_tables[1]


def _check(kind, gsize, got, want, what, tight=True):
    rel = normrel(got, want)
    mx = float(np.abs(np.asarray(got, np.float64) - np.asarray(want, np.float64)).max())
    bound = BOUND[kind] if kind != "mlp" else BOUND[("mlp", gsize)]
    if not tight:
        bound = REF_REL
    print(f"{what}: norm-relative {rel:.3e} (bound {bound:.0e}, reference's tolerance {REF_REL:.0e}), max |diff| {mx:.3e}", flush=True)
    assert np.isfinite(np.asarray(got)).all()
    assert rel <= REF_REL and mx <= ABS_TOL[kind]
    assert rel <= bound
    return rel


@pytest.mark.parametrize("name", list(gi.BLOCK_CASES))
def test_block_vs_compiled_reference(tg, oracle, blocks, block_models, ref_tables, tables, name):
    model_name, kind, rows, cached, gsize, seed = gi.BLOCK_CASES[name]
    tight = ref_tables[2] or kind != "attn"   # only attention reads the RoPE tables
    print(f"block case {name}", flush=True)
    sess = _session(block_models(model_name), tables, oracle, gsize)
    x, k, v = gi.block_inputs(name)
    if cached:
        sess.kv_prefill(0, k, v)
    if kind == "lm_head":
        y = sess.block_lm_head(x)
        _check(kind, gsize, y[:4096], blocks[f"block/{name}/head"], name + " head")
        _check(kind, gsize, y[gi.LOGIT_SAMPLE], blocks[f"block/{name}/sample"], name + " sample")
        assert abs(np.linalg.norm(y.astype(np.float64)) / float(blocks[f"block/{name}/norm"]) - 1.0) < 1e-5
        assert int(np.argmax(y)) == int(blocks[f"block/{name}/argmax"])
        return
    y = sess.block_attention(0, x) if kind == "attn" else sess.block_mlp(0, x)
    _check(kind, gsize, y[gi.block_rows(rows)], blocks[f"block/{name}/rows"], name, tight)
    assert abs(np.linalg.norm(y.astype(np.float64)) / float(blocks[f"block/{name}/norm"]) - 1.0) < 1e-4
    if kind == "attn":
        kk, vv, pp, bp = sess.kv(0)
        assert (pp, bp) == tuple(int(t) for t in blocks[f"block/{name}/kv_ptrs"])
        slot = (bp - 1) % kk.shape[0]
        assert normrel(kk[slot], blocks[f"block/{name}/k_last"]) < (5e-6 if tight else REF_REL)
        assert normrel(vv[slot], blocks[f"block/{name}/v_last"]) < 5e-6


def test_block_entry_points_reject_bad_calls(tg, oracle, block_models, tables):
    sess = _session(block_models("270m_global"), tables, oracle, 1024)
    x = np.zeros((4, 640), np.float32)
    with pytest.raises(tg.TgError) as e:
        sess.block_attention(1, x)          # the model has one layer
    assert e.value.code == -4
    sess.block_attention(0, x)
    with pytest.raises(tg.TgError) as e:    # a second prefill-style call on a used cache (decode.hpp:78-79)
        sess.block_attention(0, x)
    assert e.value.code == -7
    with pytest.raises(tg.TgError) as e:    # cache rows for a position other than the session's
        sess.kv_prefill(0, np.zeros((9, 256), np.float32), np.zeros((9, 256), np.float32))
    assert e.value.code == -7


# ---- teacher-forced random-token streams through the full models ----

@pytest.mark.parametrize("name", list(gi.STREAM_CASES))
def test_teacher_forced_random_token_stream(tg, oracle, blocks, weight_images, tables, name):
    """Seeded random ids are fed step by step, so every step sees a fresh context: the reference's picks take ~190
    distinct values over 321 steps, against 2-8 for a free-running greedy run of a random-init model.  Every pick must
    be the compiled reference's, except at a near-tie of the reference (conftest.check_picks).  Observed on the MI355X
    with the 1024-entry table: 6 of 321 picks differ on each shape, at reference gaps 2.4e-4 .. 8.0e-3 (earlier versions
    of the prefill attention: 7 + 7 and 6 + 3 at other steps, up to 1.0e-2 - which near-ties flip depends on the last
    bits of every operation), logits 3.8e-3 .. 4.5e-3 from the reference's; with the near-continuous table no pick
    differs on either shape (the smallest reference gap is 2.1e-4) and the logits agree to 6.4e-6 .. 1.0e-5."""
    shape, n_layers, seed, n_prompt, steps, gsize = gi.STREAM_CASES[name]
    fine = gsize > 8192
    print(f"stream case {name}", flush=True)
    image = weight_images(shape, n_layers, seed)
    assert hashlib.sha256(image.tobytes()).hexdigest() == str(blocks[f"stream/{name}/weights_sha"])
    model = tg.Transformer(tg.named_config(shape, n_layers))
    model.read_weights_mem(image)
    sess = model.session(rope=tables[0], rope_sw=tables[1], gelu_table=oracle.gelu_table(-4.0, 4.0, gsize))
    prompt, feed = gi.stream_ids(name)
    ref = blocks[f"stream/{name}/picks"]
    gaps = blocks[f"stream/{name}/top2_gaps"]
    pairs = blocks[f"stream/{name}/top2_ids"]
    heads = blocks[f"stream/{name}/logits_head"]
    tok, _ = sess.prefill(prompt, want_logits=False)
    picks, rels = [tok], []
    for i in range(steps):
        want = i in gi.STREAM_LOGIT_STEPS
        tok, lg = sess.decode(int(feed[i]), want_logits=want)
        picks.append(tok)
        if want:
            rels.append(normrel(lg[:4096], heads[gi.STREAM_LOGIT_STEPS.index(i)]))
    print(f"{name}: logits head norm-relative at steps {gi.STREAM_LOGIT_STEPS}: " + ", ".join(f"{r:.2e}" for r in rels), flush=True)
    # near-continuous table: fp32 summation order is all that is left and no pick may differ
    # coarse table: runner-up picks are small-number draws (CPU checker 4 and 7 of 321, this library 6 and 6, earlier
    # kernels 7 + 7 and 6 + 3): at most twice the strict-IEEE checker's count on the same stream, plus two
    check_picks(picks, ref, gaps, pairs, name, near_tie=1e-3 if fine else NEAR_TIE,
                max_mismatches=0 if fine else 2 * CHECKER_STREAM_MISMATCHES[name] + 2)
    assert max(rels) < (2e-5 if fine else 9e-3)
    sess.free()
    model.free()


# ---- greedy argmax: exact ties and the all-NaN row ----

def _lm_head_view(image, cfg_o):
    V, h = cfg_o.vocab, cfg_o.hidden
    lm_off = image.size - (h * V + 4 * V)
    W = image[lm_off:lm_off + h * V].view(np.int8).reshape(h, V)
    s = image[lm_off + h * V:].view(np.float32)
    return W, s


@pytest.mark.parametrize("c1,c2", [(8, 9), (8, 40), (8, 100), (8, 128 + 8), (5, 262143), (262016, 262143)],
                         ids=["same_lane_group", "same_wave", "other_wave", "next_workgroup", "first_and_last_tile", "last_tile"])
def test_argmax_exact_tie_takes_the_lowest_index(tg, oracle, c1, c2):
    """ops::argmax_logits scans with a strict '>' from index 0 (ops.hpp:749-757): among equal maxima the lowest
    index wins.  The LM head's columns c1 < c2 are made byte-identical copies (weights and scale) of the column that
    wins on the unmodified model, for the prefill logits and for the logits of a decode step, so the maximum is
    attained three times, bit for bit; the pairs sit in one lane's four columns, in one wave, in two waves of a
    workgroup, in two workgroups, in the first and last tile.  Both launch paths: the prefill's LM head +
    finishing launch, and the decode step's."""
    cfg_o = gi.oracle_config("270m", 2)
    image = oracle.generate_weights(cfg_o, 71).copy()
    cfg = tg.named_config("270m", 2)
    prompt = gi.prompt_ids(71, 9)
    fed = 12345

    def run(img):
        model = tg.Transformer(cfg)
        model.read_weights_mem(img)
        sess = model.session(gsize=1024)
        tp, lp = sess.prefill(prompt)
        td, ld = sess.decode(fed)
        sess.free()
        model.free()
        return tp, lp, td, ld

    a_p, lp, a_d, ld = run(image)
    assert a_p == int(np.argmax(lp)) and a_d == int(np.argmax(ld))
    W, s = _lm_head_view(image, cfg_o)
    # c1, c2 := the prefill winner; c1 + 2, c2 - 2 := the decode winner (pairs with the same geometry)
    d1, d2 = c1 + 2, c2 - 2
    assert not {a_p, a_d} & {c1, c2, d1, d2}
    for dst in (c1, c2):
        W[:, dst] = W[:, a_p]
        s[dst] = s[a_p]
    for dst in (d1, d2):
        W[:, dst] = W[:, a_d]
        s[dst] = s[a_d]
    tp, lp2, td, ld2 = run(image)
    assert lp2[c1] == lp2[c2] == lp2[a_p] == lp2.max()       # a real three-way tie, bit for bit
    assert ld2[d1] == ld2[d2] == ld2[a_d] == ld2.max()
    want_p = int(np.flatnonzero(lp2 == lp2.max())[0])        # the lowest index among the maxima
    want_d = int(np.flatnonzero(ld2 == ld2.max())[0])
    assert want_p <= min(a_p, c1) and want_d <= min(a_d, d2, d1)
    assert tp == want_p, (tp, want_p)
    assert td == want_d, (td, want_d)


def test_argmax_of_an_all_nan_row_is_minus_one(tg, oracle):
    """With every logit NaN no comparison of the reference's scan is true and its index stays at its initial -1
    (ops.hpp:749-757).  A NaN in the final norm's weights makes every logit NaN."""
    cfg_o = gi.oracle_config("270m", 2)
    image = oracle.generate_weights(cfg_o, 71).copy()
    V, h = cfg_o.vocab, cfg_o.hidden
    rmsw = image[V * h + 4 * h:V * h + 8 * h].view(np.float32)   # transformer.hpp:122-126: wte, its scales, then RMSw
    rmsw[:] = np.nan
    model = tg.Transformer(tg.named_config("270m", 2))
    model.read_weights_mem(image)
    sess = model.session(gsize=1024)
    tok, lg = sess.prefill(gi.prompt_ids(71, 9))
    assert np.isnan(lg).all() and tok == -1
    tok, lg = sess.decode(77)
    assert np.isnan(lg).all() and tok == -1
    # the id fed back by a chained decode is clamped into the vocabulary: the next step still runs
    sess.decode_enqueue(1)
    tg.synchronize()
    assert sess.read_ids(8)[-1] == -1
    sess.free()
    model.free()


# ---- a model and its sessions ----

def test_model_outlives_its_sessions_or_disables_them(tg, oracle, weight_images, tmp_path):
    """Weights are neither reloaded nor freed under a live session: a reload is refused, and after the model is
    destroyed every call on the surviving session returns TG_ERR_STATE instead of launching on freed memory."""
    image = weight_images("270m", 2, 31)
    model = tg.Transformer(tg.named_config("270m", 2))
    model.read_weights_mem(image)
    sess = model.session(gsize=1024)
    tok, _ = sess.prefill(gi.prompt_ids(3, 5), want_logits=False)
    for reload in (lambda: model.read_weights_mem(image), lambda: model.read_weights(str(tmp_path / "missing.bin"))):
        with pytest.raises(tg.TgError) as e:
            reload()
        assert e.value.code in (-7, -2)     # live session -> TG_ERR_STATE (a missing file is reported first)
    t2, _ = sess.decode(tok, want_logits=False)          # the session still works on the old weights
    assert t2 >= 0
    model.free()                                         # tg_model_destroy under a live session
    for call in (lambda: sess.decode(tok), lambda: sess.decode_enqueue(2), lambda: sess.block_mlp(0, np.zeros((1, 640), np.float32)),
                 lambda: sess.prefill(gi.prompt_ids(3, 5))):
        with pytest.raises(tg.TgError) as e:
            call()
        assert e.value.code == -7
    sess.free()                                          # the last session deletes the orphaned model
    # a model whose load failed has no weights: no session can be made from it
    m2 = tg.Transformer(tg.named_config("270m", 2))
    short = tmp_path / "short.bin"
    image[:1_000_000].tofile(short)
    with pytest.raises(tg.TgError):
        m2.read_weights(str(short))
    with pytest.raises(tg.TgError) as e:
        m2.session()
    assert e.value.code == -7
    m2.free()
