"""GPU: forward_prefill / forward_decode / greedy generation through the C ABI against the CPU
checker on the same weights, prompts and tables, and against the compiled reference's recorded
token ids (tests/golden/golden.npz).

Tolerances.  All arithmetic is fp32 on both sides; summation orders differ.  Every bound is about twice what the
MI355X run measured (the tests print the measured values).  With a near-continuous GeLU table (2^20 entries) the
two agree to fp32 rounding end to end: first block 5e-7 .. 1.05e-6 (bound 2.5e-6), every block and the logits
<= 6e-6 after 6 layers (bound 1.5e-5).  With the reference command line's 1024-entry step-function table
(csrc/include/ops.hpp:22-52) an ULP upstream can move a gate activation to the next table entry; the compiled
reference and the strict-IEEE checker differ from each other by the same mechanism (tests/conftest.py, check_picks):
6 layers 2.8e-3 (bound 5e-3), 18 / 26 layers against the reference's recordings 4.1e-3 / 3.7e-3 (bound 8e-3).
Greedy picks: the reference's, or its runner-up at a near-tie of the reference.  Observed: 270m shape 64 + 256
free-running picks identical; 1B shape 178 + 1024 free-running picks identical up to step 771, where the reference's
top-2 gap is 8.4e-3 and the library takes its runner-up; teacher-forced, that step is the only one of 1025 that differs;
near-tie seed of the 270m shape: 1 of 257 (gap 3.2e-4).
"""
import numpy as np
import pytest

import golden_inputs as gi
from conftest import NEAR_TIE, check_picks, normrel

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tables(oracle):
    cg, sg = oracle.rope_tables(1000000.0, 32768)
    cl, sl = oracle.rope_tables(10000.0, 32768)
    return (cg, sg), (cl, sl)


def build(tg, oracle, weight_images, tables, name, own_tables=False):
    shape, n_layers, seed, n_prompt, nd, nt, gsize = gi.MODEL_CASES[name]
    image = weight_images(shape, n_layers, seed)
    model = tg.Transformer(tg.named_config(shape, n_layers))
    model.read_weights_mem(image)
    if own_tables:
        sess = model.session(gsize=gsize)
    else:
        sess = model.session(rope=tables[0], rope_sw=tables[1], gelu_table=oracle.gelu_table(-4.0, 4.0, gsize))
    osess = oracle.model(gi.oracle_config(shape, n_layers), image=image).session(-4.0, 4.0, gsize)
    return model, sess, osess, gi.prompt_ids(seed, n_prompt)


def compare_run(sess, osess, prompt, n_decode, tol, tol_first, what=""):
    tok, logits = sess.prefill(prompt)
    otok, ologits, otaps = osess.prefill(prompt, taps=True)
    taps = sess.taps(rows=prompt.size)
    assert taps.shape[0] == otaps.shape[0] + 1
    first = normrel(taps[1], otaps[0])
    assert first < tol_first      # attention block of layer 0: nothing discontinuous upstream
    worst = max(normrel(taps[b + 1], otaps[b]) for b in range(otaps.shape[0]))
    assert worst < tol, worst
    worst_logits = normrel(logits, ologits)
    assert worst_logits < tol
    assert tok == otok
    toks = [tok]
    for _ in range(n_decode):
        tok, logits = sess.decode(toks[-1])
        otok, ologits, otp = osess.decode(toks[-1], taps=True)
        dt = sess.taps(rows=1)[:, 0, :]
        worst = max(worst, max(normrel(dt[b + 1], otp[b]) for b in range(otp.shape[0])))
        worst_logits = max(worst_logits, normrel(logits, ologits))
        assert normrel(logits, ologits) < tol
        assert tok == otok
        toks.append(tok)
    print(f"{what} {prompt.size} tokens + {n_decode} steps against the CPU checker: first block {first:.2e} (bound {tol_first:.0e}), "
          f"worst block {worst:.2e}, worst logits {worst_logits:.2e} (bound {tol:.0e})", flush=True)
    assert worst < tol, worst
    return np.array(toks, np.int32), worst


def test_prefill_exact_gemm_mode(tg, oracle, golden, weight_images, tables):
    """The forward with the exact-order vector-ALU GEMM (tg_set_gemm_mode(0)) instead of MFMA."""
    tg.lib().tg_set_gemm_mode(0)
    try:
        model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "small6_finelut")
        compare_run(sess, osess, prompt, 2, tol=1.5e-5, tol_first=2.5e-6)
    finally:
        tg.lib().tg_set_gemm_mode(1)


def test_embedding_tap_is_exact(tg, oracle, weight_images, tables):
    model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "small6")
    sess.prefill(prompt, want_logits=False)
    image = weight_images("270m", 6, 11)
    wte = image[:262144 * 640].view(np.int8).reshape(262144, 640)
    sc = image[262144 * 640:262144 * 640 + 4 * 640].view(np.float32)
    assert np.array_equal(sess.tap(0, rows=prompt.size), oracle.embedding(prompt, wte, sc))


def test_small_model_fine_table(tg, oracle, golden, weight_images, tables):
    model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "small6_finelut")
    toks, worst = compare_run(sess, osess, prompt, 12, tol=1.5e-5, tol_first=2.5e-6, what="small6 (near-continuous table)")
    assert np.array_equal(toks, golden["model/small6_finelut/tokens"])
    # and against the compiled reference's own activations (its rope tables differ in the last bits)
    sess.reset()
    sess.prefill(prompt)
    taps = sess.taps(rows=prompt.size)[1:]
    assert normrel(taps[:, gi.tap_rows(prompt.size), :], golden["model/small6_finelut/prefill_taps"]) < 2e-4


def test_small_model_cli_table(tg, oracle, golden, weight_images, tables):
    model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "small6")
    toks, worst = compare_run(sess, osess, prompt, 12, tol=5e-3, tol_first=2.5e-6, what="small6 (1024-entry table)")
    assert np.array_equal(toks, golden["model/small6/tokens"])


def test_library_built_tables(tg, oracle, golden, weight_images, tables):
    """NULL tables: the library computes RoPE and GeLU tables itself (decode.hpp:176-201, ops.hpp:29-39)."""
    model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "small6_finelut", own_tables=True)
    toks, worst = compare_run(sess, osess, prompt, 4, tol=1.5e-5, tol_first=2.5e-6)


@pytest.mark.parametrize("n_prompt", [1, 2, 3, 17, 33, 65, 129, 257])
def test_ragged_prompt_lengths(tg, oracle, weight_images, tables, n_prompt):
    """Prompt lengths that fill no tile of any kernel: one token, odd counts (the finishing launch of the attention
    takes two rows per workgroup), one past a 16-query / 32-key / 128-row boundary.  Two layers, near-continuous
    GeLU table: every tap and the logits against the checker, then two decode steps from the caches it left."""
    image = weight_images("270m", 2, 31)
    model = tg.Transformer(tg.named_config("270m", 2))
    model.read_weights_mem(image)
    gsize = 1 << 20
    sess = model.session(rope=tables[0], rope_sw=tables[1], gelu_table=oracle.gelu_table(-4.0, 4.0, gsize))
    osess = oracle.model(gi.oracle_config("270m", 2), image=image).session(-4.0, 4.0, gsize)
    compare_run(sess, osess, gi.prompt_ids(40 + n_prompt, n_prompt), 2, tol=1.5e-5, tol_first=2.5e-6)


def test_prompt_longer_than_window(tg, oracle, golden, weight_images, tables):
    """600-token prompt on a model with 512-slot ring caches: 513-key window in prefill
    (ops.hpp:437-443), ring of 512 in decode, tail of the prompt in slots 0..511 (decode.hpp:84-104)."""
    model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "small6_window")
    nd = gi.MODEL_CASES["small6_window"][4]
    tok, logits = sess.prefill(prompt)
    otok, ologits, otaps = osess.prefill(prompt, taps=True)
    taps = sess.taps(rows=prompt.size)
    assert normrel(taps[1], otaps[0]) < 3e-6
    assert normrel(taps[1:], otaps) < 5e-3 and normrel(logits, ologits) < 5e-3 and tok == otok
    k0, v0, pp, bp = sess.kv(0)
    ok0, ov0, opp, obp = osess.kv(0)
    assert (pp, bp) == (opp, obp) == (600, 512)
    assert normrel(k0, ok0) < 3e-6 and normrel(v0, ov0) < 3e-6  # layer 0: rows 88..599 of the prompt in slots 0..511
    toks = [tok]
    for _ in range(nd):
        tok, logits = sess.decode(toks[-1])
        otok, ologits, _ = osess.decode(toks[-1])
        assert tok == otok and normrel(logits, ologits) < 5e-3
        toks.append(tok)
    assert np.array_equal(np.array(toks, np.int32), golden["model/small6_window/tokens"])
    for layer in (0, 5):
        k, v, pp, bp = sess.kv(layer)
        ok, ov, opp, obp = osess.kv(layer)
        assert (pp, bp) == (opp, obp)
        n = 512 if layer == 0 else 600 + nd
        assert normrel(k[:n], ok[:n]) < 5e-3 and normrel(v[:n], ov[:n]) < 5e-3
    assert (sess.kv(0)[2], sess.kv(0)[3]) == (600 + nd, 512 + nd)


def test_decode_from_empty_session(tg, oracle, weight_images, tables):
    """forward_decode without a prefill: position 0, a single key."""
    model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "small6_finelut")
    tok = int(prompt[0])
    for _ in range(3):
        t, lg = sess.decode(tok)
        ot, olg, _ = osess.decode(tok)
        assert t == ot and normrel(lg, olg) < 1.5e-5
        tok = t
    assert sess.position == 3


def greedy_vs_golden(sess, golden, name, prompt, n_decode, strict=True):
    """Free-running greedy ids against the compiled reference's.  strict: identical over the whole horizon.
    Otherwise a divergence may only start at a near-tie of the reference, with the reference's runner-up
    (after it the two runs legitimately see different contexts).  Returns the first differing step or -1."""
    toks, s_prefill, s_decode = sess.greedy(prompt, n_decode)
    ref = golden[f"model/{name}/tokens"]
    gaps = golden[f"model/{name}/top2_gaps"]
    mism = np.nonzero(toks != ref)[0]
    if mism.size == 0:
        print(f"{name}: free-running greedy ids identical to the reference's over {n_decode + 1} picks "
              f"(its smallest top-2 gap: {float(gaps.min()):.2e})", flush=True)
        return -1
    i = int(mism[0])
    msg = f"{name}: free-running greedy ids leave the reference's at step {i} (reference top-2 gap there: {gaps[i]:.3e})"
    print(msg, flush=True)
    assert not strict, msg
    assert gaps[i] < NEAR_TIE and toks[i] == golden[f"model/{name}/top2_ids"][i][1], msg
    return i


def teacher_forced_vs_golden(sess, golden, name, prompt, n_decode, max_mismatches=None):
    """Fed the reference's ids step by step, every pick must be the reference's; at a near-tie of the reference
    its runner-up is the only other acceptable answer (conftest.check_picks)."""
    ref = golden[f"model/{name}/tokens"]
    tok, _ = sess.prefill(prompt, want_logits=False)
    picks = [tok]
    for i in range(n_decode):
        tok, _ = sess.decode(int(ref[i]), want_logits=False)
        picks.append(tok)
    return check_picks(picks, ref, golden[f"model/{name}/top2_gaps"], golden[f"model/{name}/top2_ids"], name + " teacher-forced",
                       max_mismatches=max_mismatches)


def check_weights(golden, weight_images, name):
    import hashlib
    shape, n_layers, seed = gi.MODEL_CASES[name][:3]
    assert hashlib.sha256(weight_images(shape, n_layers, seed).tobytes()).hexdigest() == str(golden[f"model/{name}/weights_sha"])


def test_full_270m_greedy_ids(tg, oracle, golden, weight_images, tables):
    """64-token prompt + 256 greedy steps, 18 layers: ids identical to the compiled reference."""
    check_weights(golden, weight_images, "full270m")
    model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "full270m")
    greedy_vs_golden(sess, golden, "full270m", prompt, 256)
    sess.reset()
    tok, logits = sess.prefill(prompt)
    # 18 layers of the 1024-entry table: the checker itself sits 4e-3 from the compiled reference here
    rel = normrel(logits[:4096], golden["model/full270m/prefill_logits_head"])
    print(f"full270m: prefill logits head against the reference's {rel:.2e}", flush=True)
    assert rel < 8e-3


def test_full_270m_near_ties(tg, oracle, golden, weight_images, tables):
    """A seed whose greedy path crosses near-ties of the reference's own logits (top-2 gaps down to
    3e-4 against a logit spread of 0.5).  Teacher-forced with the reference's ids, every step must
    pick the reference's id, except that at a near-tie (gap < conftest.NEAR_TIE) the reference's runner-up is the
    only other acceptable answer."""
    check_weights(golden, weight_images, "full270m_ties")
    model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "full270m_ties")
    teacher_forced_vs_golden(sess, golden, "full270m_ties", prompt, 256, max_mismatches=3)


def test_full_1b_greedy_ids(tg, oracle, golden, weight_images, tables):
    """178-token prompt + 1024 greedy steps, 26 layers (the benchmark workload).  Over 1024 steps of 26 layers with the
    1024-entry GeLU table the logits sit ~4e-3 from the compiled reference's (so does the strict-IEEE CPU checker), and
    the reference's own path crosses top-2 gaps of that size (1e-3 at the smallest): the free run may leave the
    reference's path at such a near-tie, by picking its runner-up; teacher-forced, every other pick must be identical."""
    if "model/full1B/tokens" not in golden:
        pytest.skip("fixture was written without the 1B case")
    check_weights(golden, weight_images, "full1B")
    model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "full1B")
    first = greedy_vs_golden(sess, golden, "full1B", prompt, 1024, strict=False)
    assert first < 0 or first >= 394                     # not early: the reference's smallest top-2 gap before step 394 is 0.105
    sess.reset()
    teacher_forced_vs_golden(sess, golden, "full1B", prompt, 1024, max_mismatches=4)
    # last-position activations of the prefill against the reference's
    sess.reset()
    tok, logits = sess.prefill(prompt)
    rel = normrel(logits[:4096], golden["model/full1B/prefill_logits_head"])
    last = sess.taps(rows=prompt.size)[1:, -1, :]
    want = golden["model/full1B/prefill_taps_last"]
    per_block = [normrel(last[b], want[b]) for b in range(want.shape[0])]
    print(f"full1B: prefill logits head against the reference's {rel:.2e}; last-row residuals: worst block {max(per_block):.2e}", flush=True)
    assert rel < 8e-3 and max(per_block) < 8e-3


def test_graph_replay_equals_stream_launches(tg, oracle, weight_images, tables):
    """HIP-graph replay must give the same bits as plain launches, on every replay: mode 1 (a captured step that reads
    its position from device memory) and mode 2 (a captured step of the stream path's own launches whose attention,
    merge and output-projection nodes get the position's parameters before every replay)."""
    model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "small6")
    results = []
    for graphs in (0, 1, 1, 2, 2):
        tg.lib().tg_set_graphs(graphs)
        sess.reset()
        sess.prefill(prompt, want_logits=False)
        chunks = []
        for n in (1, 5, 9):  # several enqueue calls with host work and synchronisation between replays
            sess.decode_enqueue(n)
            tg.synchronize()
            chunks.append(sess.taps(rows=1).copy())
        results.append((sess.read_ids(16).copy(), chunks))
    tg.lib().tg_set_graphs(-1)
    for ids, chunks in results[1:]:
        assert np.array_equal(ids, results[0][0])
        for a, b in zip(chunks, results[0][1]):
            assert np.array_equal(a, b)


def test_updated_graph_replay_across_attention_geometries(tg, oracle):
    """Graph replay with node updates over 80 steps that start at 990 keys: the global layer's chunk grows with the
    context (a parameter of its nodes, not another graph) and at 1025 keys its attention gets a merge launch (another
    graph).  Ids, residual stream and cache rows as with plain launches, bit for bit; sampled steps (always plain
    launches) and a stepwise call in between."""
    cfg = tg.named_config("270m", 6)   # layer 5 is a global one
    model = tg.Transformer(cfg)
    model.read_weights_mem(oracle.generate_weights(gi.oracle_config("270m", 6), 43))
    sess = model.session()
    prompt = gi.prompt_ids(53, 990)
    L = tg.lib()
    out = []
    try:
        for graphs in (0, 2):
            tg.check(L.tg_set_graphs(graphs))
            sess.reset()
            sess.prefill(prompt, want_logits=False)
            for n in (1, 30, 7):
                sess.decode_enqueue(n)
            sess.decode_enqueue_sampled(3, 0.05, 1.0, np.array([0.3, 0.6, 0.9], np.float32))
            tok, _ = sess.decode(int(sess.read_ids(64)[-1]), want_logits=False)
            sess.decode_enqueue(38)
            tg.synchronize()
            out.append((sess.read_ids(128).copy(), sess.taps(rows=1).copy(), sess.position, [sess.kv(l) for l in (0, 5)]))
    finally:
        tg.check(L.tg_set_graphs(-1))
    (ids_a, taps_a, pos_a, kv_a), (ids_b, taps_b, pos_b, kv_b) = out
    assert pos_a == pos_b == 990 + 80 and ids_a.size == ids_b.size and np.array_equal(ids_a, ids_b)
    assert np.array_equal(taps_a, taps_b)
    for (k0, v0, p0, b0), (k1, v1, p1, b1) in zip(kv_a, kv_b):
        assert (p0, b0) == (p1, b1) and np.array_equal(k0, k1) and np.array_equal(v0, v1)


def test_chained_picks_equal_a_finishing_launch_per_step(tg, oracle, weight_images, tables):
    """Inside one tg_decode_enqueue call the first launch of a step finishes the previous step's greedy pick (second
    stage of the argmax, token log, counters) instead of a launch of its own.  Same ids, same residual stream, same
    counters as with a finishing launch per step; batches of 1 (nothing to chain), 2 and many; stepwise calls and
    sampled steps in between."""
    model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "small6")
    results = []
    try:
        for chain in (0, 1):
            tg.check(tg.lib().tg_set_chain_picks(chain))
            sess.reset()
            tok, _ = sess.prefill(prompt, want_logits=False)
            for n in (1, 2, 17):
                sess.decode_enqueue(n)
            tok, _ = sess.decode(int(sess.read_ids(64)[-1]), want_logits=False)   # a stepwise call between batches
            sess.decode_enqueue(5)
            sess.decode_enqueue_sampled(3, 0.05, 1.0, np.array([0.3, 0.6, 0.9], np.float32))
            sess.decode_enqueue(4)
            tg.synchronize()
            results.append((sess.read_ids(64).copy(), sess.taps(rows=1).copy(), sess.position, sess.kv(5)[2:]))
    finally:
        tg.check(tg.lib().tg_set_chain_picks(1))
    (ids_a, taps_a, pos_a, ptr_a), (ids_b, taps_b, pos_b, ptr_b) = results
    assert ids_a.size == 1 + 1 + 2 + 17 + 1 + 5 + 3 + 4 and np.array_equal(ids_a, ids_b)
    assert np.array_equal(taps_a, taps_b) and pos_a == pos_b == prompt.size + 33 and ptr_a == ptr_b


@pytest.mark.parametrize("n_prompt", [1100, 4100])
def test_long_context_merge_path(tg, oracle, weight_images, tables, n_prompt):
    """More than 1024 keys on a global layer: 32-key workgroups plus the merge launch, which folds groups of 64
    partials (1100 keys: one partly filled group; 4100 keys: two full groups and a group of one)."""
    cfg_o = gi.oracle_config("270m", 2)
    cfg_o.pattern = 2  # layer 0 local, layer 1 global
    image = oracle.generate_weights(cfg_o, 21)
    cfg = tg.named_config("270m", 2)
    cfg.window_pattern = 2
    model = tg.Transformer(cfg)
    model.read_weights_mem(image)
    table = oracle.gelu_table(-4.0, 4.0, 1 << 20)
    sess = model.session(rope=tables[0], rope_sw=tables[1], gelu_table=table)
    osess = oracle.model(cfg_o, image=image).session(-4.0, 4.0, 1 << 20)
    prompt = gi.prompt_ids(21, n_prompt)
    tok, logits = sess.prefill(prompt)
    otok, ologits, _ = osess.prefill(prompt)
    worst = normrel(logits, ologits)
    assert tok == otok
    for _ in range(3):
        t, lg = sess.decode(tok)
        ot, olg, _ = osess.decode(tok)
        assert t == ot
        worst = max(worst, normrel(lg, olg))
        tok = t
    print(f"{n_prompt}-token prompt + 3 steps (merge path): worst logits against the CPU checker {worst:.2e} (bound 1.5e-5)", flush=True)
    assert worst < 1.5e-5


def test_error_paths(tg, oracle, weight_images, tables, tmp_path):
    model, sess, osess, prompt = build(tg, oracle, weight_images, tables, "small6")
    sess.prefill(prompt[:8], want_logits=False)
    with pytest.raises(tg.TgError) as e:       # one prefill per DecodeState (decode.hpp:78-79)
        sess.prefill(prompt[:8], want_logits=False)
    assert e.value.code == -7
    m2 = tg.Transformer(tg.named_config("270m", 6))
    with pytest.raises(tg.TgError) as e:       # transformer.hpp:163
        m2.read_weights(str(tmp_path / "missing.bin"))
    assert e.value.code == -2 and "Could not open file." in str(e.value)
    short = tmp_path / "short.bin"
    weight_images("270m", 6, 11)[:10_000_000].tofile(short)
    with pytest.raises(tg.TgError) as e:
        m2.read_weights(str(short))
    assert e.value.code == -3
    with pytest.raises(tg.TgError) as e:       # no weights yet
        m2.session()
    assert e.value.code == -7
    bad = tg.named_config("270m", 2)
    bad.hidden_size = 512
    with pytest.raises(tg.TgError) as e:
        tg.Transformer(bad)
    assert e.value.code == -1


@pytest.mark.parametrize("n_prompt", [90, 700, 2100])
def test_prefill_attention_modes_agree_inside_the_forward(tg, oracle, n_prompt):
    """The prefill attention kernels (fp32 matrix path with 16-query workgroups; the split path with 16 and with 32,
    staged or fed from pre-split plane images, in both operand formats) behind the same work lists and the same
    finishing launch: same id, logits within fp32 rounding of each other.  700 tokens: local layers with their own (windowed) work list;
    2100: plane images by default."""
    cfg = tg.named_config("270m", 2)
    model = tg.Transformer(cfg)
    model.read_weights_mem(oracle.generate_weights(gi.oracle_config("270m", 2), 24))
    sess = model.session(gsize=1 << 20)
    prompt = gi.prompt_ids(36, n_prompt)
    out = {}
    L = tg.lib()
    # (kernel mode, planes, operand format); (2, 2, 1) is the kernel on 32x32x16 matrix instructions
    combos = [(1, 0, 1), (0, 0, 1), (2, 0, 1), (3, 2, 1), (2, 2, 1), (2, 2, 2), (1, 0, 0), (2, 2, 0)]
    try:
        for mode, planes, f16 in combos:
            tg.check(L.tg_set_attn_prefill_mode(mode))
            tg.check(L.tg_set_attn_prefill_planes(planes))
            tg.check(L.tg_set_attn_prefill_format(f16))
            sess.reset()
            out[(mode, planes, f16)] = sess.prefill(prompt)
    finally:
        tg.check(L.tg_set_attn_prefill_mode(1))
        tg.check(L.tg_set_attn_prefill_planes(1))
        tg.check(L.tg_set_attn_prefill_format(1))
    for key in combos[1:]:
        assert out[key][0] == out[combos[0]][0]
        assert normrel(out[key][1], out[combos[0]][1]) < 2e-5
    # the plane images hold the same planes the staging code computes: not a bit differs
    assert np.array_equal(out[(2, 2, 2)][1], out[(2, 0, 1)][1])
    # ... and the 32x32x16 kernel sums in another order: other last bits, which shows that it is the one that ran
    assert not np.array_equal(out[(2, 2, 1)][1], out[(2, 2, 2)][1])


def test_one_session_many_prompt_lengths(tg, oracle):
    """A session keeps its prefill workspace and the attention work lists of the last prompt length; prompts of other
    lengths in between (shorter: lists rebuilt, workspace reused; longer: both regrown; workspace released) must not
    change what a length gives: the same bits every time."""
    cfg = tg.named_config("270m", 2)
    model = tg.Transformer(cfg)
    model.read_weights_mem(oracle.generate_weights(gi.oracle_config("270m", 2), 25))
    sess = model.session(gsize=1024)
    prompts = {n: gi.prompt_ids(37, n) for n in (700, 90, 2100, 1)}
    first = {}
    for step, n in enumerate([700, 90, 2100, 700, 1, 90, 2100, 700]):
        if step == 5:
            sess.release_workspace()
        sess.reset()
        tok, logits = sess.prefill(prompts[n])
        nxt, _ = sess.decode(tok)
        if n in first:
            assert tok == first[n][0] and nxt == first[n][2] and np.array_equal(logits, first[n][1])
        else:
            first[n] = (tok, logits.copy(), nxt)


def test_short_prompt_k_parts_equal_the_unsplit_products(tg, oracle):
    """A 100-token prompt: the down projection (K = 2048) runs in four parts of K over workgroups and the output
    projection (K = 1024) in two, the following norm adds the partial results.  Against the same prefill with the
    products unsplit: same id, logits equal to fp32 rounding of the extra additions, and really a different path.
    The GeLU table has 2^20 entries here: with the 1024-entry step table a rounding difference that moves one
    activation across a bin edge shows as ~2e-4 in the logits, which would say nothing about the split."""
    cfg = tg.named_config("270m", 2)
    model = tg.Transformer(cfg)
    model.read_weights_mem(oracle.generate_weights(gi.oracle_config("270m", 2), 23))
    sess = model.session(gsize=1 << 20)
    prompt = gi.prompt_ids(35, 100)
    out = []
    try:
        for split in (1, 0):
            tg.check(tg.lib().tg_set_gemm_split(split))
            sess.reset()
            out.append(sess.prefill(prompt))
    finally:
        tg.check(tg.lib().tg_set_gemm_split(1))
    (tok_a, lg_a), (tok_b, lg_b) = out
    rel = normrel(lg_a, lg_b)
    print(f"k parts vs unsplit: logits rel {rel:.2e}")
    assert tok_a == tok_b and rel < 2e-5
    assert not np.array_equal(lg_a, lg_b)


@pytest.mark.parametrize("gsize", [1024, 8192])
def test_two_gemm_workgroups_per_unit_change_no_bit_of_a_long_prefill(tg, oracle, gsize):
    """3000 tokens through two layers of the 270m shape with tg_set_gemm_lds(1): the up|gate product (fused
    gelu(gate) * up epilogue, GeLU table staged in the LDS the operand ring has left: 1024 entries; read from global
    memory: 8192 entries) runs two workgroups per compute unit.  Same arithmetic: not a bit of the logits may differ."""
    cfg = tg.named_config("270m", 2)
    model = tg.Transformer(cfg)
    model.read_weights_mem(oracle.generate_weights(gi.oracle_config("270m", 2), 22))
    sess = model.session(gsize=gsize)
    prompt = gi.prompt_ids(34, 3000)
    out, ran = [], []
    try:
        for lds in (1, 0):
            tg.check(tg.lib().tg_set_gemm_lds(lds))
            sess.reset()
            before = tg.gemm_launches()
            out.append(sess.prefill(prompt))
            ran.append(tuple(b - a for a, b in zip(before, tg.gemm_launches())))
    finally:
        tg.check(tg.lib().tg_set_gemm_lds(2))
    # 2 layers x 4 products: Q|K|V (288 tiles) and up|gate (768) on the two-workgroups kernel, the output and down
    # projections (120 tiles, under half a tile per compute unit) on one workgroup per tile either way
    assert ran == [(0, 4, 4), (0, 8, 0)]
    (tok_a, lg_a), (tok_b, lg_b) = out
    assert tok_a == tok_b and np.array_equal(lg_a, lg_b)


def test_half_k_copies_of_the_two_workgroup_kernel_equal_the_unsplit_products(tg, oracle):
    """8000 tokens through two layers of the 270m shape: output and down projection have 63 x 5 = 315 tiles for 512
    workgroup slots and run as two half-K copies of the grid, the following norm adds the two partial results
    (tg_set_gemm_lds(2), the default) - against the same products unsplit (2 + 64): same id, logits equal to fp32
    rounding of one extra addition, and really a different path."""
    cfg = tg.named_config("270m", 2)
    model = tg.Transformer(cfg)
    model.read_weights_mem(oracle.generate_weights(gi.oracle_config("270m", 2), 24))
    sess = model.session(gsize=1 << 20)
    prompt = gi.prompt_ids(36, 8000)
    out = []
    try:
        for knob in (2, 66):
            tg.check(tg.lib().tg_set_gemm_lds(knob))
            sess.reset()
            before = tg.gemm_launches()
            out.append(sess.prefill(prompt))
            assert tuple(b - a for a, b in zip(before, tg.gemm_launches())) == (0, 0, 8)  # all on the two-workgroups kernel
    finally:
        tg.check(tg.lib().tg_set_gemm_lds(2))
    (tok_a, lg_a), (tok_b, lg_b) = out
    rel = normrel(lg_a, lg_b)
    print(f"half-K copies vs unsplit (two workgroups per unit): logits rel {rel:.2e}")
    assert tok_a == tok_b and rel < 2e-5
    assert not np.array_equal(lg_a, lg_b)


def test_half_k_grid_copies_equal_the_plain_grid(tg, oracle, weight_images, tables):
    """Prefill with the output/down projections computed as two half-K copies added by the following norm
    (taken when the plain grid fills its last round badly: here 1000 rows x 5 column tiles) against the
    same prefill with the plain grid: same ids, logits equal to fp32 rounding of one extra addition."""
    cfg = tg.named_config("270m", 2)
    image = oracle.generate_weights(gi.oracle_config("270m", 2), 21)
    model = tg.Transformer(cfg)
    model.read_weights_mem(image)
    sess = model.session(gsize=1 << 20)
    prompt = gi.prompt_ids(33, 1000)
    out = []
    try:
        for split in (1, 0):
            tg.check(tg.lib().tg_set_gemm_split(split))
            sess.reset()
            out.append(sess.prefill(prompt))
    finally:
        tg.check(tg.lib().tg_set_gemm_split(1))
    (tok_a, lg_a), (tok_b, lg_b) = out
    assert tok_a == tok_b and normrel(lg_a, lg_b) < 2e-5
    # the prefill scratch can be dropped; decode goes on without it and the next prefill allocates it again
    sess.release_workspace()
    nxt, _ = sess.decode(tok_b)
    sess.reset()
    assert sess.prefill(prompt)[0] == tok_b and sess.decode(tok_b)[0] == nxt
    assert not np.array_equal(lg_a, lg_b)   # the two paths really differ (the split was taken)
