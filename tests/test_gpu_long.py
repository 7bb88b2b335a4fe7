"""GPU: the two long benchmark configurations at their full size against the compiled reference's recordings
(tests/golden/golden_long.npz, written by tests/golden/make_golden_long.py):

  prefill4096_1B   1B shape, 26 layers, one forward over 4096 random tokens (int8 matrix GEMM at 4096 rows, causal
                   attention with split key ranges on 4 global layers, 513-key windows on 22 local ones)
  long16k_270m     270m shape, 18 layers, 16384-token prefill, then 256 decode steps fed the reference's ids
                   (decode attention over 16384..16640 keys on the global layers: 512+ workgroups and the merge launch)

Bounds.  The models use the command line's 1024-entry step-function GeLU table, through 26 / 18 layers: a strict-IEEE
CPU restatement of the reference already sits 4e-3 from the reference binary (built with -ffast-math) on the 18-layer
logits, for the reason given in tests/conftest.py (check_picks).  Each bound below is about twice what the MI355X run
measured (printed by the test): prefill logits 4.3e-3 (4096 tokens, 1B shape) and 4.5e-3 (16384 tokens, 270m shape)
from the reference's, the last row's residual after every block within the same, first block 1.2e-6; layer 0 cache
rows 5e-7 .. 7e-7, global layer 5 cache rows 1.0e-3 .. 1.3e-3; decode logits at 16384+ keys 3.3e-3 .. 5.4e-3.  Picks:
the reference's, or its runner-up at a near-tie (the 16384-token prompt ends on one: top-2 gap 5.7e-3, and the
library picks the runner-up there; the other 256 picks are identical).
"""
import hashlib

import numpy as np
import pytest

import golden_inputs as gi
from conftest import check_picks, normrel

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def long_golden(golden_file):
    return golden_file("golden_long.npz")


def _build(tg, oracle, weight_images, ref_tables, long_golden, name):
    shape, n_layers, seed, n_prompt, n_decode, gsize = gi.LONG_CASES[name]
    image = weight_images(shape, n_layers, seed)
    assert hashlib.sha256(image.tobytes()).hexdigest() == str(long_golden[f"{name}/weights_sha"])
    model = tg.Transformer(tg.named_config(shape, n_layers))
    model.read_weights_mem(image)
    sess = model.session(rope=ref_tables[0], rope_sw=ref_tables[1], gelu_table=oracle.gelu_table(-4.0, 4.0, gsize))
    return model, sess, gi.prompt_ids(seed, n_prompt)


def _check_prefill(sess, g, name, prompt, tok, logits, tol_logits, tol_taps, tol_kv):
    n = prompt.size
    rel_logits = normrel(logits[:4096], g[f"{name}/prefill_logits_head"])
    norm_ratio = float(np.linalg.norm(logits.astype(np.float64)) / float(g[f"{name}/prefill_logits_norm"]))
    last = sess.taps(rows=1)[1:, 0, :]                       # a long prompt keeps the last row of every block
    want = g[f"{name}/prefill_taps_last"]
    per_block = [normrel(last[b], want[b]) for b in range(want.shape[0])]
    print(f"{name}: prefill logits head norm-relative {rel_logits:.3e} (bound {tol_logits:.0e}), ||logits|| ratio {norm_ratio:.6f}, "
          f"last-row residuals: first block {per_block[0]:.2e}, worst {max(per_block):.2e} at block {int(np.argmax(per_block))} "
          f"(bound {tol_taps:.0e})", flush=True)
    if f"{name}/top2_gaps" in g:   # the token after the prompt: the reference's, or its runner-up at a near-tie
        check_picks([tok], g[f"{name}/tokens"][:1], g[f"{name}/top2_gaps"][:1], g[f"{name}/top2_ids"][:1], name + " prefill pick")
    else:
        assert tok == int(g[f"{name}/prefill_argmax"])
    assert rel_logits < tol_logits and abs(norm_ratio - 1.0) < tol_logits
    assert per_block[0] < 2.5e-6                             # attention block of layer 0: no table lookup upstream
    assert max(per_block) < tol_taps
    rows = gi.long_kv_rows(n)
    for layer in (0, 5):
        k, v, pp, bp = sess.kv(layer)
        assert (pp, bp) == tuple(int(t) for t in g[f"{name}/kv{layer}_ptrs"])
        valid = min(k.shape[0], n)
        sel = rows[rows < valid]
        rk, rv = normrel(k[sel], g[f"{name}/kv{layer}_k_rows"]), normrel(v[sel], g[f"{name}/kv{layer}_v_rows"])
        nk = float(np.linalg.norm(k[:valid].astype(np.float64)) / float(g[f"{name}/kv{layer}_k_norm"]))
        nv = float(np.linalg.norm(v[:valid].astype(np.float64)) / float(g[f"{name}/kv{layer}_v_norm"]))
        print(f"{name}: layer {layer} cache rows: k {rk:.2e}, v {rv:.2e}; norm ratios {nk:.6f}, {nv:.6f}", flush=True)
        bound = 1.5e-6 if layer == 0 else tol_kv               # layer 0's k/v see only the embedding, a norm and a product
        assert rk < bound and rv < bound and abs(nk - 1) < max(bound, 1e-5) and abs(nv - 1) < max(bound, 1e-5)


def test_prefill_4096_tokens_1b_shape(tg, oracle, weight_images, ref_tables, long_golden):
    if not ref_tables[2]:
        pytest.skip("needs the compiled reference's RoPE tables (oracle/_ref): positions up to 4096 differ by 2e-4 with libm's")
    name = "prefill4096_1B"
    print(f"long case {name}", flush=True)
    model, sess, prompt = _build(tg, oracle, weight_images, ref_tables, long_golden, name)
    tok, logits = sess.prefill(prompt)
    _check_prefill(sess, long_golden, name, prompt, tok, logits, tol_logits=9e-3, tol_taps=9e-3, tol_kv=3e-3)
    sess.free()
    model.free()


def test_16k_prefill_then_256_steps_270m_shape(tg, oracle, weight_images, ref_tables, long_golden):
    if not ref_tables[2]:
        pytest.skip("needs the compiled reference's RoPE tables (oracle/_ref): positions up to 16640 differ by 2e-3 with libm's")
    name = "long16k_270m"
    print(f"long case {name}", flush=True)
    g = long_golden
    model, sess, prompt = _build(tg, oracle, weight_images, ref_tables, g, name)
    n_decode = gi.LONG_CASES[name][4]
    tok, logits = sess.prefill(prompt)
    _check_prefill(sess, g, name, prompt, tok, logits, tol_logits=9e-3, tol_taps=9e-3, tol_kv=3e-3)
    ref, gaps, pairs = g[f"{name}/tokens"], g[f"{name}/top2_gaps"], g[f"{name}/top2_ids"]
    heads = g[f"{name}/decode_logits_head"]
    picks, rels = [tok], []
    for i in range(n_decode):
        want = i in gi.LONG_DECODE_LOGIT_STEPS
        tok, lg = sess.decode(int(ref[i]), want_logits=want)       # teacher-forced with the reference's ids
        picks.append(tok)
        if want:
            rels.append(normrel(lg[:4096], heads[gi.LONG_DECODE_LOGIT_STEPS.index(i)]))
    print(f"{name}: decode logits head norm-relative at steps {gi.LONG_DECODE_LOGIT_STEPS}: " + ", ".join(f"{r:.2e}" for r in rels), flush=True)
    # the reference's smallest top-2 gap over the 256 steps is 0.03: no near-tie after the first pick
    mism = check_picks(picks, ref, gaps, pairs, name + " teacher-forced")
    assert set(mism.tolist()) <= {0}
    assert max(rels) < 1e-2
    k, v, pp, bp = sess.kv(5)
    assert (pp, bp) == tuple(int(t) for t in g[f"{name}/kv5_final_ptrs"]) == (prompt.size + n_decode, prompt.size + n_decode)
    rk = normrel(k[prompt.size:prompt.size + n_decode:64], g[f"{name}/kv5_k_decoded_rows"])
    print(f"{name}: keys written by decode steps (global layer 5): {rk:.2e}", flush=True)
    assert rk < 3e-3
    # the free-running loop on the device from the same state gives the same ids as the stepwise calls
    sess.reset()
    ids, _, _ = sess.greedy(prompt, 32)
    first = int(picks[0])   # the run goes on from the library's own first pick
    if first == int(ref[0]):
        assert np.array_equal(ids, ref[:33])
    else:
        assert ids[0] == first and ids.min() >= 0
    sess.free()
    model.free()
