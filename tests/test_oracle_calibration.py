"""CPU: how far can an implementation that is correct but not bit-identical to the reference binary be from it?

The acceptance rule of the GPU model tests (conftest.check_picks: a differing greedy pick is accepted only at a
near-tie of the reference and only if it is the reference's runner-up; at most CHECKER_STREAM_MISMATCHES x 2 of them)
rests on one claim: with the command line's 1024-entry step-function GeLU table (csrc/include/ops.hpp:22-52) ANY
implementation that differs from the reference binary in the last bit of some operation ends up ~4e-3 away from it
in the logits and takes its runner-up at some near-ties.  This test measures that on the CPU with the one such
implementation at hand that is independent of the GPU code: the strict-IEEE scalar restatement (oracle/tg_oracle.c,
whose GEMV/GEMM are bit-exact against the compiled reference) against the recordings of the compiled reference
(built with -ffast-math: rsqrt/rcp estimates, vectorised expf/powf), teacher-forced over the random-token streams the
GPU tests use (the reference's own end-to-end criterion is tests/csrc/test_generation.cpp:100-127).

Measured here (x86-64, gcc 11.4): stream270m 4 of 321 picks differ (steps 47, 238, 253, 317 at reference top-2 gaps
6.3e-3, 9.8e-4, 1.2e-3, 6.2e-4), logits 3.3e-3 .. 4.0e-3; stream1B, first 129 picks: 5 differ (steps 16, 23, 57, 91, 113
at 5.2e-3, 6.4e-3, 2.9e-3, 6.2e-4, 2.3e-4; all 321: 7), logits 4.2e-3 at step 0.  Every differing pick is the
reference's runner-up.  The MI355X run differs on 6 + 6 picks of the same streams, at gaps up to 8.0e-3."""
import hashlib

import numpy as np
import pytest

import golden_inputs as gi
from conftest import CHECKER_STREAM_MISMATCHES, NEAR_TIE, check_picks, normrel


@pytest.fixture(scope="module")
def blocks(golden_file):
    return golden_file("golden_blocks.npz")


# name: (steps run here, picks of the checker that differ from the reference's over those steps, as measured)
CASES = {"stream270m": (320, 4), "stream1B": (128, 5)}


@pytest.mark.parametrize("name", list(CASES))
def test_strict_ieee_checker_against_the_reference_binary(oracle, blocks, weight_images, name):
    steps, measured = CASES[name]
    shape, n_layers, seed, n_prompt, all_steps, gsize = gi.STREAM_CASES[name]
    assert gsize == 1024
    image = weight_images(shape, n_layers, seed)
    assert hashlib.sha256(image.tobytes()).hexdigest() == str(blocks[f"stream/{name}/weights_sha"])
    sess = oracle.model(gi.oracle_config(shape, n_layers), image=image).session(-4.0, 4.0, gsize)
    prompt, feed = gi.stream_ids(name)
    ref = blocks[f"stream/{name}/picks"][:steps + 1]
    gaps = blocks[f"stream/{name}/top2_gaps"][:steps + 1]
    pairs = blocks[f"stream/{name}/top2_ids"][:steps + 1]
    heads = blocks[f"stream/{name}/logits_head"]
    tok, _, _ = sess.prefill(prompt, want_logits=False)
    picks, rels = [tok], []
    for i in range(steps):
        want = i in gi.STREAM_LOGIT_STEPS
        tok, lg, _ = sess.decode(int(feed[i]), want_logits=want)
        picks.append(tok)
        if want:
            rels.append(normrel(lg[:4096], heads[gi.STREAM_LOGIT_STEPS.index(i)]))
    print(f"{name}: checker logits head against the reference binary: " + ", ".join(f"{r:.2e}" for r in rels), flush=True)
    # (i) the picks: only the reference's runner-up at a near-tie, and as many as measured, give or take
    mism = check_picks(picks, ref, gaps, pairs, f"{name} (strict-IEEE checker)", near_tie=NEAR_TIE, max_mismatches=2 * measured)
    assert mism.size >= 1, "the checker now agrees with the reference on every pick: the acceptance rule of the GPU tests can be tightened"
    if steps == all_steps:
        assert mism.size == CHECKER_STREAM_MISMATCHES[name]
    # the largest gap at which a correct implementation flips must leave NEAR_TIE a factor of two
    assert float(np.max(gaps[mism])) < NEAR_TIE / 2
    # (ii) the logits: about 4e-3 away, i.e. not within 1e-3 and not beyond twice the measured 4.3e-3
    assert 1e-3 < min(rels) and max(rels) < 8.6e-3, rels
