#!/usr/bin/env python3
"""Writes tests/golden/golden_long.npz: outputs of the REAL reference (oracle/_ref/libtg_ref.so) on the two
long benchmark configurations at their full size.

    prefill4096_1B   1B shape (26 layers), 4096 random prompt tokens, one forward_prefill
    long16k_270m     270m shape (18 layers), 16384 random prompt tokens, then 256 greedy decode steps

Run in the build container only (needs oracle/_ref; minutes of CPU per case):

    python tests/golden/make_golden_long.py [case ...]

Only results are stored (logit heads, checksums, last-row residuals, a few cache rows, token ids with their
top-2 gaps); prompts and weights are regenerated from seeds by tests/golden_inputs.py and the seeded
generator of oracle/tg_oracle.c.  Cases not named on the command line keep their old entries.
"""
import hashlib
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import golden_inputs as gi  # noqa: E402
from oracle.oracle import Oracle, Ref  # noqa: E402


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def top2(lg):
    i = np.argpartition(lg, -2)[-2:]
    i = i[np.argsort(lg[i])][::-1]
    return float(lg[i[0]] - lg[i[1]]), (int(i[0]), int(i[1]))


def record(name, r, o, out):
    shape, n_layers, seed, n_prompt, n_decode, gsize = gi.LONG_CASES[name]
    t0 = time.time()
    cfg = gi.oracle_config(shape, n_layers)
    path = f"/tmp/tg_golden_{name}.bin"
    image = o.generate_weights(cfg, seed)
    image.tofile(path)
    out[f"{name}/weights_sha"] = hashlib.sha256(image.tobytes()).hexdigest()
    del image
    sess = r.model(cfg, path).session(-4.0, 4.0, gsize)
    os.remove(path)
    prompt = gi.prompt_ids(seed, n_prompt)
    tok, logits, taps = sess.prefill(prompt, taps=True)
    print(f"{name}: prefill done after {time.time() - t0:.0f}s", flush=True)
    gap, pair = top2(logits)
    out[f"{name}/prefill_argmax"] = np.int32(tok)
    out[f"{name}/prefill_logits_head"] = logits[:4096].copy()
    out[f"{name}/prefill_logits_sha"] = sha(logits)
    out[f"{name}/prefill_logits_norm"] = np.float64(np.linalg.norm(logits.astype(np.float64)))
    out[f"{name}/prefill_taps_last"] = taps[:, -1, :].copy()
    out[f"{name}/prefill_taps_norm"] = np.linalg.norm(taps.astype(np.float64), axis=(1, 2))
    del taps
    rows = gi.long_kv_rows(n_prompt)
    for l in (0, 5):   # a local (ring of 512) and a global layer
        k, v, pp, bp = sess.kv(l)
        valid = min(k.shape[0], n_prompt)
        out[f"{name}/kv{l}_ptrs"] = np.array([pp, bp], np.int32)
        out[f"{name}/kv{l}_k_norm"] = np.float64(np.linalg.norm(k[:valid].astype(np.float64)))
        out[f"{name}/kv{l}_v_norm"] = np.float64(np.linalg.norm(v[:valid].astype(np.float64)))
        sel = rows[rows < valid]
        out[f"{name}/kv{l}_k_rows"] = k[sel].copy()
        out[f"{name}/kv{l}_v_rows"] = v[sel].copy()
    toks, gaps, pairs, heads = [tok], [gap], [pair], []
    for step in range(n_decode):
        tok, logits, _ = sess.decode(toks[-1], want_logits=True)
        toks.append(tok)
        gap, pair = top2(logits)
        gaps.append(gap)
        pairs.append(pair)
        if step in gi.LONG_DECODE_LOGIT_STEPS:
            heads.append(logits[:4096].copy())
    if n_decode:
        out[f"{name}/tokens"] = np.array(toks, np.int32)
        out[f"{name}/top2_gaps"] = np.array(gaps, np.float32)
        out[f"{name}/top2_ids"] = np.array(pairs, np.int32)
        out[f"{name}/decode_logits_head"] = np.stack(heads)
        k, v, pp, bp = sess.kv(5)
        out[f"{name}/kv5_final_ptrs"] = np.array([pp, bp], np.int32)
        out[f"{name}/kv5_k_decoded_rows"] = k[n_prompt:n_prompt + n_decode:64].copy()
    print(f"{name}: {time.time() - t0:.0f}s, distinct tokens {len(set(toks))}, min top-2 gap {min(gaps):.4g}", flush=True)


def main():
    assert Ref.available(), "oracle/_ref/libtg_ref.so missing: run `make -C oracle` where /root/reference exists"
    names = sys.argv[1:] or list(gi.LONG_CASES)
    r, o = Ref(), Oracle()
    dst = os.path.join(HERE, "golden_long.npz")
    out = dict(np.load(dst)) if os.path.exists(dst) else {}
    for name in names:
        for k in [k for k in out if k.startswith(name + "/")]:
            del out[k]
        record(name, r, o, out)
        np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
