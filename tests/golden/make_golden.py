#!/usr/bin/env python3
"""Writes tests/golden/golden.npz: outputs of the REAL reference (oracle/_ref/libtg_ref.so, compiled
from the reference's own C++ sources by oracle/Makefile) on seeded inputs.

Run in the build container only (it needs the reference checkout to have built oracle/_ref):

    python tests/golden/make_golden.py [--skip-1b]

Only results go into the fixture (outputs, checksums, token ids); inputs are regenerated from the
seeds by tests/golden_inputs.py, and model weights by the seeded generator in oracle/tg_oracle.c
(their SHA-256 is stored so a test can tell a generator change from a forward-pass change).
"""
import argparse
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--skip-1b", action="store_true")
    args = ap.parse_args()
    assert Ref.available(), "oracle/_ref/libtg_ref.so missing: run `make -C oracle` where /root/reference exists"
    r, o = Ref(), Oracle()
    out = {}

    # ---- kernels ----
    for name, (i, n, logits, seed) in gi.GEMV_CASES.items():
        x, W, s = gi.gemv_inputs(i, n, seed)
        y = r.qgemv(x, W, s, logits)
        out[f"gemv/{name}/sha"] = sha(y)
        out[f"gemv/{name}/head"] = y[:2048].copy()
        out[f"gemv/{name}/sum"] = np.float64(y.astype(np.float64).sum())
        print("gemv", name, sha(y)[:12], flush=True)
    for name, (m, i, n, seed) in gi.GEMM_CASES.items():
        A, W, s = gi.gemm_inputs(m, i, n, seed)
        Cm = r.qgemm(A, W, s)
        out[f"gemm/{name}/sha"] = sha(Cm)
        out[f"gemm/{name}/head"] = Cm.reshape(-1)[:2048].copy()
        print("gemm", name, sha(Cm)[:12], flush=True)

    # ---- ops ----
    for name, (rows, dim, seed) in gi.RMSNORM_CASES.items():
        x, w = gi.rmsnorm_inputs(rows, dim, seed)
        out[f"rmsnorm/{name}"] = r.rmsnorm(x, w)
    for theta in (1000000.0, 10000.0):
        c, s = r.rope_tables(theta, 32768)
        out[f"rope/{int(theta)}/cos_rows"] = c[gi.ROPE_ROWS].copy()
        out[f"rope/{int(theta)}/sin_rows"] = s[gi.ROPE_ROWS].copy()
        x = gi.rope_apply_input(7)
        out[f"rope/{int(theta)}/apply"] = r.rope_apply(x, theta, 2048, 1000)
    for size in (1024, 8192):
        out[f"gelu/table{size}"] = r.gelu_table(-4.0, 4.0, size)
        out[f"gelu/apply{size}"] = r.gelu(gi.gelu_input(3), -4.0, 4.0, size)
    ids, wte, sc = gi.embedding_inputs(5)
    out["embedding"] = r.embedding(ids, wte, sc)
    for name, (S, sw, ctx, seed) in gi.ATTN_PREFILL_CASES.items():
        q, k, v = gi.attn_prefill_inputs(S, seed)
        out[f"attn_prefill/{name}"] = r.attention_prefill(q, k, v, sw, ctx)[:, gi.attn_rows(S), :]
    for name, (max_pos, valid, seed) in gi.ATTN_DECODE_CASES.items():
        q, kc, vc = gi.attn_decode_inputs(max_pos, seed)
        out[f"attn_decode/{name}"] = r.attention_decode(q, kc, vc, valid)
    lg = gi.argmax_input(9)
    out["argmax"] = np.int32(r.argmax(lg))
    lg[1000] = lg[200000] = lg.max() + 1.0  # tie: the lowest index wins
    out["argmax_tie"] = np.int32(r.argmax(lg))
    for name, (seed, scale, peaked, minp, temp, randf) in gi.MINP_CASES.items():
        idx, probs = r.minp_logits(gi.minp_input(seed, scale, peaked), minp, temp, randf)
        out[f"minp/{name}/index"] = np.int32(idx)
        out[f"minp/{name}/prob_sum"] = np.float64(probs.astype(np.float64).sum())
        out[f"minp/{name}/prob_head"] = probs[:256].copy()

    # ---- models ----
    for name, (shape, n_layers, seed, n_prompt, n_decode, n_tap_steps, gsize) in gi.MODEL_CASES.items():
        if args.skip_1b and shape == "1B":
            continue
        t0 = time.time()
        cfg = gi.oracle_config(shape, n_layers)
        path = f"/tmp/tg_golden_{name}.bin"
        image = o.generate_weights(cfg, seed)
        image.tofile(path)
        out[f"model/{name}/weights_sha"] = hashlib.sha256(image.tobytes()).hexdigest()
        del image
        sess = r.model(cfg, path).session(-4.0, 4.0, gsize)
        os.remove(path)
        prompt = gi.prompt_ids(seed, n_prompt)
        tok, logits, taps = sess.prefill(prompt, taps=True)
        toks = [tok]

        def top2(lg):
            i = np.argpartition(lg, -2)[-2:]
            i = i[np.argsort(lg[i])][::-1]
            return float(lg[i[0]] - lg[i[1]]), (int(i[0]), int(i[1]))

        gap, pair = top2(logits)
        gaps, pairs = [gap], [pair]
        out[f"model/{name}/prefill_logits_head"] = logits[:4096].copy()
        out[f"model/{name}/prefill_logits_sha"] = sha(logits)
        out[f"model/{name}/prefill_logits_norm"] = np.float64(np.linalg.norm(logits.astype(np.float64)))
        out[f"model/{name}/prefill_taps_last"] = taps[:, -1, :].copy()       # residual of the last position after each block
        out[f"model/{name}/prefill_taps_norm"] = np.linalg.norm(taps.astype(np.float64), axis=(1, 2))
        if n_prompt <= 128:
            out[f"model/{name}/prefill_taps"] = taps[:, gi.tap_rows(n_prompt), :].copy()
        for l in sorted({0, min(5, n_layers - 1)}):
            k, v, pp, bp = sess.kv(l)
            nrows = min(k.shape[0], max(n_prompt, 1))
            out[f"model/{name}/kv{l}_k_norm"] = np.float64(np.linalg.norm(k[:nrows].astype(np.float64)))
            out[f"model/{name}/kv{l}_k_first"] = k[0].copy()
            out[f"model/{name}/kv{l}_k_last"] = k[min(nrows, k.shape[0]) - 1].copy()
            out[f"model/{name}/kv{l}_v_last"] = v[min(nrows, v.shape[0]) - 1].copy()
            out[f"model/{name}/kv{l}_ptrs"] = np.array([pp, bp], np.int32)
        dec_taps, dec_logits_head = [], []
        for step in range(n_decode):
            want = step < n_tap_steps
            tok, logits, tp = sess.decode(toks[-1], want_logits=True, taps=want)
            toks.append(tok)
            gap, pair = top2(logits)
            gaps.append(gap)
            pairs.append(pair)
            if want:
                dec_taps.append(tp)
                dec_logits_head.append(logits[:4096].copy())
        out[f"model/{name}/tokens"] = np.array(toks, np.int32)
        out[f"model/{name}/top2_gaps"] = np.array(gaps, np.float32)
        out[f"model/{name}/top2_ids"] = np.array(pairs, np.int32)
        if dec_taps:
            out[f"model/{name}/decode_taps"] = np.stack(dec_taps)
            out[f"model/{name}/decode_logits_head"] = np.stack(dec_logits_head)
        out[f"model/{name}/final_logits_head"] = logits[:4096].copy()
        out[f"model/{name}/final_logits_norm"] = np.float64(np.linalg.norm(logits.astype(np.float64)))
        print(f"model {name}: {time.time() - t0:.1f}s distinct tokens {len(set(toks))} min top-2 gap {min(gaps):.4g}", flush=True)

    dst = os.path.join(HERE, "golden.npz")
    if args.skip_1b and os.path.exists(dst):
        old = dict(np.load(dst))
        for k, v in old.items():
            if k.startswith("model/full1B/"):
                out.setdefault(k, v)
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
