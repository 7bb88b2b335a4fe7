#!/usr/bin/env python3
"""Writes tests/golden/golden_blocks.npz: outputs of the REAL reference (oracle/_ref/libtg_ref.so) for

  * one modules::attention / modules::mlp / modules::lm_head call at a time on a caller-supplied residual stream,
    on the shape lists of the reference's own unit tests and on cases they never run (local layers, the 1B shape);
  * teacher-forced random-token streams through the full 270m- and 1B-shaped models (per-step argmax, top-2 ids and
    gap, a few logit heads).

Run in the build container only (needs oracle/_ref):   python tests/golden/make_golden_blocks.py [blocks] [streams]
(one group named: the other group's entries are kept as they are)

Only results are stored; inputs and weights are regenerated from seeds (tests/golden_inputs.py, oracle/tg_oracle.c).
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


def top2(lg):
    i = np.argpartition(lg, -2)[-2:]
    i = i[np.argsort(lg[i])][::-1]
    return float(lg[i[0]] - lg[i[1]]), (int(i[0]), int(i[1]))


def main():
    assert Ref.available(), "oracle/_ref/libtg_ref.so missing: run `make -C oracle` where /root/reference exists"
    r, o = Ref(), Oracle()
    groups = sys.argv[1:] or ["blocks", "streams"]
    dst = os.path.join(HERE, "golden_blocks.npz")
    out = {}
    if os.path.exists(dst) and len(groups) < 2:
        keep = "stream/" if "blocks" in groups else "block"
        out = {k: v for k, v in np.load(dst).items() if k.startswith(keep)}
    models = {}

    def model_of(name):
        if name not in models:
            cfg, seed = gi.block_config(name)
            path = f"/tmp/tg_golden_block_{name}.bin"
            image = o.generate_weights(cfg, seed)
            image.tofile(path)
            out[f"block_model/{name}/weights_sha"] = hashlib.sha256(image.tobytes()).hexdigest()
            del image
            models[name] = r.model(cfg, path)
            os.remove(path)
        return models[name]

    for name, (model, kind, rows, cached, gsize, seed) in (gi.BLOCK_CASES.items() if "blocks" in groups else ()):
        t0 = time.time()
        sess = model_of(model).session(-4.0, 4.0, gsize)
        x, k, v = gi.block_inputs(name)
        if cached:
            sess.kv_prefill(0, k, v)
        if kind == "attn":
            y = sess.block_attention(0, x)
        elif kind == "mlp":
            y = sess.block_mlp(0, x)
        else:
            y = sess.block_lm_head(x)
            out[f"block/{name}/norm"] = np.float64(np.linalg.norm(y.astype(np.float64)))
            out[f"block/{name}/argmax"] = np.int32(np.argmax(y))
            out[f"block/{name}/head"] = y[:4096].copy()
            out[f"block/{name}/sample"] = y[gi.LOGIT_SAMPLE].copy()
            print(f"{name}: {time.time() - t0:.1f}s", flush=True)
            continue
        out[f"block/{name}/norm"] = np.float64(np.linalg.norm(y.astype(np.float64)))
        out[f"block/{name}/rows"] = y[gi.block_rows(rows)].copy()
        if kind == "attn":   # the cache the block leaves behind: counters and the row it wrote last
            kk, vv, pp, bp = sess.kv(0)
            out[f"block/{name}/kv_ptrs"] = np.array([pp, bp], np.int32)
            slot = (bp - 1) % kk.shape[0]
            out[f"block/{name}/k_last"] = kk[slot].copy()
            out[f"block/{name}/v_last"] = vv[slot].copy()
        print(f"{name}: {time.time() - t0:.1f}s", flush=True)
    models.clear()

    for name, (shape, n_layers, seed, n_prompt, steps, gsize) in (gi.STREAM_CASES.items() if "streams" in groups else ()):
        t0 = time.time()
        cfg = gi.oracle_config(shape, n_layers)
        path = f"/tmp/tg_golden_{name}.bin"
        image = o.generate_weights(cfg, seed)
        image.tofile(path)
        out[f"stream/{name}/weights_sha"] = hashlib.sha256(image.tobytes()).hexdigest()
        del image
        sess = r.model(cfg, path).session(-4.0, 4.0, gsize)
        os.remove(path)
        prompt, feed = gi.stream_ids(name)
        tok, logits, _ = sess.prefill(prompt)
        picks, gaps, pairs, heads = [tok], [], [], []
        gap, pair = top2(logits)
        gaps.append(gap)
        pairs.append(pair)
        for i in range(steps):
            tok, logits, _ = sess.decode(int(feed[i]), want_logits=True)
            picks.append(tok)
            gap, pair = top2(logits)
            gaps.append(gap)
            pairs.append(pair)
            if i in gi.STREAM_LOGIT_STEPS:
                heads.append(logits[:4096].copy())
        out[f"stream/{name}/picks"] = np.array(picks, np.int32)       # [0]: after the prompt; [i + 1]: after feed[i]
        out[f"stream/{name}/top2_gaps"] = np.array(gaps, np.float32)
        out[f"stream/{name}/top2_ids"] = np.array(pairs, np.int32)
        out[f"stream/{name}/logits_head"] = np.stack(heads)
        print(f"{name}: {time.time() - t0:.1f}s, distinct picks {len(set(picks))}, min top-2 gap {min(gaps):.4g}", flush=True)

    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
