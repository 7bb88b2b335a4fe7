#!/usr/bin/env python3
"""Writes tests/golden/tokenizer.npz: what the REAL reference tokenizer (sentencepiece::Tokenizer of
csrc/include/tokenizer.hpp, compiled into oracle/_ref/libtg_ref.so by oracle/Makefile) returns on the synthetic
vocabulary and texts of tests/golden_inputs.py.

Run in the build container only (it needs the reference checkout to have built oracle/_ref):

    python tests/golden/make_tokenizer_golden.py

Stored: per text and chat format the ids of encode() and the bytes of decode(ids) (length -2 where the reference
threw std::invalid_argument), and per vocabulary id the length of decode(id, prev) for prev in (1, 5), again -2
for a throw, with a checksum of all pieces.
"""
import hashlib
import os
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import golden_inputs as gi  # noqa: E402
from oracle.oracle import Ref  # noqa: E402


def main():
    assert Ref.available(), "oracle/_ref/libtg_ref.so missing: run `make -C oracle` where /root/reference exists"
    ref = Ref()
    pieces, scores = gi.tokenizer_vocab()
    texts = gi.tokenizer_texts()
    out = {}
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "tok.bin")
        gi.write_tokenizer_file(path, pieces, scores)
        for chat in (0, 1):
            t = ref.tokenizer(path, 2, 1, gi.TOKENIZER_VOCAB, chat)
            ids_all, offs, dec_all, dec_len = [], [0], [], []
            for text in texts:
                ids = t.encode(text)
                ids_all.append(ids)
                offs.append(offs[-1] + ids.size)
                try:
                    dec = t.decode(ids)
                    dec_len.append(len(dec))
                    dec_all.append(np.frombuffer(dec, np.uint8))
                except ValueError:
                    dec_len.append(-2)
            out[f"chat{chat}/ids"] = np.concatenate(ids_all).astype(np.int32)
            out[f"chat{chat}/offsets"] = np.array(offs, np.int64)
            out[f"chat{chat}/decoded_len"] = np.array(dec_len, np.int64)
            out[f"chat{chat}/decoded"] = np.concatenate(dec_all) if dec_all else np.zeros(0, np.uint8)
        t = ref.tokenizer(path, 2, 1, gi.TOKENIZER_VOCAB, 0)
        for prev in (1, 5):
            lens, h = [], hashlib.sha256()
            for tok in range(gi.TOKENIZER_VOCAB):
                try:
                    p = t.decode_piece(tok, prev)
                    lens.append(len(p))
                    h.update(p)
                except ValueError:
                    lens.append(-2)
            out[f"piece_len/prev{prev}"] = np.array(lens, np.int32)
            out[f"piece_sha/prev{prev}"] = np.array(h.hexdigest())
    dst = os.path.join(HERE, "tokenizer.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
