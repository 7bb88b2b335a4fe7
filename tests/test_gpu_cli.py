"""GPU: the command line front end (tiny-gemma_amd/host/gemma, counterpart of the reference's gemma.cpp) end to
end: weight file + tokenizer file + text prompt -> printed text and the closing tok/s line.  The expected text is
built from the same pieces through the Python binding: prompt ids from the tokenizer (whose parity with the
reference's is the subject of tests/test_tokenizer.py), greedy ids from Session.generate."""
import os
import re
import subprocess

import numpy as np
import pytest

import golden_inputs as gi
from test_tokenizer import Tok

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tiny-gemma_amd", "host", "gemma")


@pytest.fixture(scope="module")
def files(tmp_path_factory, weight_images):
    d = tmp_path_factory.mktemp("cli")
    pieces, scores = gi.tokenizer_vocab_full()
    gi.write_tokenizer_file(d / "tok.bin", pieces, scores)
    weight_images("270m", 18, 5).tofile(d / "w.bin")
    return d, pieces


def run_cli(d, *args):
    if not os.path.exists(EXE):
        pytest.fail("tiny-gemma_amd/host/gemma is not built: run __graft_entry__.build()")
    env = dict(os.environ, LD_LIBRARY_PATH=os.path.join(ROOT, "tiny-gemma_amd") + ":" + os.environ.get("LD_LIBRARY_PATH", ""))
    return subprocess.run([EXE, "--weights_path", str(d / "w.bin"), "--model_size", "270m", "--tokenizer_path", str(d / "tok.bin"), *args],
                          capture_output=True, env=env, timeout=300)


def piece_text(t, pieces, tok, prev):
    try:
        return t.decode_piece(tok, prev)
    except ValueError:   # byte token: the front end prints the byte where the reference's tokenizer throws
        return bytes([t.byte_of(tok)])


@pytest.mark.parametrize("chat", [0, 1])
def test_greedy_generation_prints_the_expected_text(tg, weight_images, files, chat):
    d, pieces = files
    prompt = b"hello world " + b" ".join(pieces[600:612]) + " café 日本語".encode()
    n_dec = 40
    r = run_cli(d, "--prompt", prompt.decode(), "--n_dec", str(n_dec), "--chat_format", str(chat))
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    t = Tok(d / "tok.bin", 2, 1, 262144, chat)
    ids = t.encode(prompt)
    assert b"Weights loaded!\n" in r.stdout and b"Prompt length: %d\n" % ids.size in r.stdout
    model = tg.Transformer(tg.named_config("270m"))
    model.read_weights(str(d / "w.bin"))
    out, _, _ = model.session().greedy(ids, n_dec)
    assert len(out) == n_dec + 1
    text, prev = t.decode(ids), int(ids[-1])
    for tok in out:
        text += piece_text(t, pieces, int(tok), prev)
        prev = int(tok)
    assert text in r.stdout
    m = re.search(rb"Generating (\d+) tokens took ([0-9.]+) seconds. Prefill Tok/s: ([0-9.]+)  Decode Tok/s ([0-9.]+) ms/token: ([0-9.]+)", r.stdout)
    assert m and int(m.group(1)) == n_dec and float(m.group(4)) > 100.0


def test_sampling_and_usage_errors(files):
    d, _ = files
    r = run_cli(d, "--prompt", "a b c", "--n_dec", "24", "--minp", "0.05", "--temp", "1.0")
    assert r.returncode == 0 and b"Generating 24 tokens" in r.stdout
    r = run_cli(d, "--prompt", "a", "--bogus", "1")
    assert r.returncode == 1 and b"unknown option: --bogus" in r.stderr
    r = run_cli(d, "--prompt", "a", "--n_dec", "many")
    assert r.returncode == 1 and b"Parse error: expected integer for many" in r.stderr
    r = run_cli(d, "--prompt")
    assert r.returncode == 1 and b"missing value for --prompt" in r.stderr
