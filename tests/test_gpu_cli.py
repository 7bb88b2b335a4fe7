"""GPU: the command line front ends (tiny-gemma_amd/host/gemma and host/passkey, counterparts of the reference's
gemma.cpp and tests/passkey.cpp) end to end: weight file + tokenizer file + text prompt -> printed text and the closing tok/s line.  The expected text is
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
PASSKEY_EXE = os.path.join(ROOT, "tiny-gemma_amd", "host", "passkey")


@pytest.fixture(scope="module")
def files(tmp_path_factory, weight_images):
    d = tmp_path_factory.mktemp("cli")
    pieces, scores = gi.tokenizer_vocab_full()
    gi.write_tokenizer_file(d / "tok.bin", pieces, scores)
    weight_images("270m", 18, 5).tofile(d / "w.bin")
    return d, pieces


def run_cli(d, *args, exe=EXE):
    if not os.path.exists(exe):
        pytest.fail(os.path.relpath(exe, ROOT) + " is not built: run __graft_entry__.build()")
    env = dict(os.environ, LD_LIBRARY_PATH=os.path.join(ROOT, "tiny-gemma_amd") + ":" + os.environ.get("LD_LIBRARY_PATH", ""))
    return subprocess.run([exe, "--weights_path", str(d / "w.bin"), "--model_size", "270m", "--tokenizer_path", str(d / "tok.bin"), *args],
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


@pytest.mark.parametrize("fixed", [False, True])
def test_passkey_run_reports_what_the_generated_text_holds(tg, files, fixed):
    """Random weights retrieve nothing, so the check is the plumbing: the prompt that reaches the model is the pass
    key prompt in chat format, the generation is greedy and stops at <end_of_turn>, and the found / not found line
    says what the generated text holds."""
    import test_passkey as tp
    d, pieces = files
    n_garbage = 1500
    L = tp.shim()
    if fixed:
        prefix, key = 1234, 31337
        r = run_cli(d, "--n_garbage", str(n_garbage), "--n_garbage_prefix", str(prefix), "--passkey", str(key), exe=PASSKEY_EXE)
    else:
        prefix, key = tp.draw(L, 11, n_garbage)
        r = run_cli(d, "--n_garbage", str(n_garbage), "--seed", "11", exe=PASSKEY_EXE)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    prompt = tp.built_prompt(L, n_garbage, prefix, key).encode()
    t = Tok(d / "tok.bin", 2, 1, 262144, 1)
    ids = t.encode(prompt)
    assert b"Prompt length: %d\n" % ids.size in r.stdout
    model = tg.Transformer(tg.named_config("270m"))
    model.read_weights(str(d / "w.bin"))
    out, _, _ = model.session().greedy(ids, 50)
    first, rest = int(out[0]), [int(x) for x in out[1:]]
    if 106 in rest:
        rest = rest[:rest.index(106)]
    text, prev = b"", first
    for tok in rest:
        text += piece_text(t, pieces, tok, prev)
        prev = tok
    shown = t.decode(ids) + piece_text(t, pieces, first, int(ids[-1])) + text
    assert shown in r.stdout
    verdict = b"found!" if str(key).encode() in text else b"not found!"
    assert b"\nPasskey=%d %s\n" % (key, verdict) in r.stdout
    m = re.search(rb"Generating (\d+) tokens took ([0-9.]+) seconds. Tok/s: ([0-9.]+) ms/token: ([0-9.]+)", r.stdout)
    assert m and int(m.group(1)) == len(rest)


def test_passkey_usage_errors(files):
    d, _ = files
    r = run_cli(d, exe=PASSKEY_EXE)
    assert r.returncode == 1 and b"--n_garbage must be at least 1" in r.stderr
    r = run_cli(d, "--n_garbage", "100", "--passkey", "5", exe=PASSKEY_EXE)
    assert r.returncode == 1 and b"go together" in r.stderr
    r = run_cli(d, "--n_garbage", "100", "--n_garbage_prefix", "101", "--passkey", "5", exe=PASSKEY_EXE)
    assert r.returncode == 1 and b"1..n_garbage" in r.stderr
