"""GPU: a converted checkpoint runs.  A synthetic Hugging Face-named checkpoint of the 270m shape (2 layers)
is converted (tiny-gemma_amd/convert.py), read from its path by the library (pinned staging + on-device
re-tiling) and by the CPU oracle, and the two forwards are compared like the other small-model cases."""
import os
from types import SimpleNamespace

import numpy as np
import pytest

import __graft_entry__ as ge
import golden_inputs as gi
from conftest import normrel

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
st = pytest.importorskip("safetensors.torch")


def test_converted_checkpoint_runs(tg, oracle, tmp_path):
    from test_convert import make_checkpoint
    from tiny_gemma_amd import convert
    n_layers = 2
    cfg = convert.named_dims("270m")
    cfg.n_layers = n_layers
    sd = make_checkpoint(cfg, 9, torch.bfloat16)
    src, dst = str(tmp_path / "model.safetensors"), str(tmp_path / "w.bin")
    st.save_file(sd, src)
    del sd
    n = convert.convert_weights(src, dst, cfg)
    os.remove(src)
    model = tg.Transformer(tg.named_config("270m", n_layers))
    assert n == model.weight_file_bytes()
    model.read_weights(dst)
    gsize = 1 << 20  # near-continuous GeLU table: tight end-to-end comparison
    sess = model.session(gsize=gsize)
    osess = oracle.model(gi.oracle_config("270m", n_layers), path=dst).session(-4.0, 4.0, gsize)
    prompt = gi.prompt_ids(9, 24)
    tok, logits = sess.prefill(prompt)
    otok, ologits, _ = osess.prefill(prompt)
    assert normrel(logits, ologits) < 5e-5 and tok == otok
    for _ in range(3):
        nxt, logits = sess.decode(tok)
        onxt, ologits, _ = osess.decode(tok)
        assert normrel(logits, ologits) < 5e-5 and nxt == onxt
        tok = nxt
