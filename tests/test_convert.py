"""CPU: the safetensors -> weight-file converter (tiny-gemma_amd/convert.py).

The reference's converter (py/convert.py:66-80, py/gemma.py:367-472) cannot run here (no checkpoint, and its
Python is read, not imported).  What a converted file must satisfy is fixed by the two formats it connects:
a torch Linear computes y = x @ W.T with W stored [out][in]; the C++ reader (transformer.hpp:122-160) takes
[in][out] int8 matrices with a scale per output column and computes y = (x @ q) * s.  So for every matrix
the dequantized file content must reproduce the torch Linear within the quantization bound, every norm
vector must land in the slot the reader assigns to it, and the LM head must be the embedding transposed.
The checkpoint is synthetic (random tensors under the Hugging Face names) with small, all-distinct
dimensions, so that a missing transpose or two swapped tensors cannot pass.
"""
import os
from types import SimpleNamespace

import numpy as np
import pytest

import __graft_entry__ as ge

torch = pytest.importorskip("torch")
st = pytest.importorskip("safetensors.torch")

CFG = SimpleNamespace(hidden_size=48, intermediate_size=80, n_layers=3, n_vocab=96, head_dim=16, n_head=4, n_kv=1,
                      n_pos=64, n_pos_local=16, window_pattern=2)


@pytest.fixture(scope="module")
def conv():
    ge.load_package()
    from tiny_gemma_amd import convert
    return convert


def make_checkpoint(cfg, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    h, f, V, hd = cfg.hidden_size, cfg.intermediate_size, cfg.n_vocab, cfg.head_dim
    qo, kv = cfg.n_head * hd, cfg.n_kv * hd

    def rnd(*shape):
        return (torch.randn(*shape, generator=g) * 0.05).to(dtype)

    sd = {"model.embed_tokens.weight": rnd(V, h), "model.norm.weight": rnd(h)}
    for l in range(cfg.n_layers):
        p = f"model.layers.{l}."
        sd[p + "self_attn.q_proj.weight"] = rnd(qo, h)
        sd[p + "self_attn.k_proj.weight"] = rnd(kv, h)
        sd[p + "self_attn.v_proj.weight"] = rnd(kv, h)
        sd[p + "self_attn.o_proj.weight"] = rnd(h, qo)
        sd[p + "self_attn.q_norm.weight"] = rnd(hd)
        sd[p + "self_attn.k_norm.weight"] = rnd(hd)
        sd[p + "input_layernorm.weight"] = rnd(h)
        sd[p + "post_attention_layernorm.weight"] = rnd(h)
        sd[p + "mlp.up_proj.weight"] = rnd(f, h)
        sd[p + "mlp.gate_proj.weight"] = rnd(f, h)
        sd[p + "mlp.down_proj.weight"] = rnd(h, f)
        sd[p + "pre_feedforward_layernorm.weight"] = rnd(h)
        sd[p + "post_feedforward_layernorm.weight"] = rnd(h)
    return sd


class FileWalker:
    """Reads the flat file the way gemma::read_weights does (transformer.hpp:122-160): sizes come from the
    configuration only, in file order."""

    def __init__(self, path):
        self.b = np.fromfile(path, np.uint8)
        self.off = 0

    def matrix(self, n_in, n_out):
        q = self.b[self.off:self.off + n_in * n_out].view(np.int8).reshape(n_in, n_out)
        self.off += n_in * n_out
        return q, self.vector(n_out)

    def vector(self, n):
        v = self.b[self.off:self.off + 4 * n].view(np.float32)
        self.off += 4 * n
        return v


def check_linear(q, s, w_torch, rng):
    """(x @ q) * s against the torch Linear x @ W.T, W [out][in]."""
    w = w_torch.float().numpy()
    n_out, n_in = w.shape
    assert q.shape == (n_in, n_out) and s.shape == (n_out,)
    x = rng.standard_normal((5, n_in)).astype(np.float32)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    got = (x.astype(np.float64) @ q.astype(np.float64)) * s.astype(np.float64)
    bound = np.abs(x).sum(axis=1, keepdims=True).astype(np.float64) * (s.astype(np.float64) * 0.5001)[None, :]
    assert np.all(np.abs(got - want) <= bound + 1e-12)
    assert np.array_equal(np.abs(q.astype(np.int32)).max(axis=0), np.full(n_out, 127))
    assert np.array_equal(s, (np.abs(w).max(axis=1) / np.float32(127.0)).astype(np.float32))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_converted_file_reproduces_the_checkpoint(conv, tmp_path, dtype):
    cfg = CFG
    sd = make_checkpoint(cfg, 3, dtype)
    src, dst = str(tmp_path / "model.safetensors"), str(tmp_path / "w.bin")
    st.save_file(sd, src)
    n = conv.convert_weights(src, dst, cfg)
    assert n == os.path.getsize(dst)
    h, f, V, hd = cfg.hidden_size, cfg.intermediate_size, cfg.n_vocab, cfg.head_dim
    qo, kv = cfg.n_head * hd, cfg.n_kv * hd
    rng = np.random.default_rng(0)
    fw = FileWalker(dst)

    def same(name, n_el):
        assert np.array_equal(fw.vector(n_el), sd[name].float().numpy()), name

    # embedding: rows are gathered, x[d] = s[d] * q[tok][d] (ops.hpp:537-568): [vocab][hidden], scale per hidden channel
    q, s = fw.matrix(V, h)
    emb = sd["model.embed_tokens.weight"].float().numpy()
    assert np.all(np.abs(q.astype(np.float64) * s[None, :].astype(np.float64) - emb) <= s[None, :] * 0.5001)
    same("model.norm.weight", h)
    for l in range(cfg.n_layers):
        p = f"model.layers.{l}."
        check_linear(*fw.matrix(h, qo), sd[p + "self_attn.q_proj.weight"], rng)
        check_linear(*fw.matrix(h, kv), sd[p + "self_attn.k_proj.weight"], rng)
        check_linear(*fw.matrix(h, kv), sd[p + "self_attn.v_proj.weight"], rng)
        check_linear(*fw.matrix(qo, h), sd[p + "self_attn.o_proj.weight"], rng)
        same(p + "self_attn.q_norm.weight", hd)
        same(p + "self_attn.k_norm.weight", hd)
        same(p + "input_layernorm.weight", h)            # attention pre-norm (modules.hpp:140)
        same(p + "post_attention_layernorm.weight", h)   # attention post-norm (modules.hpp:164-168)
        check_linear(*fw.matrix(h, f), sd[p + "mlp.up_proj.weight"], rng)
        check_linear(*fw.matrix(h, f), sd[p + "mlp.gate_proj.weight"], rng)
        check_linear(*fw.matrix(f, h), sd[p + "mlp.down_proj.weight"], rng)
        same(p + "pre_feedforward_layernorm.weight", h)
        same(p + "post_feedforward_layernorm.weight", h)
    # tied LM head: logits = x @ embed.T, one scale per vocabulary entry
    check_linear(*fw.matrix(h, V), sd["model.embed_tokens.weight"], rng)
    assert fw.off == fw.b.size


def test_named_sizes_match_the_reference_files(conv):
    ge.load_package()
    from tiny_gemma_amd import weights
    assert weights.weight_file_bytes(conv.named_dims("270m")) == 437_586_944
    assert weights.weight_file_bytes(conv.named_dims("1B")) == 1_305_168_896
    with pytest.raises(KeyError):
        conv.named_dims("7B")


def test_missing_and_misshapen_tensors_are_errors(conv, tmp_path):
    sd = make_checkpoint(CFG, 4, torch.float32)
    src, dst = str(tmp_path / "m.safetensors"), str(tmp_path / "w.bin")
    broken = dict(sd)
    del broken["model.layers.1.mlp.gate_proj.weight"]
    st.save_file(broken, src)
    with pytest.raises(KeyError):  # py/gemma.py:389-394
        conv.convert_weights(src, dst, CFG)
    broken = dict(sd)
    broken["model.layers.0.self_attn.o_proj.weight"] = sd["model.layers.0.self_attn.o_proj.weight"].T.contiguous()
    st.save_file(broken, src)
    with pytest.raises(ValueError):
        conv.convert_weights(src, dst, CFG)
