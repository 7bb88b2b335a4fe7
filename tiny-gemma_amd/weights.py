"""Random-init weight files in the reference's on-disk format.

Counterpart, for synthetic checkpoints, of the reference's converter: the int8 weight-only
quantizer of py/weight_handlers.py:10-20 and the flat, header-less little-endian file that
py/gemma.py:27-77 writes and csrc/include/transformer.hpp:99-165 reads:

    wte int8[vocab][hidden] + f32[hidden] | RMSw f32[hidden]
    per layer: Q,K,V,O (int8 + f32 scales) | RMSq RMSk attn_pre attn_post | up, gate, down | mlp_pre mlp_post
    lm_head int8[hidden][vocab] + f32[vocab]        (tied: the transpose of the fp32 wte, re-quantized)

Matrices are [in][out] row-major with one fp32 scale per output column.
"""
import numpy as np


def quantize_weight(w):
    """scale = max|w| over axis 0 / 127 (fp32); q = rint(w / scale) as int8 (ties to even)."""
    w = np.asarray(w, np.float32)
    assert w.ndim >= 2, "Error, quantizing 1d dimensional weights"
    scales = (np.max(np.abs(w), axis=0, keepdims=True) / np.float32(127.0)).astype(np.float32)
    if not np.all(scales > 0):
        raise ZeroDivisionError("all-zero column")
    q = np.rint(w / scales).astype(np.int8)
    return q, scales


def dequantize(q, scales):
    return q.astype(np.float32) * scales


def layer_is_local(cfg, l):
    return (l % cfg.window_pattern) != (cfg.window_pattern - 1)


def weight_file_bytes(cfg):
    h, f, V, hd = cfg.hidden_size, cfg.intermediate_size, cfg.n_vocab, cfg.head_dim
    qo, kv = cfg.n_head * hd, cfg.n_kv * hd
    per_layer = (h * qo + 4 * qo) + 2 * (h * kv + 4 * kv) + (qo * h + 4 * h) + 2 * 4 * hd + 2 * 4 * h \
        + 2 * (h * f + 4 * f) + (f * h + 4 * h) + 2 * 4 * h
    return V * h + 4 * h + 4 * h + per_layer * cfg.n_layers + h * V + 4 * V


def random_weight_image(cfg, seed, std=0.02, norm_std=0.1):
    """Returns the file image (uint8 array) of a random-init model: N(0, std) matrices,
    N(0, norm_std) norm weights, lm_head tied to wte."""
    rng = np.random.default_rng(seed)
    h, f, V, hd = cfg.hidden_size, cfg.intermediate_size, cfg.n_vocab, cfg.head_dim
    qo, kv = cfg.n_head * hd, cfg.n_kv * hd
    out = np.empty(weight_file_bytes(cfg), np.uint8)
    pos = 0

    def put(a):
        nonlocal pos
        b = np.ascontiguousarray(a).view(np.uint8).reshape(-1)
        out[pos:pos + b.size] = b
        pos += b.size

    def normal(shape, s):
        return rng.standard_normal(shape, dtype=np.float32) * np.float32(s)

    def put_q(shape):
        q, s = quantize_weight(normal(shape, std))
        put(q)
        put(s)

    wte = normal((V, h), std)
    q, s = quantize_weight(wte)
    put(q)
    put(s)
    put(normal(h, norm_std))
    lm_q, lm_s = quantize_weight(np.ascontiguousarray(wte.T))
    del wte
    for _ in range(cfg.n_layers):
        put_q((h, qo))
        put_q((h, kv))
        put_q((h, kv))
        put_q((qo, h))
        put(normal(hd, norm_std))
        put(normal(hd, norm_std))
        put(normal(h, norm_std))
        put(normal(h, norm_std))
        put_q((h, f))
        put_q((h, f))
        put_q((f, h))
        put(normal(h, norm_std))
        put(normal(h, norm_std))
    put(lm_q)
    put(lm_s)
    assert pos == out.size
    return out
