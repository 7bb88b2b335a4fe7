"""Seeded inputs shared by tests/golden/make_golden.py (which records the reference's outputs) and
the tests (which regenerate the same inputs).  Only numpy; nothing here touches the reference."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# name: (inDim, outDim, logits variant, seed).  cfg1 is the bare matvec of the benchmark
# configuration list: x ~ N(0,1), W uniform in [-127,127] stored [640][2048], scales ~ U(0.001,0.02).
GEMV_CASES = {
    "cfg1_640x2048": (640, 2048, False, 101),
    "q_1152x1024": (1152, 1024, False, 102),
    "kv_640x256": (640, 256, False, 103),
    "o_1024x1152": (1024, 1152, False, 104),
    "up_1152x6912": (1152, 6912, False, 105),       # row tile 8 in the reference
    "down_6912x1152": (6912, 1152, False, 106),
    "down_2048x640": (2048, 640, False, 107),
    "sq_256x256": (256, 256, False, 108),
    "lmhead_640x262144": (640, 262144, True, 109),  # row tile 4
    "lmhead_1152x262144": (1152, 262144, True, 110),
}

# name: (m, inDim, outDim, seed): ragged m around the reference's 6-row / 256-row blocking
GEMM_CASES = {
    "m1_640x256": (1, 640, 256, 201),
    "m7_640x1024": (7, 640, 1024, 202),
    "m64_640x2048": (64, 640, 2048, 203),
    "m178_1152x1024": (178, 1152, 1024, 204),
    "m257_2048x640": (257, 2048, 640, 205),
    "m13_6912x1152": (13, 6912, 1152, 206),
    "m70_1152x6912": (70, 1152, 6912, 207),
}

RMSNORM_CASES = {"h640": (5, 640, 301), "h1152": (3, 1152, 302), "hd256": (8, 256, 303)}
ROPE_ROWS = np.array([0, 1, 2, 17, 511, 512, 1000, 4095, 16384, 32767])
# name: (S, is_sw, sw_context, seed)
ATTN_PREFILL_CASES = {"causal_40": (40, False, 512, 401), "window_700": (700, True, 512, 402), "window16_50": (50, True, 16, 403)}
# name: (max_pos, valid, seed)
ATTN_DECODE_CASES = {"one_key": (512, 1, 501), "partial_37": (512, 37, 502), "full_ring": (512, 512, 503), "global_1300": (2048, 1300, 504)}

# name: (shape, n_layers, seed, prompt tokens, decode steps, decode steps with taps, GeLU table size)
MODEL_CASES = {
    "small6": ("270m", 6, 11, 70, 12, 4, 1024),           # one global layer (l = 5), short prompt
    "small6_window": ("270m", 6, 12, 600, 6, 3, 1024),    # prompt longer than the 512-slot ring
    "small6_finelut": ("270m", 6, 11, 70, 12, 4, 1 << 20),  # near-continuous GeLU table: tight end-to-end check
    "full270m": ("270m", 18, 5, 64, 256, 2, 1024),        # 64-token prompt + 256 greedy steps
    "full270m_ties": ("270m", 18, 1, 64, 256, 0, 1024),   # same, a seed whose greedy path crosses near-ties of the logits
    "full1B": ("1B", 26, 1, 178, 1024, 2, 1024),          # 178-token prompt + 1024 greedy steps
}

# The two long benchmark configurations at full size (tests/golden/golden_long.npz):
# name: (shape, n_layers, seed, prompt tokens, greedy decode steps, GeLU table size)
LONG_CASES = {
    "prefill4096_1B": ("1B", 26, 1, 4096, 0, 1024),       # one forward over 4096 random tokens (weights of full1B)
    "long16k_270m": ("270m", 18, 5, 16384, 256, 1024),    # 16384-token prefill + 256 greedy steps (weights of full270m)
}
LONG_DECODE_LOGIT_STEPS = (0, 1, 128, 255)   # decode steps whose logits head is kept


def long_kv_rows(n_prompt):
    """Cache slots of a long prompt kept in the fixture (those below the layer's valid count are used)."""
    return np.unique(np.array([0, 1, 255, 511, 512, 1000, n_prompt // 2, n_prompt - 2, n_prompt - 1]))

# Block level (tests/golden/golden_blocks.npz): one modules::attention / mlp / lm_head call on a caller-supplied
# residual stream, on the shape lists of the reference's own unit tests (tests/scripts/unittests/run_tests.sh:6-32,
# all global attention on the 270m shape) plus what those never run: local layers (513-key window, ring cache) and
# the 1B shape.  Weights: the seeded generator's one-layer model; its layer 0 is global with window pattern 1 and
# local with the usual pattern 6.
# model name: (shape, weight seed, window pattern)
BLOCK_MODELS = {"270m_global": ("270m", 61, 1), "270m_local": ("270m", 61, 6), "1B_global": ("1B", 62, 1), "1B_local": ("1B", 62, 6)}
# case name: (model, kind, rows of the residual stream, keys already cached (attention decode), GeLU table size, seed)
BLOCK_CASES = {}
for _S in (1024, 281, 593, 480, 217, 57):
    BLOCK_CASES[f"attn_prefill_{_S}"] = ("270m_global", "attn", _S, 0, 1024, 700 + _S)
for _S in (281, 593, 480, 217, 57):
    BLOCK_CASES[f"mlp_prefill_{_S}"] = ("270m_global", "mlp", _S, 0, 8192, 800 + _S)       # the unit tests' table (8192 entries)
    BLOCK_CASES[f"mlp_prefill_{_S}_lut1024"] = ("270m_global", "mlp", _S, 0, 1024, 800 + _S)  # the command line's table
BLOCK_CASES["mlp_decode"] = ("270m_global", "mlp", 1, 0, 8192, 901)
BLOCK_CASES["mlp_decode_lut1024"] = ("270m_global", "mlp", 1, 0, 1024, 901)
for _S in (648, 209, 830, 103, 389, 57):
    BLOCK_CASES[f"attn_decode_{_S}"] = ("270m_global", "attn", 1, _S, 1024, 1000 + _S)
for _S in (103, 389, 209, 57):
    BLOCK_CASES[f"lm_head_prefill_{_S}"] = ("270m_global", "lm_head", _S, 0, 1024, 1100 + _S)
BLOCK_CASES["lm_head_decode"] = ("270m_global", "lm_head", 1, 0, 1024, 1201)
# not covered by the reference's tests
BLOCK_CASES["attn_prefill_local_700"] = ("270m_local", "attn", 700, 0, 1024, 1301)       # 513-key window
BLOCK_CASES["attn_decode_local_ring_700"] = ("270m_local", "attn", 1, 700, 1024, 1302)   # ring holds rows 188..699
BLOCK_CASES["attn_decode_local_300"] = ("270m_local", "attn", 1, 300, 1024, 1303)
BLOCK_CASES["attn_decode_global_5000"] = ("270m_global", "attn", 1, 5000, 1024, 1304)    # 32-key workgroups + merge launch
BLOCK_CASES["attn_prefill_1B_217"] = ("1B_global", "attn", 217, 0, 1024, 1401)
BLOCK_CASES["attn_prefill_1B_local_600"] = ("1B_local", "attn", 600, 0, 1024, 1402)
BLOCK_CASES["attn_decode_1B_389"] = ("1B_global", "attn", 1, 389, 1024, 1403)
BLOCK_CASES["mlp_prefill_1B_217"] = ("1B_global", "mlp", 217, 0, 8192, 1404)
BLOCK_CASES["mlp_prefill_1B_217_lut1024"] = ("1B_global", "mlp", 217, 0, 1024, 1404)
BLOCK_CASES["mlp_prefill_1B_700_lut1024"] = ("1B_global", "mlp", 700, 0, 1024, 1407)      # more than 448 rows: the tiled GEMM kernels
BLOCK_CASES["mlp_decode_1B"] = ("1B_global", "mlp", 1, 0, 8192, 1405)
BLOCK_CASES["mlp_decode_1B_lut1024"] = ("1B_global", "mlp", 1, 0, 1024, 1405)
BLOCK_CASES["lm_head_decode_1B"] = ("1B_global", "lm_head", 1, 0, 1024, 1406)
BLOCK_CASES["lm_head_prefill_1B_57"] = ("1B_global", "lm_head", 57, 0, 1024, 1408)


def block_config(model):
    shape, seed, pattern = BLOCK_MODELS[model]
    cfg = oracle_config(shape, 1)
    cfg.pattern = pattern
    return cfg, seed


def block_inputs(name):
    """(x [rows][hidden] ~ N(0,1) like the reference's unit tests, cached keys, cached values)."""
    model, kind, rows, cached, gsize, seed = BLOCK_CASES[name]
    hidden = {"270m": 640, "1B": 1152}[BLOCK_MODELS[model][0]]
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    k = rng.standard_normal((cached, 256)).astype(np.float32) if cached else None
    v = rng.standard_normal((cached, 256)).astype(np.float32) if cached else None
    return x, k, v


def block_rows(rows):
    """Rows of a block's output kept in the fixture."""
    return np.unique(np.concatenate([np.arange(0, rows, 29), np.arange(max(0, rows - 4), rows)]))


LOGIT_SAMPLE = np.arange(0, 262144, 61)   # logits of an lm_head block kept in the fixture

# Teacher-forced random-token streams (tests/golden/golden_blocks.npz, "stream/..."): after a short random prompt the
# reference is fed seeded random ids, so every step sees a fresh context (free-running greedy ids of a random-init
# model settle into a loop of a few tokens).  name: (shape, n_layers, weight seed, prompt tokens, steps, GeLU table size)
STREAM_CASES = {
    "stream270m": ("270m", 18, 5, 8, 320, 1024),
    "stream1B": ("1B", 26, 1, 8, 320, 1024),
    # the same streams with a near-continuous GeLU table: what is left is fp32 summation order
    "stream270m_finelut": ("270m", 18, 5, 8, 320, 1 << 20),
    "stream1B_finelut": ("1B", 26, 1, 8, 320, 1 << 20),
}
STREAM_LOGIT_STEPS = (0, 100, 319)


def stream_ids(name):
    shape, n_layers, seed, n_prompt, steps, gsize = STREAM_CASES[name]
    rng = np.random.default_rng(5000 + seed)
    return rng.integers(0, 262144, n_prompt).astype(np.int32), rng.integers(0, 262144, steps).astype(np.int32)


def gemv_inputs(i, n, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(i).astype(np.float32)
    W = rng.integers(-127, 128, (i, n), dtype=np.int8)
    s = rng.uniform(0.001, 0.02, n).astype(np.float32)
    return x, W, s


def gemm_inputs(m, i, n, seed):
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((m, i)).astype(np.float32)
    W = rng.integers(-127, 128, (i, n), dtype=np.int8)
    s = rng.uniform(0.001, 0.02, n).astype(np.float32)
    return A, W, s


def rmsnorm_inputs(rows, dim, seed):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((rows, dim)) * 3).astype(np.float32), (rng.standard_normal(dim) * 0.1).astype(np.float32)


def rope_apply_input(seed):
    return np.random.default_rng(seed).standard_normal((4, 9, 256)).astype(np.float32)


def gelu_input(seed):
    x = (np.random.default_rng(seed).standard_normal(4096) * 2.5).astype(np.float32)
    x[:8] = [-4.0, 4.0, -4.00001, 3.99999, 0.0, -0.0, 10.0, -10.0]
    return x


def embedding_inputs(seed):
    rng = np.random.default_rng(seed)
    wte = rng.integers(-127, 128, (1000, 640), dtype=np.int8)
    sc = rng.uniform(0.001, 0.02, 640).astype(np.float32)
    ids = rng.integers(0, 1000, 17).astype(np.int32)
    return ids, wte, sc


def attn_prefill_inputs(S, seed):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((4, S, 256)).astype(np.float32)
    k = rng.standard_normal((S, 256)).astype(np.float32)
    v = rng.standard_normal((S, 256)).astype(np.float32)
    return q, k, v


def attn_decode_inputs(max_pos, seed):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((4, 256)).astype(np.float32)
    kc = rng.standard_normal((max_pos, 256)).astype(np.float32)
    vc = rng.standard_normal((max_pos, 256)).astype(np.float32)
    return q, kc, vc


def attn_rows(S):
    """Query rows of an attention output kept in the fixture."""
    return np.unique(np.concatenate([np.arange(0, S, 37), np.arange(max(0, S - 6), S)]))


def tap_rows(S):
    """Prompt positions of the residual-stream taps kept in the fixture."""
    return np.unique(np.concatenate([np.arange(0, S, 11), [S - 1]]))


def argmax_input(seed):
    return np.random.default_rng(seed).standard_normal(262144).astype(np.float32)


# min-p sampler (ops::minp_logits): name -> (logit seed, logit scale, peaked, minp, temp, randf)
MINP_CASES = {
    "flat": (31, 0.5, False, 0.05, 1.0, 0.3),
    "warm": (32, 2.0, False, 0.2, 0.7, 0.93),
    "nomask": (33, 6.0, False, 0.0, 1.3, 0.5),
    "cold": (34, 3.0, False, 0.5, 0.25, 0.999),
    "masked_mass": (35, 1.0, False, 0.9, 1.0, 0.01),    # below-cut tokens keep their mass: the "probabilities" sum to >> 1
    "masked_late": (35, 1.0, False, 0.9, 1.0, 0.9999),
    "peaked": (36, 1.0, True, 0.05, 0.8, 0.77),          # a handful of dominant logits, like a trained model
    "peaked_tail": (36, 1.0, True, 0.0, 1.0, 0.99),
    "zero_draw": (37, 2.0, False, 0.1, 1.0, 0.0),        # randf = 0: the very first token
    "never_reached": (33, 6.0, False, 0.0, 1.3, 1.0),    # the running sum stays below randf: index 0 (ops.hpp:850)
}


def minp_input(seed, scale, peaked):
    rng = np.random.default_rng(seed)
    lg = (rng.standard_normal(262144) * scale).astype(np.float32)
    if peaked:
        hot = rng.integers(0, 262144, 12)
        lg[hot] += rng.uniform(8.0, 14.0, 12).astype(np.float32)
    return lg


def prompt_ids(seed, n):
    return np.random.default_rng(1000 + seed).integers(0, 262144, n).astype(np.int32)


def oracle_config(shape, n_layers):
    from oracle.oracle import named_config
    return named_config(shape, n_layers)


# ---- tokenizer (tokenizer.hpp; file format of py/convert.py:83-113) ----
TOKENIZER_VOCAB = 5000
TOKENIZER_SEED = 77


def tokenizer_vocab(seed=TOKENIZER_SEED, vocab_size=TOKENIZER_VOCAB):
    """A synthetic vocabulary laid out like Gemma's: specials, <start_of_turn>/<end_of_turn>/newline at 105-107,
    byte tokens <0x00>..<0xFF> at 238..493, "user" at 2364, "model" at 4368, unique pieces elsewhere.
    Returns (pieces: list of bytes, scores: float32 array); scores are multiples of 0.5 so that ties occur."""
    rng = np.random.default_rng(seed)
    pieces = [None] * vocab_size
    fixed = {0: b"<pad>", 1: b"<eos>", 2: b"<bos>", 3: b"<unk>", 4: b"<mask>", 105: b"<start_of_turn>", 106: b"<end_of_turn>",
             107: b"\n", 2364: b"user", 4368: b"model"}
    for i in range(256):
        fixed[238 + i] = ("<0x%02X>" % i).encode()
    fixed[494] = b"<0xabc>"   # three hex digits: still matches the reference's byte pattern
    fixed[495] = b" <0x41>"   # becomes a byte piece once its leading space is stripped
    for i, p in fixed.items():
        pieces[i] = p
    used = set(fixed.values())
    letters = "abcdefghijklmnopqrstuvwxyzABCDEFGH0123456789.,;:!?-'\"()"
    cands = [c.encode() for c in letters] + [b" "]
    cands += ["é".encode(), "ü".encode(), "ñ".encode(), "日".encode(), "本".encode(), "語".encode(),
              "\U0001F600".encode(), b"\xf0\x9f\x98\x80\x80"]
    cands += [(" " + c).encode() for c in "abcdefghijklmnopqrstuvwxyz"]
    small = "abcdefghij "
    for a in small:
        for b in small:
            cands.append((a + b).encode())
    while len(cands) < 3 * vocab_size:
        n = int(rng.integers(3, 9))
        w = "".join(small[int(k)] for k in rng.integers(0, len(small), n))
        cands.append(w.encode())
    it = iter(cands)
    for i in range(vocab_size):
        if pieces[i] is None:
            p = next(it)
            while p in used:
                p = next(it)
            used.add(p)
            pieces[i] = p
    scores = (-np.round(rng.uniform(0.0, 20.0, vocab_size) * 2.0) / 2.0).astype(np.float32)
    for i in fixed:
        scores[i] = 0.0
    return pieces, scores


def write_tokenizer_file(path, pieces, scores):
    import struct
    with open(path, "wb") as f:
        f.write(struct.pack("I", max(len(p) for p in pieces)))
        for p, s in zip(pieces, scores):
            f.write(struct.pack("fI", float(s), len(p)))
            f.write(p)


def tokenizer_texts(seed=TOKENIZER_SEED):
    """Byte strings to encode: vocabulary words, random letters, UTF-8 (1-4 byte code points), malformed UTF-8."""
    rng = np.random.default_rng(seed + 1)
    pieces, _ = tokenizer_vocab()
    small = "abcdefghij "
    texts = [b"", b" ", b"a", b"hello world", b"user model\n", "café 日本語 \U0001F600!".encode(),
             b"\x80\x80\x80", b"a\xc3", b"\xf0\x9f\x98\x80\x80\x80\x80 b", b"\xff\xfe abc", b"<0x41> <bos>"]
    for _ in range(24):
        n = int(rng.integers(1, 60))
        texts.append("".join(small[int(k)] for k in rng.integers(0, len(small), n)).encode())
    for _ in range(12):
        words = [pieces[int(k)] for k in rng.integers(496, TOKENIZER_VOCAB, int(rng.integers(2, 12)))]
        texts.append(b" ".join(words))
    texts.append("".join(small[int(k)] for k in rng.integers(0, len(small), 1500)).encode())
    return texts


def tokenizer_vocab_full(n=262144):
    """A full-size vocabulary for the command line front end (it always loads 262144 entries): the 5000 pieces of
    tokenizer_vocab() followed by unique filler pieces '~' + base-10 digits written with the letters k..t."""
    pieces, scores = tokenizer_vocab()
    tr = bytes.maketrans(b"0123456789", b"klmnopqrst")
    pieces = pieces + [b"~" + str(i).encode().translate(tr) for i in range(len(pieces), n)]
    scores = np.concatenate([scores, np.full(n - scores.size, -30.0, np.float32)])
    return pieces, scores
