"""TEST INFRASTRUCTURE, NOT PRODUCT CODE.

ctypes loaders for the two CPU checkers:

  * ``Oracle``  -> oracle/libtg_oracle.so, the scalar C restatement (tg_oracle.c)
  * ``Ref``     -> oracle/_ref/libtg_ref.so, the real reference compiled from its own sources
                   (exists only where the reference checkout was present at build time)

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module.
"""
import ctypes as C
import os
import subprocess
import threading

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "libtg_oracle.so")
REF_SO = os.path.join(HERE, "_ref", "libtg_ref.so")

c_f32p = C.POINTER(C.c_float)
c_i8p = C.POINTER(C.c_int8)
c_i32p = C.POINTER(C.c_int32)


def build(with_ref=True):
    """Compile the checkers (make). `ref` is skipped by the Makefile if the reference is absent."""
    targets = ["libtg_oracle.so"] + (["ref"] if with_ref else [])
    subprocess.run(["make", "-B", "-C", HERE] + targets, check=True, capture_output=True)


def _f(a):
    return a.ctypes.data_as(c_f32p) if a is not None else None


def _b(a):
    return a.ctypes.data_as(c_i8p)


def _i(a):
    return a.ctypes.data_as(c_i32p)


class Config(C.Structure):
    _fields_ = [("hidden", C.c_int), ("ffn", C.c_int), ("n_layers", C.c_int), ("vocab", C.c_int),
                ("n_pos", C.c_int), ("n_pos_local", C.c_int), ("head_dim", C.c_int), ("n_head", C.c_int),
                ("n_kv", C.c_int), ("theta", C.c_float), ("theta_local", C.c_float), ("pattern", C.c_int)]

    def as_tuple(self):
        return tuple(getattr(self, f) for f, _ in self._fields_)


def named_config(name, n_layers=None):
    base = {"270m": (640, 2048, 18), "1B": (1152, 6912, 26)}[name]
    cfg = Config(base[0], base[1], base[2] if n_layers is None else n_layers, 262144, 32768, 512, 256, 4, 1,
                 1000000.0, 10000.0, 6)
    return cfg


def run_big_stack(fn, *args, stack_mb=256):
    """Run fn on a thread with a large stack (the reference GEMM keeps its pack buffers,
    up to 7.5 MB, on the stack: csrc/include/linalg.hpp:258-259)."""
    out = {}

    def tgt():
        try:
            out["r"] = fn(*args)
        except BaseException as e:  # noqa: BLE001
            out["e"] = e

    old = threading.stack_size(stack_mb * 1024 * 1024)
    try:
        t = threading.Thread(target=tgt)
        t.start()
        t.join()
    finally:
        threading.stack_size(old)
    if "e" in out:
        raise out["e"]
    return out["r"]


class Oracle:
    def __init__(self, path=ORACLE_SO):
        if not os.path.exists(path):
            build(with_ref=False)
        L = self.L = C.CDLL(path)
        L.tgo_qgemv.argtypes = [c_f32p, c_f32p, c_i8p, c_f32p, C.c_int, C.c_int]
        L.tgo_qgemv_logits.argtypes = L.tgo_qgemv.argtypes
        L.tgo_qgemm.argtypes = [c_f32p, c_f32p, c_i8p, c_f32p, C.c_int, C.c_int, C.c_int]
        L.tgo_rmsnorm.argtypes = [c_f32p, c_f32p, C.c_int, C.c_int]
        L.tgo_rope_tables.argtypes = [C.c_float, C.c_int, C.c_int, c_f32p, c_f32p]
        L.tgo_rope_apply.argtypes = [c_f32p, C.c_int, C.c_int, C.c_int, c_f32p, c_f32p, C.c_int]
        L.tgo_gelu_table.argtypes = [C.c_float, C.c_float, C.c_int, c_f32p]
        L.tgo_gelu.argtypes = [c_f32p, C.c_size_t, c_f32p, C.c_float, C.c_float, C.c_int]
        L.tgo_embedding.argtypes = [c_f32p, c_i32p, C.c_int, c_i8p, c_f32p, C.c_int]
        L.tgo_attention_prefill.argtypes = [c_f32p, c_f32p, c_f32p, c_f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
        L.tgo_attention_decode.argtypes = [c_f32p, c_f32p, c_f32p, c_f32p, C.c_int, C.c_int, C.c_int]
        L.tgo_argmax.argtypes = [c_f32p, C.c_int]
        L.tgo_minp_logits.argtypes = [c_f32p, C.c_int, C.c_float, C.c_float, C.c_float]
        L.tgo_quantize.argtypes = [c_f32p, C.c_size_t, C.c_size_t, c_i8p, c_f32p]
        L.tgo_normal.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64, C.c_float]
        L.tgo_normal.restype = C.c_float
        L.tgo_weight_file_bytes.argtypes = [C.POINTER(Config)]
        L.tgo_weight_file_bytes.restype = C.c_size_t
        L.tgo_generate_weights_mem.argtypes = [C.POINTER(Config), C.c_uint64, C.c_void_p]
        L.tgo_generate_weights_file.argtypes = [C.POINTER(Config), C.c_uint64, C.c_char_p]
        L.tgo_model_create.argtypes = [C.POINTER(Config)]
        L.tgo_model_create.restype = C.c_void_p
        L.tgo_model_load_file.argtypes = [C.c_void_p, C.c_char_p]
        L.tgo_model_load_mem.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.tgo_model_destroy.argtypes = [C.c_void_p]
        L.tgo_session_create.argtypes = [C.c_void_p, C.c_float, C.c_float, C.c_int]
        L.tgo_session_create.restype = C.c_void_p
        L.tgo_session_destroy.argtypes = [C.c_void_p]
        L.tgo_prefill.argtypes = [C.c_void_p, c_i32p, C.c_int, c_f32p, c_i32p, c_f32p]
        L.tgo_decode.argtypes = [C.c_void_p, C.c_int32, c_f32p, c_i32p, c_f32p]
        L.tgo_kv_read.argtypes = [C.c_void_p, C.c_int, c_f32p, c_f32p, c_i32p, c_i32p, c_i32p]

    # ---- kernels ----
    def qgemv(self, x, W, s, logits=False):
        inn, out = W.shape
        y = np.zeros(out, np.float32)
        fn = self.L.tgo_qgemv_logits if logits else self.L.tgo_qgemv
        rc = fn(_f(y), _f(x), _b(W), _f(s), inn, out)
        if rc != 0:
            raise RuntimeError("Unsupported dimension")
        return y

    def qgemm(self, A, W, s):
        m = A.shape[0]
        inn, out = W.shape
        Cm = np.empty((m, out), np.float32)
        rc = self.L.tgo_qgemm(_f(Cm), _f(A), _b(W), _f(s), m, inn, out)
        if rc != 0:
            raise RuntimeError("Unsupported dimension")
        return Cm

    # ---- ops ----
    def rmsnorm(self, x, w):
        x = np.ascontiguousarray(x, np.float32).copy()
        rows = x.size // x.shape[-1]
        self.L.tgo_rmsnorm(_f(x), _f(w), rows, x.shape[-1])
        return x

    def rope_tables(self, theta, n_pos, dhead=256):
        c = np.empty((n_pos, dhead), np.float32)
        s = np.empty((n_pos, dhead), np.float32)
        self.L.tgo_rope_tables(theta, n_pos, dhead, _f(c), _f(s))
        return c, s

    def rope_apply(self, x, cos_t, sin_t, offset):
        x = np.ascontiguousarray(x, np.float32).copy()
        heads, seq, dhead = x.shape
        self.L.tgo_rope_apply(_f(x), heads, seq, dhead, _f(cos_t), _f(sin_t), offset)
        return x

    def gelu_table(self, gmin, gmax, size):
        t = np.empty(size, np.float32)
        self.L.tgo_gelu_table(gmin, gmax, size, _f(t))
        return t

    def gelu(self, x, table, gmin, gmax):
        x = np.ascontiguousarray(x, np.float32).copy()
        self.L.tgo_gelu(_f(x), x.size, _f(table), gmin, gmax, table.size)
        return x

    def embedding(self, ids, wte, scales):
        ids = np.ascontiguousarray(ids, np.int32)
        out = np.empty((ids.size, wte.shape[1]), np.float32)
        self.L.tgo_embedding(_f(out), _i(ids), ids.size, _b(wte), _f(scales), wte.shape[1])
        return out

    def attention_prefill(self, q, k, v, is_sw, sw_context=512):
        heads, S, dim = q.shape
        o = np.empty_like(q)
        self.L.tgo_attention_prefill(_f(o), _f(q), _f(k), _f(v), heads, S, dim, int(is_sw), sw_context)
        return o

    def attention_decode(self, q, kc, vc, valid):
        heads, dim = q.shape
        o = np.empty_like(q)
        self.L.tgo_attention_decode(_f(o), _f(q), _f(kc), _f(vc), heads, dim, valid)
        return o

    def argmax(self, logits):
        return self.L.tgo_argmax(_f(logits), logits.size)

    def minp_logits(self, logits, minp, temp, randf):
        """Returns (index, probabilities as the reference leaves them in the logits buffer)."""
        p = np.array(logits, np.float32, copy=True)
        idx = self.L.tgo_minp_logits(_f(p), p.size, minp, temp, randf)
        return idx, p

    # ---- producer ----
    def quantize(self, w):
        w = np.ascontiguousarray(w, np.float32)
        q = np.empty(w.shape, np.int8)
        s = np.empty(w.shape[1], np.float32)
        rc = self.L.tgo_quantize(_f(w), w.shape[0], w.shape[1], _b(q), _f(s))
        if rc != 0:
            raise ZeroDivisionError("all-zero column")
        return q, s

    def normal(self, seed, tensor_id, i, std):
        return self.L.tgo_normal(seed, tensor_id, i, std)

    def weight_file_bytes(self, cfg):
        return self.L.tgo_weight_file_bytes(C.byref(cfg))

    def generate_weights(self, cfg, seed):
        """Returns the weight file image as a uint8 array."""
        buf = np.empty(self.weight_file_bytes(cfg), np.uint8)
        rc = self.L.tgo_generate_weights_mem(C.byref(cfg), seed, buf.ctypes.data_as(C.c_void_p))
        if rc != 0:
            raise RuntimeError(f"generate_weights rc={rc}")
        return buf

    def generate_weights_file(self, cfg, seed, path):
        rc = self.L.tgo_generate_weights_file(C.byref(cfg), seed, path.encode())
        if rc != 0:
            raise RuntimeError(f"generate_weights_file rc={rc}")

    # ---- model ----
    def model(self, cfg, image=None, path=None):
        return _OracleModel(self, cfg, image, path)


class _Session:
    """Common prefill/decode front end of both checkers."""

    def prefill(self, ids, want_logits=True, taps=False):
        ids = np.ascontiguousarray(ids, np.int32)
        logits = np.empty(self.cfg.vocab, np.float32) if want_logits else None
        arg = C.c_int32(-1)
        tp = np.empty((2 * self.cfg.n_layers, ids.size, self.cfg.hidden), np.float32) if taps else None
        rc = self._prefill(ids, logits, arg, tp)
        if rc != 0:
            raise RuntimeError(f"prefill rc={rc}")
        return arg.value, logits, tp

    def decode(self, tok, want_logits=True, taps=False):
        logits = np.empty(self.cfg.vocab, np.float32) if want_logits else None
        arg = C.c_int32(-1)
        tp = np.empty((2 * self.cfg.n_layers, self.cfg.hidden), np.float32) if taps else None
        rc = self._decode(int(tok), logits, arg, tp)
        if rc != 0:
            raise RuntimeError(f"decode rc={rc}")
        return arg.value, logits, tp

    def greedy(self, prompt, n_decode):
        """gemma::generate's greedy branch (transformer.hpp:204-250) without tokenizer or EOS stop.
        Returns the n_decode + 1 sampled ids (first one comes from the prefill logits)."""
        tok, _, _ = self.prefill(prompt, want_logits=False)
        out = [tok]
        for _ in range(n_decode):
            tok, _, _ = self.decode(tok, want_logits=False)
            out.append(tok)
        return np.array(out, np.int32)


class _OracleModel:
    def __init__(self, orc, cfg, image, path):
        self.o, self.cfg = orc, cfg
        self.h = orc.L.tgo_model_create(C.byref(cfg))
        if image is not None:
            rc = orc.L.tgo_model_load_mem(self.h, image.ctypes.data_as(C.c_void_p), image.size)
        else:
            rc = orc.L.tgo_model_load_file(self.h, path.encode())
        if rc != 0:
            orc.L.tgo_model_destroy(self.h)
            self.h = None
            raise RuntimeError("Could not open file." if rc == -1 else f"load rc={rc}")

    def session(self, gmin=-4.0, gmax=4.0, gsize=1024):
        return _OracleSession(self, gmin, gmax, gsize)

    def __del__(self):
        if getattr(self, "h", None):
            self.o.L.tgo_model_destroy(self.h)
            self.h = None


class _OracleSession(_Session):
    def __init__(self, model, gmin, gmax, gsize):
        self.model, self.cfg, self.L = model, model.cfg, model.o.L
        self.h = self.L.tgo_session_create(model.h, gmin, gmax, gsize)

    def _prefill(self, ids, logits, arg, tp):
        return self.L.tgo_prefill(self.h, _i(ids), ids.size, _f(logits), C.byref(arg), _f(tp))

    def _decode(self, tok, logits, arg, tp):
        return self.L.tgo_decode(self.h, tok, _f(logits), C.byref(arg), _f(tp))

    def kv(self, layer):
        mp, pp, bp = C.c_int32(), C.c_int32(), C.c_int32()
        self.L.tgo_kv_read(self.h, layer, None, None, C.byref(pp), C.byref(bp), C.byref(mp))
        k = np.empty((mp.value, self.cfg.head_dim), np.float32)
        v = np.empty_like(k)
        self.L.tgo_kv_read(self.h, layer, _f(k), _f(v), None, None, None)
        return k, v, pp.value, bp.value

    def __del__(self):
        if getattr(self, "h", None):
            self.L.tgo_session_destroy(self.h)
            self.h = None


class Ref:
    """The real reference behind oracle/ref_wrap.cpp."""

    @staticmethod
    def available():
        return os.path.exists(REF_SO)

    def __init__(self, path=REF_SO):
        L = self.L = C.CDLL(path)
        L.ref_qgemv.argtypes = [c_f32p, c_f32p, c_i8p, c_f32p, C.c_int, C.c_int]
        L.ref_qgemv_logits.argtypes = L.ref_qgemv.argtypes
        L.ref_qgemm.argtypes = [c_f32p, c_f32p, c_i8p, c_f32p, C.c_int, C.c_int, C.c_int]
        L.ref_rmsnorm.argtypes = [c_f32p, c_f32p, C.c_int, C.c_int]
        L.ref_rope_tables.argtypes = [C.c_float, C.c_int, C.c_int, c_f32p, c_f32p]
        L.ref_rope_apply.argtypes = [c_f32p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int, C.c_int]
        L.ref_gelu_table.argtypes = [C.c_float, C.c_float, C.c_int, c_f32p]
        L.ref_gelu.argtypes = [c_f32p, C.c_int, C.c_float, C.c_float, C.c_int]
        L.ref_embedding.argtypes = [c_f32p, c_i32p, C.c_int, c_i8p, c_f32p, C.c_int, C.c_int]
        L.ref_attention_prefill.argtypes = [c_f32p, c_f32p, c_f32p, c_f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
        L.ref_attention_decode.argtypes = [c_f32p, c_f32p, c_f32p, c_f32p, C.c_int, C.c_int, C.c_int, C.c_int]
        L.ref_argmax.argtypes = [c_f32p]
        L.ref_minp_logits.argtypes = [c_f32p, C.c_float, C.c_float, C.c_float]
        L.ref_model_create.argtypes = [C.c_int] * 9 + [C.c_float, C.c_float, C.c_int]
        L.ref_model_create.restype = C.c_void_p
        L.ref_model_load.argtypes = [C.c_void_p, C.c_char_p]
        L.ref_model_destroy.argtypes = [C.c_void_p]
        L.ref_session_create.argtypes = [C.c_void_p, C.c_float, C.c_float, C.c_int]
        L.ref_session_create.restype = C.c_void_p
        L.ref_session_destroy.argtypes = [C.c_void_p]
        L.ref_prefill.argtypes = [C.c_void_p, c_i32p, C.c_int, c_f32p, c_i32p, c_f32p]
        L.ref_decode.argtypes = [C.c_void_p, C.c_int, c_f32p, c_i32p, c_f32p]
        L.ref_kv_read.argtypes = [C.c_void_p, C.c_int, c_f32p, c_f32p, c_i32p, c_i32p, c_i32p]
        L.ref_block_attention.argtypes = [C.c_void_p, C.c_int, c_f32p, C.c_int]
        L.ref_block_mlp.argtypes = [C.c_void_p, C.c_int, c_f32p, C.c_int]
        L.ref_block_lm_head.argtypes = [C.c_void_p, c_f32p, C.c_int, c_f32p]
        L.ref_kv_prefill.argtypes = [C.c_void_p, C.c_int, c_f32p, c_f32p, C.c_int]
        L.ref_tok_create.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_int, C.c_int]
        L.ref_tok_create.restype = C.c_void_p
        L.ref_tok_destroy.argtypes = [C.c_void_p]
        L.ref_tok_encode.argtypes = [C.c_void_p, C.c_char_p, C.c_int, c_i32p, C.c_int]
        L.ref_tok_decode_piece.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_char_p, C.c_int]
        L.ref_tok_decode.argtypes = [C.c_void_p, c_i32p, C.c_int, C.c_char_p, C.c_int]

    def qgemv(self, x, W, s, logits=False):
        inn, out = W.shape
        y = np.zeros(out, np.float32)
        fn = self.L.ref_qgemv_logits if logits else self.L.ref_qgemv
        rc = fn(_f(y), _f(x), _b(W), _f(s), inn, out)
        if rc != 0:
            raise RuntimeError("Unsupported dimension")
        return y

    def qgemm(self, A, W, s):
        m = A.shape[0]
        inn, out = W.shape
        Cm = np.empty((m, out), np.float32)
        rc = run_big_stack(self.L.ref_qgemm, _f(Cm), _f(A), _b(W), _f(s), m, inn, out)
        if rc != 0:
            raise RuntimeError("Unsupported dimension")
        return Cm

    def rmsnorm(self, x, w):
        x = np.ascontiguousarray(x, np.float32).copy()
        self.L.ref_rmsnorm(_f(x), _f(w), x.size // x.shape[-1], x.shape[-1])
        return x

    def rope_tables(self, theta, n_pos, dhead=256):
        c = np.empty((n_pos, dhead), np.float32)
        s = np.empty((n_pos, dhead), np.float32)
        self.L.ref_rope_tables(theta, n_pos, dhead, _f(c), _f(s))
        return c, s

    def rope_apply(self, x, theta, n_pos, offset):
        x = np.ascontiguousarray(x, np.float32).copy()
        heads, seq, dhead = x.shape
        self.L.ref_rope_apply(_f(x), heads, seq, dhead, theta, n_pos, offset)
        return x

    def gelu_table(self, gmin, gmax, size):
        t = np.empty(size, np.float32)
        self.L.ref_gelu_table(gmin, gmax, size, _f(t))
        return t

    def gelu(self, x, gmin, gmax, size):
        x = np.ascontiguousarray(x, np.float32).copy()
        self.L.ref_gelu(_f(x), x.size, gmin, gmax, size)
        return x

    def embedding(self, ids, wte, scales):
        ids = np.ascontiguousarray(ids, np.int32)
        out = np.empty((ids.size, wte.shape[1]), np.float32)
        self.L.ref_embedding(_f(out), _i(ids), ids.size, _b(wte), _f(scales), wte.shape[0], wte.shape[1])
        return out

    def attention_prefill(self, q, k, v, is_sw, sw_context=512):
        heads, S, dim = q.shape
        o = np.empty_like(q)
        self.L.ref_attention_prefill(_f(o), _f(q), _f(k), _f(v), heads, S, dim, int(is_sw), sw_context)
        return o

    def attention_decode(self, q, kc, vc, valid):
        heads, dim = q.shape
        o = np.empty_like(q)
        self.L.ref_attention_decode(_f(o), _f(q), _f(kc), _f(vc), heads, dim, kc.shape[0], valid)
        return o

    def argmax(self, logits):
        assert logits.size == 262144
        return self.L.ref_argmax(_f(logits))

    def minp_logits(self, logits, minp, temp, randf):
        assert logits.size == 262144
        p = np.array(logits, np.float32, copy=True)
        idx = self.L.ref_minp_logits(_f(p), minp, temp, randf)
        return idx, p

    def tokenizer(self, path, bos_id, eos_id, vocab_size, chat_format):
        return _RefTokenizer(self, path, bos_id, eos_id, vocab_size, chat_format)

    def model(self, cfg, path):
        return _RefModel(self, cfg, path)


class _RefModel:
    def __init__(self, ref, cfg, path):
        self.r, self.cfg = ref, cfg
        self.h = ref.L.ref_model_create(*cfg.as_tuple())
        if ref.L.ref_model_load(self.h, path.encode()) != 0:
            ref.L.ref_model_destroy(self.h)
            self.h = None
            raise RuntimeError("Could not open file.")

    def session(self, gmin=-4.0, gmax=4.0, gsize=1024):
        return _RefSession(self, gmin, gmax, gsize)

    def __del__(self):
        if getattr(self, "h", None):
            self.r.L.ref_model_destroy(self.h)
            self.h = None


class _RefSession(_Session):
    def __init__(self, model, gmin, gmax, gsize):
        self.model, self.cfg, self.L = model, model.cfg, model.r.L
        self.h = self.L.ref_session_create(model.h, gmin, gmax, gsize)

    def _prefill(self, ids, logits, arg, tp):
        return run_big_stack(self.L.ref_prefill, self.h, _i(ids), ids.size, _f(logits), C.byref(arg), _f(tp))

    def _decode(self, tok, logits, arg, tp):
        return self.L.ref_decode(self.h, tok, _f(logits), C.byref(arg), _f(tp))

    # ---- one block at a time (modules::attention / mlp / lm_head) ----
    def block_attention(self, layer, x):
        x = np.array(x, np.float32, copy=True, order="C").reshape(-1, self.cfg.hidden)
        run_big_stack(self.L.ref_block_attention, self.h, layer, _f(x), x.shape[0])
        return x

    def block_mlp(self, layer, x):
        x = np.array(x, np.float32, copy=True, order="C").reshape(-1, self.cfg.hidden)
        run_big_stack(self.L.ref_block_mlp, self.h, layer, _f(x), x.shape[0])
        return x

    def block_lm_head(self, x):
        x = np.ascontiguousarray(x, np.float32).reshape(-1, self.cfg.hidden)
        logits = np.empty(self.cfg.vocab, np.float32)
        self.L.ref_block_lm_head(self.h, _f(x), x.shape[0], _f(logits))
        return logits

    def kv_prefill(self, layer, keys, values):
        keys = np.ascontiguousarray(keys, np.float32)
        values = np.ascontiguousarray(values, np.float32)
        self.L.ref_kv_prefill(self.h, layer, _f(keys), _f(values), keys.shape[0])

    def kv(self, layer):
        mp, pp, bp = C.c_int32(), C.c_int32(), C.c_int32()
        self.L.ref_kv_read(self.h, layer, None, None, C.byref(pp), C.byref(bp), C.byref(mp))
        k = np.empty((mp.value, self.cfg.head_dim), np.float32)
        v = np.empty_like(k)
        self.L.ref_kv_read(self.h, layer, _f(k), _f(v), None, None, None)
        return k, v, pp.value, bp.value

    def __del__(self):
        if getattr(self, "h", None):
            self.L.ref_session_destroy(self.h)
            self.h = None


class _RefTokenizer:
    """sentencepiece::Tokenizer of the reference (tokenizer.hpp), bytes in / bytes out."""

    def __init__(self, ref, path, bos_id, eos_id, vocab_size, chat_format):
        self.L = ref.L
        self.h = self.L.ref_tok_create(str(path).encode(), bos_id, eos_id, vocab_size, int(bool(chat_format)))
        if not self.h:
            raise RuntimeError("Cannot open model file: " + str(path))

    def encode(self, text):
        cap = 16 + 4 * len(text)
        ids = np.empty(cap, np.int32)
        n = self.L.ref_tok_encode(self.h, text, len(text), _i(ids), cap)
        assert n <= cap
        return ids[:n].copy()

    def decode_piece(self, token, prev_token):
        buf = C.create_string_buffer(4096)
        n = self.L.ref_tok_decode_piece(self.h, int(token), int(prev_token), buf, 4096)
        if n == -2:
            raise ValueError("the reference threw std::invalid_argument")
        assert n >= 0
        return buf.raw[:n]

    def decode(self, ids):
        ids = np.ascontiguousarray(ids, np.int32)
        cap = 1 << 20
        buf = C.create_string_buffer(cap)
        n = self.L.ref_tok_decode(self.h, _i(ids), ids.size, buf, cap)
        if n == -2:
            raise ValueError("the reference threw std::invalid_argument")
        assert 0 <= n <= cap
        return buf.raw[:n]

    def __del__(self):
        if getattr(self, "h", None):
            self.L.ref_tok_destroy(self.h)
            self.h = None
