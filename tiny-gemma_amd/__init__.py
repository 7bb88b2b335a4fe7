"""Python binding (ctypes) of libtinygemma_hip.so, the gfx950 implementation of tiny-gemma's
int8 weight-only path.  Everything here goes through the C ABI of include/tinygemma_hip.h;
there is no CPU fallback: importing works anywhere, every call needs the built library and a GPU.

The directory name carries a hyphen, so load it with ``load_package()`` from
``__graft_entry__`` (or importlib) under the module name ``tiny_gemma_amd``.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtinygemma_hip.so")
CSRC = os.path.join(HERE, "csrc")
SOURCES = ["tg_api.hip", "tg_gemv.hip", "tg_attn.hip", "tg_attn_prefill.hip", "tg_rows.hip", "tg_gemm_mfma.hip", "tg_sample.hip", "tg_repack.hip", "tg_probe.hip", "tg_decode_fused.hip"]
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-function",
               # leading scalar kernel arguments are preloaded into SGPRs by the dispatcher (no s_load round trip)
               "-mllvm", "-amdgpu-kernarg-preload-count=14"]

c_f32p = C.POINTER(C.c_float)
c_i8p = C.POINTER(C.c_int8)
c_i32p = C.POINTER(C.c_int32)


class TgError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"[{code}] {msg}")
        self.code = code


class Config(C.Structure):
    """tg_config == config::Config (csrc/include/config.hpp:7-44 of the reference)."""
    _fields_ = [("hidden_size", C.c_int), ("intermediate_size", C.c_int), ("n_layers", C.c_int), ("n_vocab", C.c_int),
                ("n_pos", C.c_int), ("n_pos_local", C.c_int), ("head_dim", C.c_int), ("n_head", C.c_int),
                ("n_kv", C.c_int), ("rope_theta", C.c_float), ("rope_theta_local", C.c_float), ("window_pattern", C.c_int)]


def build_library(verbose=False, changed_only=False):
    """hipcc cross-compiles for gfx950 without a GPU: one object per source, compiled in parallel, then one link.
    changed_only: recompile only sources newer than their object (a development convenience; the default compiles all)."""
    from concurrent.futures import ThreadPoolExecutor
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    headers = [os.path.join(CSRC, h) for h in ("tg_internal.h", "tg_gemv_parts.h", "tg_attn_decode.h")] + [os.path.join(HERE, "..", "include", "tinygemma_hip.h")]

    def compile_one(src):
        path, obj = os.path.join(CSRC, src), os.path.join(objdir, src + ".o")
        if changed_only and os.path.exists(obj) and all(os.path.getmtime(obj) > os.path.getmtime(d) for d in [path] + headers):
            return obj
        cmd = ["hipcc"] + flags + ["-c", path, "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed on " + src + ":\n" + r.stderr[-4000:])
        if verbose:
            print(" ".join(cmd))
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB_PATH]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc link failed:\n" + r.stderr[-4000:])
    return LIB_PATH


_lib = None


def lib():
    """Loads the built library; fails loudly if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(f"{LIB_PATH} is not built: run __graft_entry__.build() (hipcc --offload-arch=gfx950)")
    L = C.CDLL(LIB_PATH)
    L.tg_last_error.restype = C.c_char_p
    L.tg_status_string.restype = C.c_char_p
    L.tg_status_string.argtypes = [C.c_int]
    L.tg_device_name.restype = C.c_char_p
    L.tg_stream.restype = C.c_void_p
    L.tg_init.argtypes = [C.c_int]
    L.tg_config_named.argtypes = [C.c_char_p, C.POINTER(Config)]
    L.tg_qgemv.argtypes = [c_f32p, c_f32p, c_i8p, c_f32p, C.c_int, C.c_int]
    L.tg_qgemv_logits.argtypes = L.tg_qgemv.argtypes
    L.tg_qgemm.argtypes = [c_f32p, c_f32p, c_i8p, c_f32p, C.c_int, C.c_int, C.c_int]
    L.tg_qweight_create.argtypes = [c_i8p, c_f32p, C.c_int, C.c_int, C.POINTER(C.c_void_p)]
    L.tg_qweight_destroy.argtypes = [C.c_void_p]
    L.tg_dev_alloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
    L.tg_dev_free.argtypes = [C.c_void_p]
    L.tg_copy_h2d.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    L.tg_copy_d2h.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    L.tg_dev_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    L.tg_qgemv_dev.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
    L.tg_qgemm_dev.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
    L.tg_model_create.argtypes = [C.POINTER(Config), C.POINTER(C.c_void_p)]
    L.tg_model_load_weights.argtypes = [C.c_void_p, C.c_char_p]
    L.tg_model_load_weights_mem.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    L.tg_weight_file_bytes.argtypes = [C.POINTER(Config)]
    L.tg_weight_file_bytes.restype = C.c_size_t
    L.tg_model_destroy.argtypes = [C.c_void_p]
    L.tg_session_create.argtypes = [C.c_void_p, c_f32p, c_f32p, c_f32p, c_f32p, c_f32p, C.c_float, C.c_float, C.c_int,
                                    C.POINTER(C.c_void_p)]
    L.tg_session_reset.argtypes = [C.c_void_p]
    L.tg_session_release_workspace.argtypes = [C.c_void_p]
    L.tg_session_destroy.argtypes = [C.c_void_p]
    L.tg_session_position.argtypes = [C.c_void_p]
    L.tg_forward_prefill.argtypes = [C.c_void_p, c_i32p, C.c_int, c_f32p, c_i32p]
    L.tg_forward_decode.argtypes = [C.c_void_p, C.c_int32, c_f32p, c_i32p]
    L.tg_generate_greedy.argtypes = [C.c_void_p, c_i32p, C.c_int, C.c_int, c_i32p, C.POINTER(C.c_double), C.POINTER(C.c_double)]
    L.tg_decode_enqueue.argtypes = [C.c_void_p, C.c_int]
    L.tg_attention_prefill.argtypes = [c_f32p, c_f32p, c_f32p, c_f32p, C.c_int, C.c_int, C.c_int]
    L.tg_minp_logits.argtypes = [c_f32p, C.c_int, C.c_float, C.c_float, C.c_float, c_i32p]
    L.tg_decode_enqueue_sampled.argtypes = [C.c_void_p, C.c_int, C.c_float, C.c_float, c_f32p]
    L.tg_generate.argtypes = [C.c_void_p, c_i32p, C.c_int, C.c_int, C.c_float, C.c_float, c_f32p, c_i32p,
                              C.POINTER(C.c_double), C.POINTER(C.c_double)]
    L.tg_session_read_ids.argtypes = [C.c_void_p, c_i32p, C.c_int, c_i32p]
    L.tg_session_tap.argtypes = [C.c_void_p, C.c_int, c_f32p, C.c_int]
    L.tg_session_kv.argtypes = [C.c_void_p, C.c_int, c_f32p, c_f32p, c_i32p, c_i32p, c_i32p]
    L.tg_qgemm_dev_static.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
    L.tg_debug_launch_chain.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_double)]
    L.tg_debug_grid_barrier.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double), c_i32p]
    L.tg_set_fused_decode.argtypes = [C.c_int, C.c_int, C.c_int]
    L.tg_debug_gemm_clock.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double), c_i32p]
    L.tg_debug_fused_timestamps.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
    L.tg_debug_handover.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double), c_i32p, c_i32p, c_i32p]
    L.tg_debug_gemm_launches.argtypes = [C.POINTER(C.c_longlong)] * 3
    L.tg_debug_mfma_clock.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]
    L.tg_debug_xcd_deal.argtypes = [C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]
    L.tg_debug_l1_fill.argtypes = [C.c_int] * 5 + [C.POINTER(C.c_double)] * 3
    L.tg_decode_profile.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_double), c_i32p]
    L.tg_debug_repeat_kernel.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int]
    L.tg_block_attention.argtypes = [C.c_void_p, C.c_int, c_f32p, C.c_int]
    L.tg_block_mlp.argtypes = [C.c_void_p, C.c_int, c_f32p, C.c_int]
    L.tg_block_lm_head.argtypes = [C.c_void_p, c_f32p, C.c_int, c_f32p]
    L.tg_session_kv_prefill.argtypes = [C.c_void_p, C.c_int, c_f32p, c_f32p, C.c_int]
    _lib = L
    return L


def check(rc):
    if rc != 0:
        raise TgError(rc, lib().tg_last_error().decode(errors="replace"))


def _f(a):
    return a.ctypes.data_as(c_f32p) if a is not None else None


def init(device=0):
    check(lib().tg_init(device))
    return lib().tg_device_name().decode()


def named_config(name, n_layers=None):
    cfg = Config()
    check(lib().tg_config_named(name.encode(), C.byref(cfg)))
    if n_layers is not None:
        cfg.n_layers = n_layers
    return cfg


# ---- kernel level (mirrors gemv::launch_qgemv / launch_qgemv_logits / gemm::launch_qgemm) ----
def launch_qgemv(Cv, A, B, scales, inDim, outDim, logits=False):
    """C (zero on entry) += A.B ; C *= scales — host arrays in the reference layout."""
    fn = lib().tg_qgemv_logits if logits else lib().tg_qgemv
    check(fn(_f(Cv), _f(A), B.ctypes.data_as(c_i8p), _f(scales), inDim, outDim))


def launch_qgemm(Cm, A, B, scales, m, inDim, outDim):
    check(lib().tg_qgemm(_f(Cm), _f(A), B.ctypes.data_as(c_i8p), _f(scales), m, inDim, outDim))


def attention_prefill(q, k, v, is_sw, sw_context=512):
    """ops::attention_prefill on the device: q [4][S][256], k, v [S][256] -> o [4][S][256]."""
    q = np.ascontiguousarray(q, np.float32)
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    S = k.shape[0]
    assert q.shape == (4, S, 256) and k.shape == (S, 256) and v.shape == (S, 256)
    o = np.empty_like(q)
    check(lib().tg_attention_prefill(_f(o), _f(q), _f(k), _f(v), S, int(bool(is_sw)), int(sw_context)))
    return o


def minp_logits(logits, minp, temp, randf):
    """ops::minp_logits (ops.hpp:762): the sampled token id; `logits` is left untouched."""
    logits = np.ascontiguousarray(logits, np.float32)
    tok = C.c_int32(-1)
    check(lib().tg_minp_logits(_f(logits), logits.size, minp, temp, randf, C.byref(tok)))
    return tok.value


class DeviceBuffer:
    def __init__(self, nbytes):
        self.p = C.c_void_p()
        self.nbytes = nbytes
        check(lib().tg_dev_alloc(C.byref(self.p), nbytes))

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        check(lib().tg_copy_h2d(b.p, a.ctypes.data_as(C.c_void_p), a.nbytes))
        return b

    def to_numpy(self, dtype, shape):
        out = np.empty(shape, dtype)
        check(lib().tg_copy_d2h(out.ctypes.data_as(C.c_void_p), self.p, out.nbytes))
        return out

    def free(self):
        if self.p:
            lib().tg_dev_free(self.p)
            self.p = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:  # noqa: BLE001
            pass


class QWeight:
    """A reference-layout int8 matrix [in][out] + scales[out], resident on the GPU."""

    def __init__(self, B, scales):
        self.inDim, self.outDim = B.shape
        self.h = C.c_void_p()
        B = np.ascontiguousarray(B, np.int8)
        scales = np.ascontiguousarray(scales, np.float32)
        check(lib().tg_qweight_create(B.ctypes.data_as(c_i8p), _f(scales), self.inDim, self.outDim, C.byref(self.h)))

    def gemv(self, y_dev, x_dev, logits=False):
        check(lib().tg_qgemv_dev(y_dev.p, x_dev.p, self.h, int(logits)))

    def gemm(self, C_dev, A_dev, m):
        check(lib().tg_qgemm_dev(C_dev.p, A_dev.p, self.h, m))

    def gemm_clock(self, C_dev, A_dev, m):
        """tg_qgemm_dev with the matrix kernel reporting the shader clock it ran at: (MHz, average workgroup lifetime in us, workgroups)."""
        mhz, us, n = C.c_double(), C.c_double(), C.c_int32()
        check(lib().tg_debug_gemm_clock(C_dev.p, A_dev.p, self.h, m, C.byref(mhz), C.byref(us), C.byref(n)))
        return mhz.value, us.value, n.value

    def gemm_static(self, C_dev, A_dev, m):
        """tg_qgemm_dev on the library's fixed scratch: allocates nothing."""
        check(lib().tg_qgemm_dev_static(C_dev.p, A_dev.p, self.h, m))

    def free(self):
        if self.h:
            lib().tg_qweight_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:  # noqa: BLE001
            pass


def gemm_launches():
    """(few-row kernel, one workgroup per tile, two workgroups per compute unit): GEMM launches so far, by kernel."""
    a, b_, c = C.c_longlong(), C.c_longlong(), C.c_longlong()
    check(lib().tg_debug_gemm_launches(C.byref(a), C.byref(b_), C.byref(c)))
    return a.value, b_.value, c.value


def synchronize():
    check(lib().tg_synchronize())


# ---- model level (mirrors gemma::Transformer / read_weights / forward_* / generate) ----
class Transformer:
    def __init__(self, cfg):
        self.cfg = cfg
        self.h = C.c_void_p()
        check(lib().tg_model_create(C.byref(cfg), C.byref(self.h)))

    def read_weights(self, path):
        check(lib().tg_model_load_weights(self.h, path.encode()))

    def read_weights_mem(self, image):
        image = np.ascontiguousarray(image, np.uint8)
        check(lib().tg_model_load_weights_mem(self.h, image.ctypes.data_as(C.c_void_p), image.size))

    def weight_file_bytes(self):
        return lib().tg_weight_file_bytes(C.byref(self.cfg))

    def session(self, rope=None, rope_sw=None, gelu_table=None, gmin=-4.0, gmax=4.0, gsize=1024):
        return Session(self, rope, rope_sw, gelu_table, gmin, gmax, gsize)

    def free(self):
        if self.h:
            lib().tg_model_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:  # noqa: BLE001
            pass


class Session:
    """DecodeState + RoPE tables + GeLU table of one generation (transformer.hpp:193-202)."""

    def __init__(self, model, rope, rope_sw, gelu_table, gmin, gmax, gsize):
        self.model, self.cfg = model, model.cfg
        self.h = C.c_void_p()
        rc, rs = rope if rope is not None else (None, None)
        lc, ls = rope_sw if rope_sw is not None else (None, None)
        if gelu_table is not None:
            gsize = gelu_table.size
        check(lib().tg_session_create(model.h, _f(rc), _f(rs), _f(lc), _f(ls), _f(gelu_table), gmin, gmax, gsize, C.byref(self.h)))

    def release_workspace(self):
        check(lib().tg_session_release_workspace(self.h))

    def reset(self):
        check(lib().tg_session_reset(self.h))

    @property
    def position(self):
        return lib().tg_session_position(self.h)

    def prefill(self, ids, want_logits=True):
        ids = np.ascontiguousarray(ids, np.int32)
        logits = np.empty(self.cfg.n_vocab, np.float32) if want_logits else None
        arg = C.c_int32(-1)
        check(lib().tg_forward_prefill(self.h, ids.ctypes.data_as(c_i32p), ids.size, _f(logits), C.byref(arg)))
        return arg.value, logits

    def decode(self, tok, want_logits=True):
        logits = np.empty(self.cfg.n_vocab, np.float32) if want_logits else None
        arg = C.c_int32(-1)
        check(lib().tg_forward_decode(self.h, int(tok), _f(logits), C.byref(arg)))
        return arg.value, logits

    def greedy(self, prompt, n_decode):
        prompt = np.ascontiguousarray(prompt, np.int32)
        out = np.empty(n_decode + 1, np.int32)
        sp, sd = C.c_double(), C.c_double()
        check(lib().tg_generate_greedy(self.h, prompt.ctypes.data_as(c_i32p), prompt.size, n_decode,
                                       out.ctypes.data_as(c_i32p), C.byref(sp), C.byref(sd)))
        return out, sp.value, sd.value

    def decode_enqueue(self, n):
        check(lib().tg_decode_enqueue(self.h, n))

    def decode_enqueue_sampled(self, n, minp, temp, randf):
        randf = np.ascontiguousarray(randf, np.float32)
        assert randf.size >= n
        check(lib().tg_decode_enqueue_sampled(self.h, n, minp, temp, _f(randf)))

    def generate(self, prompt, n_decode, minp, temp, randf):
        """gemma::generate on ids: randf[n_decode + 1] uniform draws, used when minp < 1."""
        prompt = np.ascontiguousarray(prompt, np.int32)
        randf = np.ascontiguousarray(randf, np.float32)
        assert randf.size >= n_decode + 1
        out = np.empty(n_decode + 1, np.int32)
        sp, sd = C.c_double(), C.c_double()
        check(lib().tg_generate(self.h, prompt.ctypes.data_as(c_i32p), prompt.size, n_decode, minp, temp, _f(randf),
                                out.ctypes.data_as(c_i32p), C.byref(sp), C.byref(sd)))
        return out, sp.value, sd.value

    def read_ids(self, max_ids):
        out = np.empty(max_ids, np.int32)
        n = C.c_int32()
        check(lib().tg_session_read_ids(self.h, out.ctypes.data_as(c_i32p), max_ids, C.byref(n)))
        return out[:n.value]

    def tap(self, b, rows=1):
        out = np.empty((rows, self.cfg.hidden_size), np.float32)
        check(lib().tg_session_tap(self.h, b, _f(out), rows))
        return out

    def taps(self, rows=1):
        return np.stack([self.tap(b, rows) for b in range(2 * self.cfg.n_layers + 1)])

    def kv(self, layer):
        mp, pp, bp = C.c_int32(), C.c_int32(), C.c_int32()
        check(lib().tg_session_kv(self.h, layer, None, None, C.byref(pp), C.byref(bp), C.byref(mp)))
        k = np.empty((mp.value, self.cfg.head_dim), np.float32)
        v = np.empty_like(k)
        check(lib().tg_session_kv(self.h, layer, _f(k), _f(v), None, None, None))
        return k, v, pp.value, bp.value

    # ---- block level (modules::attention / mlp / lm_head one call at a time) ----
    def block_attention(self, layer, x):
        """x [rows][hidden] -> the attention block's output (rows > 1: prefill kernels, 1 row: decode kernels)."""
        x = np.array(x, np.float32, copy=True, order="C").reshape(-1, self.cfg.hidden_size)
        check(lib().tg_block_attention(self.h, layer, _f(x), x.shape[0]))
        return x

    def block_mlp(self, layer, x):
        x = np.array(x, np.float32, copy=True, order="C").reshape(-1, self.cfg.hidden_size)
        check(lib().tg_block_mlp(self.h, layer, _f(x), x.shape[0]))
        return x

    def block_lm_head(self, x):
        x = np.ascontiguousarray(x, np.float32).reshape(-1, self.cfg.hidden_size)
        logits = np.empty(self.cfg.n_vocab, np.float32)
        check(lib().tg_block_lm_head(self.h, _f(x), x.shape[0], _f(logits)))
        return logits

    def kv_prefill(self, layer, keys, values):
        """KVCache::update_prefill on one layer of an empty session: keys/values [rows][head_dim]."""
        keys = np.ascontiguousarray(keys, np.float32)
        values = np.ascontiguousarray(values, np.float32)
        assert keys.shape == values.shape and keys.shape[1] == self.cfg.head_dim
        check(lib().tg_session_kv_prefill(self.h, layer, _f(keys), _f(values), keys.shape[0]))

    def free(self):
        if self.h:
            lib().tg_session_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:  # noqa: BLE001
            pass
