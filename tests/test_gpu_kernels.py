"""GPU: the int8 GEMV / GEMM through the C ABI against the CPU checker on the same seeded inputs.

Tolerance: the GEMV sums each column in fp32 in a different (parallel) order than the reference's
row-by-row walk, so it agrees to fp32 rounding: norm-relative error <= 3e-6 here (the bound of
the task is 1e-3).  On integer-valued inputs with power-of-two scales every order gives the same
bits, so those must match exactly.  The prefill GEMM keeps the reference's per-element order
(one fused chain over k) and must be bit-exact.
"""
import numpy as np
import pytest

import golden_inputs as gi
from conftest import normrel

pytestmark = pytest.mark.gpu
GEMV_TOL = 3e-6


@pytest.mark.parametrize("name", list(gi.GEMV_CASES))
def test_qgemv_vs_checker(tg, oracle, golden, name):
    i, n, logits, seed = gi.GEMV_CASES[name]
    x, W, s = gi.gemv_inputs(i, n, seed)
    y = np.zeros(n, np.float32)
    tg.launch_qgemv(y, x, W, s, i, n, logits=logits)
    ref = oracle.qgemv(x, W, s, logits)
    assert normrel(y, ref) < GEMV_TOL
    assert np.abs(y - ref).max() <= 2e-5 * np.abs(ref).max()
    assert normrel(y[:2048], golden[f"gemv/{name}/head"]) < GEMV_TOL  # the compiled reference's own output


@pytest.mark.parametrize("i,n,logits", [(256, 256, False), (640, 2048, False), (1152, 6912, False), (6912, 1152, False),
                                        (2048, 640, False), (1152, 262144, True)])
def test_qgemv_integer_inputs_bit_exact(tg, i, n, logits):
    rng = np.random.default_rng(i * 7 + n)
    x = rng.integers(-8, 9, i).astype(np.float32)
    W = rng.integers(-127, 128, (i, n), dtype=np.int8)
    s = np.full(n, 2.0 ** -10, np.float32)
    y = np.zeros(n, np.float32)
    tg.launch_qgemv(y, x, W, s, i, n, logits=logits)
    exact = (x.astype(np.int64) @ W.astype(np.int64)).astype(np.float64) * 2.0 ** -10
    assert np.array_equal(y.astype(np.float64), exact)


def test_qgemv_extreme_weights(tg, oracle):
    """All weights at +-127 and at 0; a zero input; a one-hot input picks out one row of W."""
    i, n = 640, 2048
    s = np.linspace(0.001, 0.02, n).astype(np.float32)
    x = np.random.default_rng(1).standard_normal(i).astype(np.float32)
    for fill in (127, -127, 0):
        W = np.full((i, n), fill, np.int8)
        y = np.zeros(n, np.float32)
        tg.launch_qgemv(y, x, W, s, i, n)
        assert normrel(y, oracle.qgemv(x, W, s)) < GEMV_TOL if fill else not y.any()
    W = np.random.default_rng(2).integers(-127, 128, (i, n), dtype=np.int8)
    y = np.zeros(n, np.float32)
    tg.launch_qgemv(y, np.zeros(i, np.float32), W, s, i, n)
    assert not y.any()
    e = np.zeros(i, np.float32)
    e[333] = 1.0
    tg.launch_qgemv(y, e, W, s, i, n)
    assert np.array_equal(y, W[333].astype(np.float32) * s)


def test_qgemv_accumulates_into_c_like_the_reference(tg, oracle):
    """linalg.hpp:52-107: C += A.B, then C *= scales: a non-zero C is carried through the scale."""
    x, W, s = gi.gemv_inputs(640, 256, 5)
    c0 = np.random.default_rng(6).standard_normal(256).astype(np.float32)
    y = c0.copy()
    tg.launch_qgemv(y, x, W, s, 640, 256)
    ref = (c0.astype(np.float64) + x.astype(np.float64) @ W.astype(np.float64)) * s
    assert normrel(y, ref) < GEMV_TOL


def test_unsupported_shapes_raise(tg):
    """Same legal set and same failure as ROW_SWITCH / COL_SWITCH (static_switch.hpp:7-58)."""
    for i, n in [(512, 256), (256, 512), (262144, 256), (100, 100)]:
        x = np.zeros(i, np.float32)
        W = np.zeros((i, n), np.int8)
        s = np.ones(n, np.float32)
        with pytest.raises(tg.TgError) as e:
            tg.launch_qgemv(np.zeros(n, np.float32), x, W, s, i, n)
        assert e.value.code == -1 and "Unsupported" in str(e.value)
        with pytest.raises(tg.TgError):
            tg.launch_qgemm(np.zeros((2, n), np.float32), np.zeros((2, i), np.float32), W, s, 2, i, n)


@pytest.fixture
def exact_gemm(tg):
    """The vector-ALU GEMM that keeps the reference's per-element order (tg_set_gemm_mode(0))."""
    tg.lib().tg_set_gemm_mode(0)
    yield
    tg.lib().tg_set_gemm_mode(1)


@pytest.mark.parametrize("name", list(gi.GEMM_CASES))
def test_qgemm_exact_mode_bit_exact(tg, oracle, golden, exact_gemm, name):
    m, i, n, seed = gi.GEMM_CASES[name]
    A, W, s = gi.gemm_inputs(m, i, n, seed)
    Cm = np.full((m, n), np.nan, np.float32)  # launch_qgemm overwrites C (linalg.hpp:244)
    tg.launch_qgemm(Cm, A, W, s, m, i, n)
    assert np.array_equal(Cm, oracle.qgemm(A, W, s))
    assert np.array_equal(Cm.reshape(-1)[:2048], golden[f"gemm/{name}/head"])


@pytest.mark.parametrize("name", list(gi.GEMM_CASES))
def test_qgemm_mfma(tg, oracle, golden, name):
    """Default prefill GEMM: int8 matrix cores on three int8 digit planes of the power-of-two scaled activations
    (22 bits + sign of the row maximum), exact int32 sums: norm-relative error at the fp32-rounding level (<= 3e-6)."""
    m, i, n, seed = gi.GEMM_CASES[name]
    A, W, s = gi.gemm_inputs(m, i, n, seed)
    Cm = np.full((m, n), np.nan, np.float32)
    tg.launch_qgemm(Cm, A, W, s, m, i, n)
    ref = oracle.qgemm(A, W, s)
    assert not np.isnan(Cm).any()
    assert normrel(Cm, ref) < 3e-6
    assert np.abs(Cm - ref).max() <= 2e-5 * np.abs(ref).max()
    assert normrel(Cm.reshape(-1)[:2048], golden[f"gemm/{name}/head"]) < 3e-6


def test_qgemm_mfma_exact_cases(tg):
    """Integer activations and power-of-two scales are exact through the digit planes;
    rows of very different magnitude (1e-6 ... 1e4, and an all-zero row) keep their own scaling."""
    rng = np.random.default_rng(7)
    A = rng.integers(-8, 9, (70, 1152)).astype(np.float32)
    A[3] = 0.0
    W = rng.integers(-127, 128, (1152, 1024), dtype=np.int8)
    s = np.full(1024, 2.0 ** -7, np.float32)
    Cm = np.empty((70, 1024), np.float32)
    tg.launch_qgemm(Cm, A, W, s, 70, 1152, 1024)
    exact = (A.astype(np.int64) @ W.astype(np.int64)).astype(np.float64) * 2.0 ** -7
    assert np.array_equal(Cm.astype(np.float64), exact)
    A = rng.standard_normal((9, 640)).astype(np.float32) * np.float32(10.0) ** rng.integers(-6, 5, (9, 1)).astype(np.float32)
    W = rng.integers(-127, 128, (640, 256), dtype=np.int8)
    s = rng.uniform(0.001, 0.02, 256).astype(np.float32)
    Cm = np.empty((9, 256), np.float32)
    tg.launch_qgemm(Cm, A, W, s, 9, 640, 256)
    ref = (A.astype(np.float64) @ W.astype(np.float64)) * s.astype(np.float64)
    for r in range(9):
        assert normrel(Cm[r], ref[r]) < 3e-6


def _digit_plane_closed_form(A, W, s):
    """The int8-MFMA GEMM's documented arithmetic, restated with numpy integers: per-row power-of-two scaling into
    [2^21, 2^22), round to nearest even, three signed base-256 digits, exact integer contractions, fp32 recombination
    (two fused multiply-adds), inverse row factor, column scale."""
    A = A.astype(np.float32)
    amax = np.abs(A).max(axis=1)
    _, e = np.frexp(amax)  # amax = f * 2^e, f in [0.5, 1)
    e = np.where(amax > 0, e, 22)
    mul = np.ldexp(np.float32(1.0), 22 - e).astype(np.float32)
    inv = np.ldexp(np.float32(1.0), e - 22).astype(np.float32)
    xi = np.rint(A * mul[:, None]).astype(np.int64)
    a0 = ((xi + 128) & 255) - 128
    r1 = (xi - a0) >> 8
    a1 = ((r1 + 128) & 255) - 128
    a2 = (r1 - a1) >> 8
    assert np.abs(a2).max() <= 127 and np.array_equal(65536 * a2 + 256 * a1 + a0, xi)
    # |sum| <= 127 * 128 * K < 2^31: float64 products and sums of these integers are exact (and go through BLAS)
    Wf = W.astype(np.float64)
    s0, s1, s2 = ((a.astype(np.float64) @ Wf).astype(np.int64) for a in (a0, a1, a2))
    f32 = lambda z: z.astype(np.float32)
    inner = f32(f32(s1).astype(np.float64) * 256.0 + f32(s0).astype(np.float64))   # one rounding: fused multiply-add
    v = f32(f32(s2).astype(np.float64) * 65536.0 + inner.astype(np.float64))
    return (v * inv[:, None]) * s[None, :].astype(np.float32)


@pytest.mark.parametrize("shape", [(70, 1152, 1024, 11), (33, 6912, 1152, 12), (200, 1152, 6912, 13), (5, 256, 640, 14)])
def test_qgemm_mfma_equals_digit_plane_closed_form(tg, shape):
    """Bit-for-bit: a dropped or mis-weighted digit plane, a wrong rounding of the activations or a wrong row factor
    cannot hide inside a tolerance here."""
    m, i, n, seed = shape
    A, W, s = gi.gemm_inputs(m, i, n, seed)
    A[0] *= np.float32(1e-5)
    A[m - 1] *= np.float32(3e4)
    Cm = np.empty((m, n), np.float32)
    tg.launch_qgemm(Cm, A, W, s, m, i, n)
    assert np.array_equal(Cm, _digit_plane_closed_form(A, W, s))


@pytest.mark.parametrize("shape", [(2048, 1152, 6912, 31), (1920, 1152, 6912, 32), (2300, 1024, 6912, 33), (6200, 640, 2048, 34),
                                   (2048, 256, 6912, 35), (2048, 2048, 6912, 36)])
def test_qgemm_two_workgroups_per_unit_equal_the_other_kernels_and_the_closed_form(tg, shape):
    """The default kernel for products of more than 448 rows with at least one output tile per compute unit
    (tg_set_gemm_lds(n): from n / 2 tiles per unit; 0 = never): two workgroups share a compute unit, both operands go
    through an LDS ring and a third of the accumulators sit in ordinary vector registers.  Same integer
    sums and epilogue: the result must equal the one-workgroup-per-tile kernel's (tg_set_gemm_lds(0)) and the closed
    form bit for bit.  Shapes: K of 9,
    8, 5, 2 and 16 groups of four k steps; row blocks a multiple of 8, 15 (a tile count that is no multiple of 8: no
    XCD mapping), 18 and 49; a last row block that is partly padding."""
    m, i, n, seed = shape
    A, W, s = gi.gemm_inputs(m, i, n, seed)
    A[1] *= np.float32(1e-4)
    A[m - 1] *= np.float32(3e3)
    out, ran = [], []
    try:
        for lds in (1, 0):
            tg.check(tg.lib().tg_set_gemm_lds(lds))
            Cm = np.full((m, n), np.nan, np.float32)
            before = tg.gemm_launches()
            tg.launch_qgemm(Cm, A, W, s, m, i, n)
            ran.append(tuple(b - a for a, b in zip(before, tg.gemm_launches())))
            out.append(Cm)
    finally:
        tg.check(tg.lib().tg_set_gemm_lds(2))
    assert ran == [(0, 0, 1), (0, 1, 0)]     # the two calls really ran on the two kernels
    assert np.array_equal(out[0], out[1])
    assert np.array_equal(out[0], _digit_plane_closed_form(A, W, s))


def test_device_resident_gemv_matches_host_entry(tg, oracle):
    x, W, s = gi.gemv_inputs(1152, 6912, 9)
    w = tg.QWeight(W, s)
    xd = tg.DeviceBuffer.from_numpy(x)
    yd = tg.DeviceBuffer(4 * 6912)
    for _ in range(3):
        w.gemv(yd, xd)
    tg.synchronize()
    y = yd.to_numpy(np.float32, 6912)
    y2 = np.zeros(6912, np.float32)
    tg.launch_qgemv(y2, x, W, s, 1152, 6912)
    assert np.array_equal(y, y2)  # deterministic: same bits every launch
    assert normrel(y, oracle.qgemv(x, W, s)) < GEMV_TOL


def test_full_size_properties(tg):
    """LM-head size (302 MB of weights): linearity and a checksum of checksums, no CPU checker needed."""
    i, n = 1152, 262144
    rng = np.random.default_rng(3)
    W = rng.integers(-127, 128, (i, n), dtype=np.int8)
    s = np.full(n, 2.0 ** -9, np.float32)
    w = tg.QWeight(W, s)
    xa = rng.integers(-4, 5, i).astype(np.float32)
    xb = rng.integers(-4, 5, i).astype(np.float32)
    outs = []
    for x in (xa, xb, xa + xb):
        xd = tg.DeviceBuffer.from_numpy(x)
        yd = tg.DeviceBuffer(4 * n)
        w.gemv(yd, xd, logits=True)
        tg.synchronize()
        outs.append(yd.to_numpy(np.float32, n))
    assert np.array_equal(outs[0] + outs[1], outs[2])  # exact on integer data
    colsum = W.astype(np.int64).sum(axis=1)            # sum_c y[c] = s * sum_r x[r] * rowsum(W)[r]
    assert float(outs[0].astype(np.float64).sum()) == float((xa.astype(np.int64) * colsum).sum()) * 2.0 ** -9


# ---- prefill attention (ops::attention_prefill, ops.hpp:377-526) through the op-level entry point ----

def _dense_rows(q, k, v, rows, is_sw, ctx):
    """float64 softmax(q.k/16).v for the given query rows, keys qs-ctx..qs (local) or 0..qs (causal)."""
    out = np.zeros((q.shape[0], len(rows), 256), np.float64)
    k64, v64 = k.astype(np.float64), v.astype(np.float64)
    for n, i in enumerate(rows):
        lo = max(0, i - ctx) if is_sw else 0
        sc = (q[:, i, :].astype(np.float64) @ k64[lo:i + 1].T) / 16.0
        p = np.exp(sc - sc.max(axis=1, keepdims=True))
        out[:, n, :] = (p / p.sum(axis=1, keepdims=True)) @ v64[lo:i + 1]
    return out


ATTN_MODES = {
    # name: (kernel mode, planes mode, fp16 format)
    "fp32_mfma": (0, 1, 1),
    "f16x2": (1, 1, 1),                 # the default: two fp16 planes, 16- or 32-query workgroups by prompt length
    "f16x2_32q": (2, 1, 1),
    "f16x2_16q_planes": (3, 2, 1),      # fed from pre-split plane images at any length (what 2048 tokens and more get)
    "f16x2_32q_planes": (2, 2, 1),      # 32x32x16 matrix instructions, two waves per head (what long prompts get)
    "f16x2_32q_planes_16x16": (2, 2, 2),  # the same images and workgroups on the 16x16x32 kernel
    "bf16x3": (1, 1, 0),                # three bf16 planes, six products
    "bf16x3_16q_planes": (3, 2, 0),
    "bf16x3_32q_planes": (2, 2, 0),
}


@pytest.fixture(params=list(ATTN_MODES.values()), ids=list(ATTN_MODES))
def attn_mode(tg, request):
    """The fp32 matrix path and the split paths: both operand formats, both workgroup sizes, operands staged by the
    workgroup or copied from pre-split plane images."""
    mode, planes, f16 = request.param
    L = tg.lib()
    tg.check(L.tg_set_attn_prefill_mode(mode))
    tg.check(L.tg_set_attn_prefill_planes(planes))
    tg.check(L.tg_set_attn_prefill_format(f16))
    yield mode
    tg.check(L.tg_set_attn_prefill_mode(1))
    tg.check(L.tg_set_attn_prefill_planes(1))
    tg.check(L.tg_set_attn_prefill_format(1))


def test_attention_prefill_operand_outside_the_fp16_range_is_an_error(tg):
    """The two-plane fp16 format cannot hold a value beyond +-65504: the call must fail, not return infinities; the
    three-plane bf16 format takes the same input (fp32's range) and gives the dense float64 result."""
    S = 70
    q, k, v = gi.attn_prefill_inputs(S, 77)
    v[5, 100] = 1.0e5
    L = tg.lib()
    try:
        for planes in (1, 2):
            tg.check(L.tg_set_attn_prefill_planes(planes))
            with pytest.raises(tg.TgError) as e:
                tg.attention_prefill(q, k, v, False, 512)
            assert e.value.code == -7 and "65504" in str(e.value)
        tg.check(L.tg_set_attn_prefill_format(0))
        o = tg.attention_prefill(q, k, v, False, 512)
        assert normrel(o, _dense_rows(q, k, v, np.arange(S), False, 512)) < 2e-6
    finally:
        tg.check(L.tg_set_attn_prefill_planes(1))
        tg.check(L.tg_set_attn_prefill_format(1))
    q[0, 3, 7] = np.nan                      # NaN in an operand is reported the same way
    with pytest.raises(tg.TgError):
        tg.attention_prefill(q, k, gi.attn_prefill_inputs(S, 77)[2], False, 512)


@pytest.mark.parametrize("name", list(gi.ATTN_PREFILL_CASES))
def test_attention_prefill_vs_fixture_and_checker(tg, oracle, golden, attn_mode, name):
    S, sw, ctx, seed = gi.ATTN_PREFILL_CASES[name]
    q, k, v = gi.attn_prefill_inputs(S, seed)
    o = tg.attention_prefill(q, k, v, sw, ctx)
    # fp32 throughout; only the summation order differs from the reference's per-key scan
    assert normrel(o[:, gi.attn_rows(S), :], golden[f"attn_prefill/{name}"]) < 2e-6
    assert normrel(o, oracle.attention_prefill(q, k, v, sw, ctx)) < 2e-6


@pytest.mark.parametrize("S", [1500, 4099])
def test_attention_prefill_split_key_ranges(tg, oracle, attn_mode, S):
    """Causal layers long enough for the key ranges to be cut into chunks and merged (S > 512); 4099 is ragged
    against both the 16-query and the 32-key tiling."""
    q, k, v = gi.attn_prefill_inputs(S, 410 + S)
    o = tg.attention_prefill(q, k, v, False, 512)
    rows = np.unique(np.concatenate([np.arange(0, S, 97), np.arange(505, 530), np.arange(S - 20, S)]))
    assert normrel(o[:, rows, :], _dense_rows(q, k, v, rows, False, 512)) < 2e-6
    if S <= 2000:
        assert normrel(o, oracle.attention_prefill(q, k, v, False, 512)) < 2e-6
    # the same tokens through a local layer: 513-key window
    ol = tg.attention_prefill(q, k, v, True, 512)
    assert normrel(ol[:, rows, :], _dense_rows(q, k, v, rows, True, 512)) < 2e-6
    assert np.array_equal(ol[:, :513, :], o[:, :513, :]) or normrel(ol[:, :513, :], o[:, :513, :]) < 2e-6


@pytest.mark.parametrize("S,ctx", [(33, 512), (178, 512), (300, 15), (300, 47), (513, 512), (514, 512), (1000, 100), (1000, 512)])
def test_attention_prefill_short_prompts_cut_into_key_chunks(tg, attn_mode, S, ctx):
    """Prompts with fewer query tiles than compute units: causal and local layers are both cut into chunks of key
    tiles (down to one tile) and merged.  With a window of 15 or 47 keys a chunk starts before the window of the
    tile's later queries: a chunk without a single valid key for some query must come out as weight 0."""
    q, k, v = gi.attn_prefill_inputs(S, 900 + S + ctx)
    rows = np.arange(S)
    for is_sw in (False, True):
        o = tg.attention_prefill(q, k, v, is_sw, ctx)
        assert np.isfinite(o).all()
        assert normrel(o, _dense_rows(q, k, v, rows, is_sw, ctx)) < 2e-6


def test_machine_probes_return_sane_figures(tg):
    """The three timing probes behind the C ABI run, end normally (every wait in them is bounded) and report figures
    of the right order: a dependent launch costs microseconds, a barrier round did not time out, and the matrix cores
    issue one 32x32x32 int8 instruction per 32 clocks at a clock between 1 and 2.6 GHz."""
    import ctypes as C
    L = tg.lib()
    us, flag, cpm, mhz = C.c_double(), C.c_int32(), C.c_double(), C.c_double()
    tg.check(L.tg_debug_launch_chain(200, 256, C.byref(us)))
    assert 0.5 < us.value < 50.0
    tg.check(L.tg_debug_grid_barrier(50, 64, 0, 1 << 16, C.byref(us), C.byref(flag)))
    assert flag.value == 0 and 0.1 < us.value < 100.0
    for operands in (0, 1, 2):
        tg.check(L.tg_debug_mfma_clock(256, 2000, operands, C.byref(cpm), C.byref(mhz)))
        print(f"mfma probe operands {operands}: {cpm.value:.2f} clocks per instruction at {mhz.value:.0f} MHz")
        assert 31.9 < cpm.value < 36.0 and 1000.0 < mhz.value < 2600.0
    assert L.tg_debug_mfma_clock(0, 10, 0, C.byref(cpm), C.byref(mhz)) == -4
    assert L.tg_debug_mfma_clock(8, 10, 3, C.byref(cpm), C.byref(mhz)) == -4
    # what a compute unit pulls through its L1: from its XCD's L2 (a shared megabyte) far more than from memory
    per_wg, total, per_wg_mem, total_mem = C.c_double(), C.c_double(), C.c_double(), C.c_double()
    tg.check(L.tg_debug_l1_fill(256, 8, 256, 1024, 0, C.byref(per_wg), C.byref(total), C.byref(mhz)))
    tg.check(L.tg_debug_l1_fill(256, 8, 126, 1 << 20, 1, C.byref(per_wg_mem), C.byref(total_mem), C.byref(mhz)))
    print(f"l1 fill: {per_wg.value:.0f} GB/s per workgroup from L2 ({total.value / 1e3:.1f} TB/s), {per_wg_mem.value:.0f} from memory ({total_mem.value / 1e3:.1f} TB/s)")
    assert 30.0 < per_wg.value < 400.0 and 5.0 < per_wg_mem.value < per_wg.value and total_mem.value < 8000.0
    assert L.tg_debug_l1_fill(256, 5, 256, 1024, 0, C.byref(per_wg), C.byref(total), C.byref(mhz)) == -4
    # the deal of workgroups to the XCDs that the few-row GEMM, the prefetch workgroups and the tile mappings rely on:
    # round-robin inside a launch, and launches that follow each other on the stream start on the same XCD
    wgs = [288, 416, 16, 3, 1000, 257]
    n = len(wgs)
    first, bad = (C.c_int * n)(), (C.c_int * n)()
    tg.check(L.tg_debug_xcd_deal(n, (C.c_int * n)(*wgs), first, bad))
    print("xcd deal: first", list(first), "out of order", list(bad))
    assert list(bad) == [0] * n and len(set(first)) == 1 and 0 <= first[0] < 8
    assert L.tg_debug_xcd_deal(0, (C.c_int * n)(*wgs), first, bad) == -4
    assert L.tg_debug_l1_fill(256, 8, 255, 1024, 0, C.byref(per_wg), C.byref(total), C.byref(mhz)) == -4
    assert L.tg_debug_l1_fill(256, 8, 256, 1000, 0, C.byref(per_wg), C.byref(total), C.byref(mhz)) == -4
    assert L.tg_debug_l1_fill(4096, 16, 65536, 1024, 0, C.byref(per_wg), C.byref(total), C.byref(mhz)) == -4  # hours of reads
