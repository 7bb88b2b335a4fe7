"""CPU: the C-ABI library loads and exports every symbol include/tinygemma_hip.h declares, and the
host-side logic that needs no GPU behaves (configs, file sizes, error reporting).  No compute."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import __graft_entry__ as ge

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def pkg():
    tg = ge.load_package()
    if not os.path.exists(tg.LIB_PATH):
        tg.build_library()
    return tg


def declared_symbols(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tg_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(pkg):
    """Both headers: the contract (tinygemma_hip.h) and the knobs, probes and planning helpers (tinygemma_hip_debug.h)."""
    lib = C.CDLL(pkg.LIB_PATH)
    contract, debug = declared_symbols("tinygemma_hip.h"), declared_symbols("tinygemma_hip_debug.h")
    assert len(contract) >= 30 and len(debug) >= 20
    assert not set(contract) & set(debug)
    missing = [n for n in contract + debug if not hasattr(lib, n)]
    assert not missing, missing


def test_the_contract_header_holds_no_knobs_or_probes():
    """What a maintainer of the reference binds to: entry points that stand for a reference interface, the lifetime of
    models and sessions, taps, and the entry point that allocates nothing.  Process-wide knobs (other than the taps
    switch), timing probes and planning helpers live in the debug header."""
    contract = declared_symbols("tinygemma_hip.h")
    stray = [n for n in contract if n.startswith(("tg_debug_", "tg_plan_")) or (n.startswith("tg_set_") and n != "tg_set_taps")
             or n in ("tg_decode_profile", "tg_reset_knobs")]
    assert not stray, stray
    debug = declared_symbols("tinygemma_hip_debug.h")
    for n in ("tg_reset_knobs", "tg_set_fused_decode", "tg_debug_handover", "tg_debug_grid_barrier", "tg_decode_profile",
              "tg_plan_attention_prefill"):
        assert n in debug, n


def test_every_exported_symbol_is_declared(pkg):
    """Nothing is exported behind the headers' backs."""
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", pkg.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted({ln.split()[-1] for ln in out.splitlines() if " T tg_" in ln})
    declared = set(declared_symbols("tinygemma_hip.h")) | set(declared_symbols("tinygemma_hip_debug.h"))
    undeclared = [n for n in exported if n not in declared]
    assert not undeclared, undeclared


def test_named_configs(pkg):
    """CONFIG_MAP of csrc/include/config.hpp:46-48."""
    c = pkg.named_config("270m")
    assert (c.hidden_size, c.intermediate_size, c.n_layers, c.n_vocab, c.n_pos, c.n_pos_local, c.head_dim, c.n_head, c.n_kv,
            c.window_pattern) == (640, 2048, 18, 262144, 32768, 512, 256, 4, 1, 6)
    c = pkg.named_config("1B")
    assert (c.hidden_size, c.intermediate_size, c.n_layers) == (1152, 6912, 26)
    assert c.rope_theta == 1000000.0 and c.rope_theta_local == 10000.0
    with pytest.raises(pkg.TgError):
        pkg.named_config("7B")


def test_weight_file_bytes(pkg):
    lib = pkg.lib()
    assert lib.tg_weight_file_bytes(C.byref(pkg.named_config("270m"))) == 437586944
    assert lib.tg_weight_file_bytes(C.byref(pkg.named_config("1B"))) == 1305168896


def test_status_strings(pkg):
    lib = pkg.lib()
    assert lib.tg_status_string(0) == b"ok"
    assert lib.tg_status_string(-2) == b"Could not open file."  # transformer.hpp:163
    assert b"dimension" in lib.tg_status_string(-1)


def test_no_gpu_is_an_error_not_a_fallback(pkg):
    """Without a device every compute entry point must fail loudly."""
    import subprocess
    import sys
    code = ("import sys; sys.path.insert(0, %r); import __graft_entry__ as ge; tg = ge.load_package(); import numpy as np\n"
            "try:\n    tg.init(0)\nexcept tg.TgError as e:\n    print('ERR', e.code); sys.exit(0)\nprint('HAVE_GPU')\n") % ROOT
    env = dict(os.environ, HIP_VISIBLE_DEVICES="-1", ROCR_VISIBLE_DEVICES="-1")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    assert "ERR -6" in r.stdout, r.stdout


def test_missing_library_is_reported(pkg, tmp_path, monkeypatch):
    monkeypatch.setattr(pkg, "_lib", None)
    monkeypatch.setattr(pkg, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(FileNotFoundError):
        pkg.lib()


# ---- host-side planning of a prefill (no GPU) ---------------------------------------------------------------------

def attention_plan(lib, S, n_cu, window):
    cap = 1 << 16
    items = np.zeros((cap, 4), np.int32)
    tq, n, nsplit = C.c_int(), C.c_int(), C.c_int()
    lib.tg_plan_attention_prefill.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int32), C.c_int,
                                              C.POINTER(C.c_int), C.POINTER(C.c_int)]
    rc = lib.tg_plan_attention_prefill(S, n_cu, window, C.byref(tq), items.ctypes.data_as(C.POINTER(C.c_int32)), cap, C.byref(n),
                                       C.byref(nsplit))
    assert rc == 0 and n.value <= cap
    return tq.value, items[:n.value].copy(), nsplit.value


@pytest.mark.parametrize("S,window", [(1, -1), (33, -1), (178, -1), (178, 512), (300, 15), (300, 47), (513, 512), (514, 512),
                                      (1000, -1), (1000, 512), (1000, 100), (4096, -1), (4096, 512), (4099, -1), (16384, -1),
                                      (16384, 512)])
def test_attention_work_list_covers_every_visible_key_exactly_once(pkg, S, window):
    """What the list must guarantee whatever its balance: for every query, every key it may see (causal; local: the
    `window` keys before it and itself) lies in exactly one work item of the query's tile; slots are numbered 0..n-1;
    items come heaviest first."""
    n_cu = 256
    tq, items, nsplit = attention_plan(pkg.lib(), S, n_cu, window)
    assert tq in (16, 32)
    nq = (S + tq - 1) // tq
    if len(items) == 0:
        # one workgroup per query tile over its whole range: only where that is balanced or cannot be improved
        assert nq >= n_cu or nq == 1 or (window >= 0 and S > 2048)
        return
    per_tile = {}
    for qt, tb, te, slot in items:
        assert 0 <= qt < nq and 0 <= tb < te
        per_tile.setdefault(int(qt), []).append((int(tb), int(te), int(slot)))
    assert sorted(per_tile) == list(range(nq))
    slots = sorted(slot for chunks in per_tile.values() for _, _, slot in chunks if slot >= 0)
    assert slots == list(range(len(slots)))
    assert sum(1 for chunks in per_tile.values() if len(chunks) > 1) == nsplit
    lengths = [int(te - tb) for _, tb, te, _ in items]
    assert lengths == sorted(lengths, reverse=True)
    # every query tile cuts its key range at the same places (multiples of the chunk length from its first key tile),
    # so that workgroups running side by side walk the same keys
    full = max(int(te - tb) for qt, tb, te, slot in items if slot >= 0) if nsplit else 0
    for qt, chunks in per_tile.items():
        chunks.sort()
        if len(chunks) > 1:
            clen = chunks[0][1] - chunks[0][0]
            assert all(c[1] - c[0] == clen for c in chunks[:-1]) and clen <= full
            assert clen // 2 <= chunks[-1][1] - chunks[-1][0] < clen + (clen + 1) // 2
        assert all(a[1] == b[0] for a, b in zip(chunks, chunks[1:]))        # contiguous, disjoint
        assert (len(chunks) == 1) == (chunks[0][2] == -1)                     # whole tiles write the output themselves
        q_first, q_last = qt * tq, min(qt * tq + tq, S) - 1
        lo = max(0, q_first - window) if window >= 0 else 0                   # first key any query of the tile sees
        assert chunks[0][0] * 32 <= lo and chunks[0][0] * 32 + 32 > lo        # starts at the key tile that holds it
        assert (chunks[-1][1] - 1) * 32 <= q_last < chunks[-1][1] * 32        # ends at the key tile of the last query
    if nq < n_cu:
        # fewer query tiles than compute units: chains as short as the number of units allows (one item per unit);
        # causal layers of long prompts take several rounds instead (a row's last chunk takes a remainder of less than
        # half a chunk with it)
        assert len(items) <= n_cu or max(lengths) == 1 or window < 0
    if window < 0 and len(items) > n_cu:
        # several rounds: the chunk length is the one whose list ends earliest when the units take the items in list
        # order (an item costs its key tiles + 4); never later than with the plain rule (about 8 items per unit, chunks
        # of 16 key tiles or more)
        def span(lens):
            import heapq
            free_at = [0] * n_cu
            end = 0
            for n in lens:
                t = heapq.heappop(free_at) + 4 + n
                heapq.heappush(free_at, t)
                end = max(end, t)
            return end
        nts = [(min(qt * tq + tq, S) + 31) // 32 for qt in range(nq)]
        c = max(16, sum(nts) // (n_cu * 8))
        plain = []
        for nt in nts:
            nc = (nt + c - 1) // c
            if nc > 1 and nt - (nc - 1) * c < (c + 1) // 2:
                nc -= 1
            plain += [nt - ch * c if ch + 1 == nc else c for ch in range(nc)]
        plain.sort(reverse=True)
        assert span(lengths) <= span(plain)
        if S == 4096:
            assert span(lengths) <= 0.85 * span(plain)   # 527 items of up to 23 key tiles -> 492 of up to 25


@pytest.mark.parametrize("S,n_cu", [(100, 1), (178, 2), (600, 3), (2100, 8), (4096, 16), (5000, 40)])
def test_attention_work_list_on_few_compute_units(pkg, S, n_cu):
    """The planner with far fewer compute units than query tiles (several rounds even for short prompts, chunks longer
    than any key range): every key tile of every query tile still lies in exactly one item."""
    tq, items, nsplit = attention_plan(pkg.lib(), S, n_cu, -1)
    nq = (S + tq - 1) // tq
    covered = {}
    for qt, tb, te, slot in items:
        covered.setdefault(int(qt), []).append((int(tb), int(te)))
    if len(items) == 0:
        return   # one workgroup per query tile over its whole range
    for qt in range(nq):
        chunks = sorted(covered[qt])
        assert chunks[0][0] == 0 and all(a[1] == b[0] for a, b in zip(chunks, chunks[1:]))
        assert chunks[-1][1] == (min(qt * tq + tq, S) + 31) // 32


def test_decode_launch_mode_rule(pkg, monkeypatch):
    """Left to the library, greedy steps of a model that streams under 5 MB of weights per launch (the 270m shape: 3.0 MB)
    replay updated graphs, larger ones (the 1B shape: 7.7 MB) are stream launches; an explicit setting wins; under a
    profiler the library's own choice is stream launches and graph replay is refused."""
    lib = pkg.lib()
    f = lib.tg_plan_decode_launch_mode
    f.argtypes = [C.c_void_p]
    small, big = pkg.named_config("270m"), pkg.named_config("1B")
    assert lib.tg_set_graphs(-1) == 0
    assert f(C.byref(small)) == 2 and f(C.byref(big)) == 0 and f(None) == -1
    try:
        for mode in (0, 1, 2):
            assert lib.tg_set_graphs(mode) == 0
            assert f(C.byref(small)) == mode and f(C.byref(big)) == mode
        assert lib.tg_set_graphs(3) != 0 and lib.tg_set_graphs(-2) != 0
        assert lib.tg_set_graphs(-1) == 0
        monkeypatch.setenv("ROCP_TOOL_LIBRARIES", "librocprofiler-sdk-tool.so")
        assert f(C.byref(small)) == 0 and f(C.byref(big)) == 0
        assert lib.tg_set_graphs(2) != 0 and lib.tg_set_graphs(1) != 0 and lib.tg_set_graphs(0) == 0
    finally:
        monkeypatch.delenv("ROCP_TOOL_LIBRARIES", raising=False)
        assert lib.tg_set_graphs(-1) == 0


def test_gemm_k_parts_rule(pkg):
    f = pkg.lib().tg_plan_gemm_k_parts
    f.argtypes = [C.c_int] * 4
    assert f(178, 6912, 1152, 256) == 4      # few rows, 108 stages of K: 4 x 27
    assert f(178, 1024, 1152, 256) == 2      # 16 stages: 2 x 8
    assert f(100, 2048, 640, 256) == 4 and f(100, 1024, 640, 256) == 2
    assert f(1000, 6912, 1152, 256) == 2     # 72 workgroups on 256 units: two half-K copies
    assert f(4096, 6912, 1152, 256) == 2     # 288 tiles on 512 workgroup slots (two per unit): two half-K copies fill them
    assert f(4096, 1024, 1152, 256) == 1     # the same tiles with a short K: a second start-up costs more than idle slots
    assert f(4096, 1152, 6912, 256) == 1     # 1728 tiles
    assert f(8192, 6912, 1152, 256) == 1     # 576 tiles: more than 3/4 of the slots
    assert f(4096, 1152, 1536, 256) == 1     # 384 tiles, but 36 k steps do not halve into whole groups of four
    try:                                     # the rule of the one-workgroup-per-unit kernels
        assert pkg.lib().tg_set_gemm_lds(0) == 0
        assert f(4096, 6912, 1152, 256) == 2     # 288 workgroups on 256 units: two half-K copies
        assert f(4096, 1152, 6912, 256) == 1     # 18 stages do not split into whole pairs per half
        assert f(8192, 6912, 1152, 256) == 1     # last round filled to 0.75
        assert f(1000, 6912, 1152, 256) == 2
    finally:
        assert pkg.lib().tg_set_gemm_lds(2) == 0


def test_bench_refuses_more_than_one_gpu():
    """This path runs on one GPU: `bench.py --gpus N` with N above 1 says so and exits (no GPU needed for that)."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr or "--gpus 1" in r.stderr, r.stderr[-500:]
    assert r.stdout.strip() == ""
