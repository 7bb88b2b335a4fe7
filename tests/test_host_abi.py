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


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tinygemma_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tg_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(pkg):
    lib = C.CDLL(pkg.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 30
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


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
