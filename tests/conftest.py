import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

import __graft_entry__ as ge  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def normrel(a, b):
    """||a - b||_2 / ||b||_2 in float64: the metric of the reference's own tests
    (csrc/include/test_utils.hpp:72-76)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


@pytest.fixture(scope="session")
def golden():
    path = os.path.join(ROOT, "tests", "golden", "golden.npz")
    return np.load(path)


@pytest.fixture(scope="session")
def orc():
    return ge.load_oracle()


@pytest.fixture(scope="session")
def oracle(orc):
    if not os.path.exists(orc.ORACLE_SO):
        orc.build(with_ref=False)
    return orc.Oracle()


@pytest.fixture(scope="session")
def tg():
    """The package, with the GPU initialised.  Fails loudly when the HIP library is not built."""
    mod = ge.load_package()
    mod.init(0)
    mod.lib().tg_set_taps(1)  # the model tests compare the residual stream block by block
    return mod


@pytest.fixture(scope="session")
def weight_images(oracle):
    """Weight-file images of the test models, generated once per session by the seeded generator."""
    import golden_inputs as gi
    cache = {}

    def get(shape, n_layers, seed):
        key = (shape, n_layers, seed)
        if key not in cache:
            cache[key] = oracle.generate_weights(gi.oracle_config(shape, n_layers), seed)
        return cache[key]

    return get
