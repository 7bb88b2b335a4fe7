"""GPU: the C++20 host mirror (tiny-gemma_amd/host/tinygemma.hpp) driven like the reference's own
harness, compared with the CPU checker's greedy ids."""
import os
import subprocess

import numpy as np
import pytest

import golden_inputs as gi

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "host", "host_mirror_test")


def test_cpp_mirror_generates_the_reference_ids(tg, oracle, golden, weight_images, tmp_path):
    if not os.path.exists(EXE):
        pytest.fail("tests/host/host_mirror_test is not built: run __graft_entry__.build()")
    image = weight_images("270m", 6, 11)
    wpath, ppath = tmp_path / "w.bin", tmp_path / "prompt.i32"
    image.tofile(wpath)
    prompt = gi.prompt_ids(11, 70)
    prompt.tofile(ppath)
    env = dict(os.environ, LD_LIBRARY_PATH=os.path.join(ROOT, "tiny-gemma_amd") + ":" + os.environ.get("LD_LIBRARY_PATH", ""))
    r = subprocess.run([EXE, str(wpath), "6", str(ppath), "12"], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    ids = [int(l.split()[1]) for l in r.stdout.splitlines() if l.startswith("id ")]
    gids = [int(l.split()[1]) for l in r.stdout.splitlines() if l.startswith("gid ")]
    ref = golden["model/small6/tokens"].tolist()
    assert ids == ref and gids == ref
    assert "position 82" in r.stdout and "failures 0" in r.stdout
    sampled = [l.split()[1:] for l in r.stdout.splitlines() if l.startswith("sid ")]
    assert len(sampled) == 13 and all(a == b for a, b in sampled)      # stepwise minp_logits loop == generate_ids
    assert len({a for a, _ in sampled}) > 6                            # and it does sample
