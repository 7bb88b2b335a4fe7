"""The kernels that copy straight into LDS read their matrix operands with LDS instructions written as text (so that
the compiler does not serialise them with the copies) and wait for them with counted s_waitcnt.  The compiler takes
the destination register of such a read to hold the value from the instruction on; the hardware fills it when the LDS
answers.  Nothing may read or write that register in between.  This test compiles the two source files to assembly
(no GPU needed) and walks every kernel that uses the technique: LDS instructions complete in order, every LDS
and scalar-memory instruction counts towards lgkmcnt, and from a read to the wait that covers it no instruction may
name its destination registers.  (A read hoisted above an if/else once made the compiler copy the not-yet-arrived
"value" to another register in one branch; only the waves that ran second on their SIMD saw stale lanes.)"""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tiny-gemma_amd", "csrc")


def _regs(tok):
    m = re.match(r"v\[(\d+):(\d+)\]$", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def violations(asm_text, kernel_substrings):
    """[(kernel, line number, instruction)] for instructions that touch a register with an LDS read in flight.
    Straight-line approximation: labels are fallen through, branches are not followed."""
    out = []
    for func in re.split(r"\n(?=_Z[^\n]*:)", asm_text):
        name = func.split(":")[0]
        if not name.startswith("_Z") or not any(s in name for s in kernel_substrings):
            continue
        in_flight = []  # destination registers of the outstanding lgkm instructions, oldest first
        for n, line in enumerate(func.split("\n")):
            line = line.split(";")[0].strip()
            if not line or line.startswith(".") or line.endswith(":"):
                continue
            op = line.split()[0]
            toks = re.findall(r"v\[\d+:\d+\]|v\d+", line)
            touched = set().union(*[_regs(t) for t in toks]) if toks else set()
            if op.startswith("s_waitcnt"):
                m = re.search(r"lgkmcnt\((\d+)\)", line)
                if m:
                    del in_flight[:max(0, len(in_flight) - int(m.group(1)))]
                continue
            pending = set().union(*in_flight) if in_flight else set()
            if touched & pending:
                out.append((name, n, line))
            if op.startswith("ds_read"):
                in_flight.append(_regs(toks[0]))
            elif op.startswith("ds_") or op.startswith("s_load") or op.startswith("s_buffer_load"):
                in_flight.append(set())
    return out


def test_checker_sees_an_early_use():
    asm = "_Zk:\n\tds_read_b128 v[4:7], v1\n\tds_read_b128 v[8:11], v1 offset:16\n\ts_waitcnt lgkmcnt(1)\n\tv_add_f32 v0, v4, v5\n" \
          "\tv_mov_b32 v12, v9\n\ts_waitcnt lgkmcnt(0)\n\tv_mov_b32 v13, v9\n"
    assert violations(asm, ["k"]) == [("_Zk", 5, "v_mov_b32 v12, v9")]


@pytest.mark.parametrize("source,kernels", [
    ("tg_attn_prefill.hip", ["attn_prefill_wide_kernel", "attn_prefill_planes_kernel"]),
    ("tg_gemm_mfma.hip", ["gemm_i8_lds_kernel"]),
])
def test_no_register_of_an_lds_read_in_flight_is_touched(tmp_path, source, kernels):
    import importlib.util
    spec = importlib.util.spec_from_file_location("tiny_gemma_amd_flags", os.path.join(ROOT, "tiny-gemma_amd", "__init__.py"))
    pkg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(pkg)
    flags = [f for f in pkg.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    asm = tmp_path / (source + ".s")
    r = subprocess.run(["hipcc"] + flags + ["-S", "--cuda-device-only", os.path.join(CSRC, source), "-o", str(asm)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    text = asm.read_text()
    for k in kernels:
        assert k in text
    assert violations(text, kernels) == []
