"""The kernels that copy straight into LDS read their matrix operands with LDS instructions written as text (so that
the compiler does not serialise them with the copies) and wait for them with counted s_waitcnt; one of them also issues
its matrix instructions as text (to choose the register class of every accumulator), so the compiler inserts no
result-latency wait for those either.  In both cases the compiler takes a destination register to hold its value from
the instruction on, while the hardware fills it later.  Nothing may read or write such a register in between.

This test compiles the two source files to assembly (no GPU needed) and walks every kernel that uses the techniques,
along the control-flow graph: the function is cut into basic blocks at labels and branches, the set of results still in
flight is carried along every edge (at a join: the union, aligned at the newest entry), to a fixed point.
  * LDS: LDS instructions complete in order, every LDS and scalar-memory instruction counts towards lgkmcnt, and from
    a read to the wait that covers it no instruction may name its destination registers.  (A read hoisted above an
    if/else once made the compiler copy the not-yet-arrived "value" to another register in one branch; only the waves
    that ran second on their SIMD saw stale lanes.)
  * Matrix instructions written as text: an 8-pass matrix instruction needs 11 wait states before an ordinary
    instruction may name its destination; the test asks for 18, counting s_nop N as N + 1, another matrix instruction as
    4 and anything else as 1.
The kernels it covers are also held bit-equal to compiler-scheduled kernels on the GPU (tests/test_gpu_kernels.py)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tiny-gemma_amd", "csrc")
MFMA_WAIT_STATES = 18


def _regs(tok):
    """'v[4:7]' -> {('v', 4), ..}, 'a12' -> {('a', 12)}"""
    m = re.match(r"([va])\[(\d+):(\d+)\]$", tok)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.match(r"([va])(\d+)$", tok)
    return {(m.group(1), int(m.group(2)))} if m else set()


REG_TOKEN = re.compile(r"\b[va]\[\d+:\d+\]|\b[va]\d+\b")


def _blocks(func_text):
    """[(label or None, [(line number, instruction text)], [successor labels], falls_through)]"""
    blocks, cur, label = [], [], None
    for n, raw in enumerate(func_text.split("\n")):
        line = raw.split(";")[0].strip()
        if not line or line.startswith("."):
            if re.match(r"\.L\w+:$", line):
                blocks.append((label, cur, [], True))
                cur, label = [], line[:-1]
            continue
        if line.endswith(":"):
            if cur or label is not None:
                blocks.append((label, cur, [], True))
            cur, label = [], line[:-1]
            continue
        cur.append((n, line))
        op = line.split()[0]
        if op == "s_branch" or op.startswith("s_cbranch") or op == "s_endpgm" or op.startswith("s_setpc"):
            succ = [line.split()[-1]] if op != "s_endpgm" and not op.startswith("s_setpc") else []
            blocks.append((label, cur, succ, op.startswith("s_cbranch")))
            cur, label = [], None
    if cur or label is not None:
        blocks.append((label, cur, [], False))
    return blocks


def _merge(a, b):
    """Join of two in-flight states: (ordered LDS entries, {register: wait states still owed})."""
    la, lb = a[0], b[0]
    n = max(len(la), len(lb))
    pa, pb = [set()] * (n - len(la)) + la, [set()] * (n - len(lb)) + lb
    lds = [x | y for x, y in zip(pa, pb)]
    owed = dict(a[1])
    for r, w in b[1].items():
        owed[r] = max(owed.get(r, 0), w)
    return lds, owed


def _walk(block, state, out, name, check_mfma):
    lds, owed = [set(s) for s in state[0]], dict(state[1])
    for n, line in block:
        op = line.split()[0]
        toks = REG_TOKEN.findall(line)
        touched = set().union(*[_regs(t) for t in toks]) if toks else set()
        if op.startswith("s_waitcnt"):
            m = re.search(r"lgkmcnt\((\d+)\)", line)
            if m:
                del lds[:max(0, len(lds) - int(m.group(1)))]
        else:
            pending = set().union(*lds) if lds else set()
            if touched & pending and out is not None:
                out.add((name, n, line))
            is_mfma = op.startswith("v_mfma")
            if check_mfma and not is_mfma and touched & {r for r, w in owed.items() if w > 0} and out is not None:
                out.add((name, n, line))
            if op.startswith("ds_read"):
                lds.append(_regs(toks[0]))
            elif op.startswith("ds_") or op.startswith("s_load") or op.startswith("s_buffer_load"):
                lds.append(set())
            lds = lds[-32:]
        # wait states this instruction is worth to the matrix results before it
        m = re.match(r"s_nop\s+(\d+)", line)
        worth = int(m.group(1)) + 1 if m else (4 if op.startswith("v_mfma") else 1)
        owed = {r: w - worth for r, w in owed.items() if w - worth > 0}
        if check_mfma and op.startswith("v_mfma") and toks:
            for r in _regs(toks[0]):
                owed[r] = MFMA_WAIT_STATES
    return lds, owed


def violations(asm_text, kernel_substrings, check_mfma=False):
    """[(kernel, line number, instruction)] for instructions that name a register whose LDS read is still in flight or
    (check_mfma) whose matrix instruction has not had its wait states."""
    out = set()
    for func in re.split(r"\n(?=_Z[^\n]*:)", asm_text):
        name = func.split(":")[0]
        if not name.startswith("_Z") or not any(s in name for s in kernel_substrings):
            continue
        blocks = _blocks(func)
        index = {lab: i for i, (lab, _, _, _) in enumerate(blocks) if lab is not None}
        entry = [None] * len(blocks)
        entry[0] = ([], {})
        work = [0]
        rounds = 0
        while work:
            rounds += 1
            assert rounds < 200000, "the dataflow does not settle"
            i = work.pop()
            lab, body, succ, falls = blocks[i]
            lds, owed = _walk(body, entry[i], None, name, check_mfma)
            nxt = [index[s] for s in succ if s in index]
            if falls and i + 1 < len(blocks):
                nxt.append(i + 1)
            for j in nxt:
                merged = (lds, owed) if entry[j] is None else _merge(entry[j], (lds, owed))
                if entry[j] is None or merged != entry[j]:
                    entry[j] = merged
                    work.append(j)
        for i, (lab, body, succ, falls) in enumerate(blocks):
            if entry[i] is not None:
                _walk(body, entry[i], out, name, check_mfma)
    return sorted(out, key=lambda v: (v[0], v[1]))


def test_checker_sees_an_early_use():
    asm = "_Zk:\n\tds_read_b128 v[4:7], v1\n\tds_read_b128 v[8:11], v1 offset:16\n\ts_waitcnt lgkmcnt(1)\n\tv_add_f32 v0, v4, v5\n" \
          "\tv_mov_b32 v12, v9\n\ts_waitcnt lgkmcnt(0)\n\tv_mov_b32 v13, v9\n"
    assert violations(asm, ["k"]) == [("_Zk", 5, "v_mov_b32 v12, v9")]


def test_checker_follows_branches():
    """The wait sits in one arm of an if/else, the use behind the join: the other arm reaches it with the read in flight."""
    asm = ("_Zk:\n\tds_read_b128 v[4:7], v1\n\ts_cbranch_scc0 .LBB0_2\n\ts_waitcnt lgkmcnt(0)\n\tv_mov_b32 v20, v1\n\ts_branch .LBB0_3\n"
           ".LBB0_2:\n\tv_mov_b32 v21, v1\n.LBB0_3:\n\tv_add_f32 v0, v4, v5\n\ts_endpgm\n")
    assert [v[2] for v in violations(asm, ["k"])] == ["v_add_f32 v0, v4, v5"]
    # and around a loop's back edge: the read at the bottom of the body is still in flight at its top
    asm = ("_Zk:\n.LBB0_1:\n\tv_add_f32 v0, v4, v5\n\ts_waitcnt lgkmcnt(0)\n\tds_read_b128 v[4:7], v1\n\ts_cbranch_scc1 .LBB0_1\n\ts_endpgm\n")
    assert [v[2] for v in violations(asm, ["k"])] == ["v_add_f32 v0, v4, v5"]


def test_checker_counts_wait_states_behind_a_matrix_instruction():
    head = "_Zk:\n\tv_mfma_i32_32x32x32_i8 a[0:15], v[0:3], v[4:7], a[0:15]\n"
    assert [v[2] for v in violations(head + "\ts_nop 15\n\tv_accvgpr_read_b32 v9, a3\n", ["k"], check_mfma=True)] == ["v_accvgpr_read_b32 v9, a3"]
    assert violations(head + "\ts_nop 15\n\ts_nop 1\n\tv_accvgpr_read_b32 v9, a3\n", ["k"], check_mfma=True) == []
    # four more matrix instructions behind it are 16 wait states: not enough by this count
    more = "".join(f"\tv_mfma_i32_32x32x32_i8 a[{16 * i}:{16 * i + 15}], v[0:3], v[4:7], a[{16 * i}:{16 * i + 15}]\n" for i in range(1, 5))
    assert [v[2] for v in violations(head + more + "\tv_accvgpr_read_b32 v9, a3\n", ["k"], check_mfma=True)] == ["v_accvgpr_read_b32 v9, a3"]
    # another matrix instruction may accumulate into the same registers at once
    assert violations(head + head.split("\n", 1)[1] + "\ts_nop 15\n\ts_nop 15\n\tv_accvgpr_read_b32 v9, a3\n", ["k"], check_mfma=True) == []


def _compile(tmp_path, source):
    if shutil.which("hipcc") is None:
        pytest.skip("hipcc is not on PATH")
    import importlib.util
    spec = importlib.util.spec_from_file_location("tiny_gemma_amd_flags", os.path.join(ROOT, "tiny-gemma_amd", "__init__.py"))
    pkg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(pkg)
    flags = [f for f in pkg.HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    asm = tmp_path / (source + ".s")
    r = subprocess.run(["hipcc"] + flags + ["-S", "--cuda-device-only", os.path.join(CSRC, source), "-o", str(asm)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    return asm.read_text()


@pytest.mark.parametrize("source,kernels,mfma_as_text", [
    ("tg_attn_prefill.hip", ["attn_prefill_wide_kernel", "attn_prefill_planes_kernel"], False),
    ("tg_gemm_mfma.hip", ["gemm_i8_lds_kernel"], True),
])
def test_no_register_with_a_result_in_flight_is_touched(tmp_path, source, kernels, mfma_as_text):
    text = _compile(tmp_path, source)
    for k in kernels:
        assert k in text
    assert violations(text, kernels, check_mfma=mfma_as_text) == []
    if mfma_as_text:
        # the kernel must fit two waves per SIMD without spilling: the plain-store and the staged-table instantiations
        # use no scratch at all; the instantiation that reads a large GeLU table from memory may spill two dwords at the
        # loop exit, never inside the loop
        sizes = {}
        for m in re.finditer(r"\.amdhsa_kernel (\S*gemm_i8_lds_kernel\S*)\n(.*?)\.end_amdhsa_kernel", text, flags=re.S):
            pm = re.search(r"\.amdhsa_private_segment_fixed_size (\d+)", m.group(2))
            sizes[m.group(1)] = int(pm.group(1)) if pm else 0
        assert len(sizes) == 3, sizes
        for name, size in sizes.items():
            assert size <= (16 if "ILb1ELb0EE" in name else 0), (name, size)
