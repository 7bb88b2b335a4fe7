#!/usr/bin/env python3
"""Decode benchmark of the int8 weight-only path on one MI355X.

A step is one greedy decode token (forward_decode + argmax) of a Gemma-3-1B-shaped model with
random-init weights, after a 178-token random prompt has been prefilled: the workload the
reference's README quotes its decode tok/s on (1024-token completions, mean prompt 178 tokens).
Weights, KV cache and the prompt are resident in HBM before the timed region; nothing crosses
PCIe inside it (each step feeds the device-side argmax of the previous one).

Prints one JSON line.  `value` is steps / wall time of the one timed region; `decode_step.blocks` gives the
same region cut into five blocks by HIP events (median and spread).  `roofline` is for the dominant kernel of a
step, the LM-head GEMV (tg_gemv_lmhead_argmax: 1152 x 262144 int8 + scales + x + logits = 304,091,648
algorithmic bytes per launch), timed with HIP events on the library's stream during real decode steps; its
`traffic` is a constant taken from the committed counter profile named beside it, not measured by this run.
`extra_rooflines` holds the same kind of statement for the decode attention launch and the prefill GEMM;
`launch_floor` the cost of a dependent launch and of a device-wide barrier on this machine, and the same decode
steps replayed from captured graphs.
Reported beside it: `gemv_lmhead_shape` (the plain GEMV entry point tg_qgemv_dev at the same shape,
launched back to back in rotation over three copies of the matrix so that none is served from cache), `gemv_640x2048` (the bare matvec of the first benchmark configuration, warm and
rotating over 512 MB of distinct copies) and `prefill.long_prompt` (a 4096-token prefill of the same
model: the matrix-matrix path on the int8 matrix cores).
`settle_ms` is the pause between the warm-up's synchronisation and the timed region (the host's first launches right
behind a long wait are slow), `host_pace` the time the host needs to issue 32 steps against the time the device needs to
run them, and `gemma3_270m` the 270m shape in the launch form the library chooses for it (a replayed graph whose
position-dependent nodes are updated every step) with the same steps as stream launches beside it.
`cpu_baseline` times the reference's single-threaded AVX2 path (oracle/_ref, built from the
reference's own sources) — or, where that library is absent, the scalar C restatement — on
this machine's host cores over a bounded sample of the same workload.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as ge  # noqa: E402

HBM_PEAK_GBS = 8000.0
INT8_PEAK_TOPS = 5000.0   # dense int8 matrix rate
# HBM bytes of one tg_gemv_lmhead_argmax launch from two `rocprofv3 --pmc` runs (FETCH_SIZE x 1.9999 +
# WRITE_SIZE x 1.0000, both in KiB, scaled on a 256 MiB copy kernel): profiles/decode_1B_hbm_traffic.md
LMHEAD_TRAFFIC_BYTES = {"1B": 304_496_732}

MODELS = {
    # name: (prompt tokens, decode bytes of weights+scales per token, LM-head GEMV algorithmic bytes)
    "1B": (178, 1_002_637_312, 304_091_648),
    "270m": (64, 269_588_480, 169_871_872),
}


class HipEvents:
    """hipEvent timing on a given stream through libamdhip64 (torch's events only see torch's stream)."""

    def __init__(self):
        self.hip = C.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [C.c_void_p]
        self.hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]

    def create(self):
        e = C.c_void_p()
        assert self.hip.hipEventCreate(C.byref(e)) == 0
        return e

    def record(self, e, stream):
        assert self.hip.hipEventRecord(e, stream) == 0

    def elapsed_ms(self, e0, e1):
        assert self.hip.hipEventSynchronize(e1) == 0
        ms = C.c_float()
        assert self.hip.hipEventElapsedTime(C.byref(ms), e0, e1) == 0
        return float(ms.value)


def host_cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(image_path, cfg_name, prompt, n_decode):
    """Decode tok/s of the CPU path on one core: prefill the same prompt, then n_decode greedy steps.
    The thread is pinned to the core it is running on for the duration of the sample."""
    orc = ge.load_oracle()
    old_affinity, pinned = None, None
    try:
        old_affinity = os.sched_getaffinity(0)
        cpu = None
        try:
            with open("/proc/self/stat") as f:
                cpu = int(f.read().rsplit(")", 1)[1].split()[36])   # field 39: processor last run on
        except (OSError, ValueError, IndexError):
            pass
        if cpu not in old_affinity:
            cpu = min(old_affinity)
        os.sched_setaffinity(0, {cpu})
        pinned = cpu
    except (AttributeError, OSError):
        pass
    try:
        out = _cpu_baseline_run(orc, image_path, cfg_name, prompt, n_decode)
    finally:
        if old_affinity is not None:
            try:
                os.sched_setaffinity(0, old_affinity)
            except OSError:
                pass
    out["pinned_to_cpu"] = pinned
    out["host_cpu_model"] = host_cpu_model()
    return out


def _cpu_baseline_run(orc, image_path, cfg_name, prompt, n_decode):
    cfg = orc.named_config(cfg_name)
    if orc.Ref.available():
        kind, sess_model = "reference", orc.Ref().model(cfg, image_path)
    else:
        kind, sess_model = "port", orc.Oracle().model(cfg, path=image_path)
    sess = sess_model.session()
    t0 = time.perf_counter()
    tok, _, _ = sess.prefill(prompt, want_logits=False)
    t1 = time.perf_counter()
    for _ in range(n_decode):
        tok, _, _ = sess.decode(tok, want_logits=False)
    t2 = time.perf_counter()
    return {
        "value": n_decode / (t2 - t1),
        "unit": "tok/s",
        "cores": 1,
        "kind": kind,
        "prefill_tok_s": len(prompt) / (t1 - t0),
        "prefill_tokens": len(prompt),
        "decode_steps": n_decode,
        "sample": f"{n_decode} greedy decode steps after the same {len(prompt)}-token prompt; prefill_tok_s = that prompt through "
                  f"forward_prefill alone on the same core (the reference's own figure also counts table and cache set-up, gemma.cpp:53-58)",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1024)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--stream-launches", action="store_true", help="plain stream launches for the decode steps, whatever the library would choose for the model")
    ap.add_argument("--model", default="1B", choices=sorted(MODELS))
    ap.add_argument("--seed", type=int, default=20251)
    ap.add_argument("--cpu-steps", type=int, default=128, help="decode steps of the CPU baseline sample (0 = skip)")
    ap.add_argument("--profile-steps", type=int, default=32)
    ap.add_argument("--long-prefill", type=int, default=4096,
                    help="tokens of the extra long-prompt prefill measurement, reported beside the headline (0 = skip)")
    ap.add_argument("--headline-only", action="store_true",
                    help="skip the extra measurements that launch the same kernels at other shapes (640x2048 matvec; 270m shape), "
                         "so that a profiler's per-kernel statistics describe the headline workload only")
    ap.add_argument("--graphs", action="store_true", help="replay captured HIP graphs instead of plain stream launches")
    ap.add_argument("--gemv-max-blocks", type=int, default=None, help="tuning knob: workgroups per GEMV launch (0 = one per tile)")
    ap.add_argument("--prefetch-blocks", type=int, default=None, help="tuning knob: weight-prefetch workgroups per launch")
    ap.add_argument("--prefetch-plan", type=int, default=None, help="tuning knob")
    ap.add_argument("--counter-run", nargs="?", const="decode", default=None, choices=["decode", "gemm"],
                    help="for rocprofv3 --pmc, no timing.  decode (default): prefill, a few decode steps and 4 launches of a "
                         "256 MiB copy kernel; gemm: 4 launches of the prefill GEMM at 4096 x 1152 x 6912 and nothing else")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is single-GPU (batch-1 decode has no data parallelism to spread); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    tg = ge.load_package()
    from tiny_gemma_amd import weights as tgw

    dev = tg.init(0)
    # the headline model's steps: stream launches unless --graphs; the library's own choice (-1) would be the same for the
    # 1B shape and updated-graph replay for the 270m shape (its section below runs both)
    if tg.lib().tg_set_graphs(1 if args.graphs else (0 if (args.model == "1B" or args.stream_launches) else -1)) != 0:
        print("bench.py: " + tg.lib().tg_last_error().decode(), file=sys.stderr)
        sys.exit(2)
    if args.prefetch_blocks is not None:
        tg.check(tg.lib().tg_set_prefetch_blocks(args.prefetch_blocks))
    if args.prefetch_plan is not None:
        tg.lib().tg_set_prefetch_plan(args.prefetch_plan)
    if args.gemv_max_blocks is not None:
        tg.lib().tg_set_gemv_max_blocks(args.gemv_max_blocks)
    n_prompt, step_bytes, lm_bytes = MODELS[args.model]
    cfg = tg.named_config(args.model)
    if args.counter_run == "gemm":
        gm, gk, gn = 4096, cfg.hidden_size, cfg.intermediate_size
        grng = np.random.default_rng(7)
        gw = tg.QWeight(grng.integers(-127, 128, (gk, gn), dtype=np.int8), grng.uniform(0.001, 0.02, gn).astype(np.float32))
        ga = tg.DeviceBuffer.from_numpy(grng.standard_normal((gm, gk)).astype(np.float32))
        gc = tg.DeviceBuffer(4 * gm * gn)
        for _ in range(4):
            gw.gemm(gc, ga, gm)
        tg.synchronize()
        print(json.dumps({"counter_run": "gemm", "shape": [gm, gk, gn], "launches": 4}))
        return
    if n_prompt + args.warmup + args.steps + args.profile_steps + 600 > cfg.n_pos:
        print("bench.py: steps exceed the model's context (n_pos)", file=sys.stderr)
        sys.exit(2)

    t0 = time.perf_counter()
    image = tgw.random_weight_image(cfg, args.seed)
    t_gen = time.perf_counter() - t0
    model = tg.Transformer(cfg)
    t0 = time.perf_counter()
    model.read_weights_mem(image)
    t_load = time.perf_counter() - t0
    sess = model.session()
    rng = np.random.default_rng(args.seed)
    prompt = rng.integers(0, cfg.n_vocab, n_prompt).astype(np.int32)

    # prefill (untimed part of the warm-up; reported separately).  The first call of a session also allocates
    # its prefill workspace; the second is the steady state.
    tg.synchronize()
    t0 = time.perf_counter()
    sess.prefill(prompt, want_logits=False)
    t_prefill_first = time.perf_counter() - t0
    sess.reset()
    tg.synchronize()
    t0 = time.perf_counter()
    sess.prefill(prompt, want_logits=False)
    t_prefill = time.perf_counter() - t0

    if args.counter_run:
        sess.decode_enqueue(min(args.steps, 8))
        n = 256 << 20
        a, b = tg.DeviceBuffer(n), tg.DeviceBuffer(n)
        for _ in range(4):
            tg.check(tg.lib().tg_dev_copy(b.p, a.p, n))
        tg.synchronize()
        print(json.dumps({"counter_run": True, "copy_bytes": n}))
        return

    ev = HipEvents()
    stream = tg.lib().tg_stream()
    e0, e1 = ev.create(), ev.create()
    sess.decode_enqueue(args.warmup)
    tg.synchronize()
    # The host gets 2 ms between the synchronisation and the timed region.  Launches issued right behind a wait of a few
    # milliseconds take the host 7.5 us each instead of 2.9 for about a millisecond (HIP runtime 7.2; a pause of 0.2 ms or
    # more, or a wait shorter than a millisecond, and they do not), the device, which needs 4.7 us per launch, then waits
    # for the host, and the first timed step takes 1.0 instead of 0.61 ms: 4 % of a 20-step region.  A serving loop
    # pays that once per batch of steps it synchronises on; `settle_ms` in the JSON names the pause.
    settle_ms = 2.0
    time.sleep(settle_ms * 1e-3)
    # ---- timed region: exactly `steps` decode steps, enqueued in five blocks with an event between blocks (an event
    # record does not wait for anything: the stream runs through) ----
    n_blocks = 5 if args.steps >= 5 else 1
    sizes = [args.steps // n_blocks + (1 if b < args.steps % n_blocks else 0) for b in range(n_blocks)]
    marks = [ev.create() for _ in range(n_blocks + 1)]
    t0 = time.perf_counter()
    ev.record(marks[0], stream)
    for b in range(n_blocks):
        sess.decode_enqueue(sizes[b])
        ev.record(marks[b + 1], stream)
    tg.synchronize()
    wall = time.perf_counter() - t0
    gpu_ms = ev.elapsed_ms(marks[0], marks[-1])
    block_order = [sizes[b] / (1e-3 * ev.elapsed_ms(marks[b], marks[b + 1])) for b in range(n_blocks)]
    block_tok_s = sorted(block_order)
    ids = sess.read_ids(1 + args.warmup + args.steps)
    assert ids.size == 1 + args.warmup + args.steps and ids.min() >= 0
    # The host's own pace: how long it takes to issue 32 further steps (4192 launches, which the queue takes without
    # making the host wait) against how long the device takes to run them.
    time.sleep(settle_ms * 1e-3)
    t0 = time.perf_counter()
    sess.decode_enqueue(32)
    host_32 = time.perf_counter() - t0
    tg.synchronize()
    dev_32 = time.perf_counter() - t0

    # ---- per-kernel-class event timing over further real decode steps ----
    ms_sum = (C.c_double * 7)()
    launches = (C.c_int * 7)()
    pos_profile = sess.position   # position of the first profiled step
    tg.check(tg.lib().tg_decode_profile(sess.h, args.profile_steps, ms_sum, launches))
    names = ["qkv", "attention", "oproj", "upgate_geglu", "down", "lmhead_argmax", "argmax_finish"]
    per_kernel_us = {n: 1e3 * ms_sum[i] / max(1, launches[i]) for i, n in enumerate(names)}
    lm_s = 1e-6 * per_kernel_us["lmhead_argmax"]
    achieved = lm_bytes / lm_s / 1e9
    # the same kernel re-launched 50x back to back on the session's buffers (dispatch latency amortised)
    L = tg.lib()
    tg.check(L.tg_debug_repeat_kernel(sess.h, 5, 0, 5))
    tg.synchronize()
    ev.record(e0, stream)
    tg.check(L.tg_debug_repeat_kernel(sess.h, 5, 0, 50))
    ev.record(e1, stream)
    tg.synchronize()
    lm_iso_us = ev.elapsed_ms(e0, e1) * 1e3 / 50

    # ---- the plain int8 GEMV entry point (launch_qgemv on device-resident operands) at the LM-head shape ----
    h, V = cfg.hidden_size, cfg.n_vocab
    tail = image[-(h * V + 4 * V):]
    # three copies, launched in rotation: 906 MB pass through the 256 MB memory-side cache between two launches
    # on one copy, so every launch streams from HBM (re-launched on ONE copy, part of the matrix is still cached)
    qws = [tg.QWeight(tail[:h * V].view(np.int8).reshape(h, V), tail[h * V:].view(np.float32)) for _ in range(3)]
    xd = tg.DeviceBuffer.from_numpy(rng.standard_normal(h).astype(np.float32))
    yd = tg.DeviceBuffer(4 * V)

    def time_plain(n_copies, iters=60):
        for k in range(6):
            qws[k % n_copies].gemv(yd, xd)
        tg.synchronize()
        ev.record(e0, stream)
        for k in range(iters):
            qws[k % n_copies].gemv(yd, xd)
        ev.record(e1, stream)
        tg.synchronize()
        return ev.elapsed_ms(e0, e1) * 1e3 / iters

    bare_us = time_plain(3)
    bare_same_us = time_plain(1)
    for qw in qws:
        qw.free()

    # ---- the bare matvec of the first benchmark configuration: 640 x 2048, warm (one matrix, re-launched) and cold
    # (rotating over distinct copies that together exceed the 256 MB memory-side cache twice over) ----
    ci, cn = 640, 2048
    c1_bytes = ci * cn + 4 * cn + 4 * ci + 4 * cn
    c1 = None
    if not args.headline_only:
        n_copies = (512 << 20) // (ci * cn) + 1
        crng = np.random.default_rng(101)
        Wc = crng.integers(-127, 128, (ci, cn), dtype=np.int8)
        sc = crng.uniform(0.001, 0.02, cn).astype(np.float32)
        copies = [tg.QWeight(Wc, sc) for _ in range(n_copies)]
        cx = tg.DeviceBuffer.from_numpy(crng.standard_normal(ci).astype(np.float32))
        cy = tg.DeviceBuffer(4 * cn)
        for q_ in copies[:8]:
            q_.gemv(cy, cx)
        tg.synchronize()
        ev.record(e0, stream)
        for _ in range(200):
            copies[0].gemv(cy, cx)
        ev.record(e1, stream)
        tg.synchronize()
        c1_warm_us = ev.elapsed_ms(e0, e1) * 1e3 / 200
        ev.record(e0, stream)
        for q_ in copies:
            q_.gemv(cy, cx)
        ev.record(e1, stream)
        tg.synchronize()
        c1_cold_us = ev.elapsed_ms(e0, e1) * 1e3 / n_copies
        for q_ in copies:
            q_.free()
        del copies
        c1 = {
            "entry": "tg_qgemv_dev",
            "algorithmic_bytes": c1_bytes,
            "warm_us_per_launch": c1_warm_us,
            "cold_us_per_launch": c1_cold_us,
            "cold_GBps": c1_bytes / c1_cold_us / 1e3,
            "timing": f"HIP events around 200 launches on one matrix (warm) and one launch on each of {n_copies} distinct copies "
                      f"({n_copies * ci * cn >> 20} MB, cold); 1.3 MB per launch is launch-latency bound on this machine",
        }

    # ---- the decode attention launch as a roofline statement: K and V rows of the valid keys, 2 KiB per key ----
    n_local = sum(1 for l in range(cfg.n_layers) if l % cfg.window_pattern != cfg.window_pattern - 1)
    n_global = cfg.n_layers - n_local
    keys = [n_local * min(p + 1, cfg.n_pos_local) + n_global * min(p + 1, cfg.n_pos) for p in range(pos_profile, pos_profile + args.profile_steps)]
    attn_bytes = 2 * 4 * cfg.head_dim * (sum(keys) / len(keys)) / cfg.n_layers
    attn_us = per_kernel_us["attention"]
    extra_rooflines = {
        "attention_decode": {
            "kernel": "attn_decode_kernel", "bound": "hbm", "unit": "GB/s", "peak": HBM_PEAK_GBS,
            "algorithmic_bytes_per_launch": attn_bytes, "avg_launch_us": attn_us, "achieved": attn_bytes / attn_us / 1e3,
            "frac": attn_bytes / attn_us / 1e3 / HBM_PEAK_GBS,
            "note": f"average over {n_local} local layers (ring of {cfg.n_pos_local} keys) and {n_global} global layers at positions "
                    f"{pos_profile}..{pos_profile + args.profile_steps - 1}; 2*4*head_dim bytes per valid key; a launch over a few hundred "
                    "keys is bound by its dependent steps (latency), not by bytes",
        }
    }

    # ---- the prefill GEMM as a roofline statement: the up-projection-shaped product of a 4096-token prompt ----
    if not args.headline_only and args.model == "1B":
        gm, gk, gn = 4096, cfg.hidden_size, cfg.intermediate_size
        grng = np.random.default_rng(7)
        gw = tg.QWeight(grng.integers(-127, 128, (gk, gn), dtype=np.int8), grng.uniform(0.001, 0.02, gn).astype(np.float32))
        ga = tg.DeviceBuffer.from_numpy(grng.standard_normal((gm, gk)).astype(np.float32))
        gc = tg.DeviceBuffer(4 * gm * gn)
        for _ in range(3):
            gw.gemm(gc, ga, gm)
        tg.synchronize()
        ev.record(e0, stream)
        for _ in range(20):
            gw.gemm(gc, ga, gm)
        ev.record(e1, stream)
        tg.synchronize()
        g_us = ev.elapsed_ms(e0, e1) * 1e3 / 20
        g_flops = 2.0 * gm * gk * gn
        extra_rooflines["prefill_gemm"] = {
            "kernel": "gemm_i8_lds_kernel (+ row_scale_kernel, quant_pack_kernel)", "bound": "mfma", "unit": "TFLOP/s", "peak": INT8_PEAK_TOPS,
            "shape": [gm, gk, gn], "algorithmic_flops_per_launch": g_flops, "avg_launch_us": g_us,
            "achieved": g_flops / g_us / 1e6, "frac": g_flops / g_us / 1e6 / INT8_PEAK_TOPS,
            "note": "tg_qgemm_dev, 20 back-to-back launches incl. the quantising pre-pass; algorithmic 2*M*K*N flops against the dense int8 "
                    "rate; the matrix cores execute 3x that (three int8 digit planes of the activations)",
        }
        # the shader clock the part held inside the matrix kernel itself (every workgroup reports its own clocks): random
        # operands as above, and all-zero activations, for which the power limit leaves the clock higher
        gz = tg.DeviceBuffer.from_numpy(np.zeros((gm, gk), np.float32))
        clocks = {}
        for label, abuf in (("random_operands", ga), ("zero_activations", gz)):
            for _ in range(3):
                gw.gemm(gc, abuf, gm)
            mhz, wg_us, nwg = gw.gemm_clock(gc, abuf, gm)
            tg.synchronize()
            ev.record(e0, stream)
            for _ in range(10):
                gw.gemm(gc, abuf, gm)
            ev.record(e1, stream)
            tg.synchronize()
            clocks[label] = {"shader_clock_mhz": mhz, "workgroup_lifetime_us": wg_us, "workgroups": nwg,
                             "entry_point_us": ev.elapsed_ms(e0, e1) * 1e3 / 10}
        extra_rooflines["prefill_gemm"]["clock_inside_the_kernel"] = clocks
        gz.free()
        gw.free()
        del ga, gc, gz
        # what the integer matrix cores sustain when every compute unit issues nothing else (register operands, no
        # memory traffic): 32 clocks per instruction always, but the clock the part holds depends on the operand values
        cpm, mhz = C.c_double(), C.c_double()
        ceiling = {}
        for label, operands in (("zero", 0), ("int8_in_pm6", 2), ("uniform_int8", 1)):
            tg.check(L.tg_debug_mfma_clock(256, 20000, operands, C.byref(cpm), C.byref(mhz)))
            ceiling[label] = {"clocks_per_mfma": cpm.value, "clock_mhz": mhz.value,
                              "TOPs": 1024 * 65536.0 / cpm.value * mhz.value / 1e6}
        tg.check(L.tg_debug_mfma_clock(8, 20000, 1, C.byref(cpm), C.byref(mhz)))
        ceiling["uniform_int8_8_workgroups_only"] = {"clocks_per_mfma": cpm.value, "clock_mhz": mhz.value}
        pg = extra_rooflines["prefill_gemm"]
        pg["mfma_ceiling"] = ceiling
        pg["executed_TOPs"] = 3.0 * pg["achieved"]
        pg["frac_of_sustained_int8_rate"] = 3.0 * pg["achieved"] / ceiling["uniform_int8"]["TOPs"]
        pg["mfma_ceiling_note"] = ("tg_debug_mfma_clock: 256 workgroups x 4 waves issuing only v_mfma_i32_32x32x32_i8 on register operands; "
                                   "TOPs = 1024 SIMDs x 65536 ops / clocks_per_mfma x clock.  With every compute unit busy the part lowers its "
                                   "clock under the power limit, more so the more operand bits toggle: the nominal 5.0 POP/s needs 2.4 GHz, "
                                   "which it only holds for all-zero operands or a mostly idle chip.  frac_of_sustained_int8_rate = executed "
                                   "(3 x algorithmic) rate / the uniform_int8 figure")

        # what a compute unit pulls through its vector L1 (one workgroup of 4 waves per unit): from its XCD's L2, and
        # from memory with every unit streaming a share of its own
        a, b, c3 = C.c_double(), C.c_double(), C.c_double()
        fill = {}
        for label, wgs, kib, disjoint, steps in (("l2_256wg", 256, 1024, 0, 256), ("l2_512wg", 512, 1024, 0, 256), ("l2_1024wg", 1024, 1024, 0, 256),
                                                  ("memory_256wg", 256, 1 << 20, 1, 126), ("memory_1024wg", 1024, 1 << 20, 1, 30)):
            tg.check(L.tg_debug_l1_fill(wgs, 8, steps, kib, disjoint, C.byref(a), C.byref(b), C.byref(c3)))
            fill[label] = {"GBps_per_workgroup": a.value, "TBps_all": b.value / 1e3, "clock_mhz": c3.value}
        pg["l1_fill"] = fill
        pg["l1_fill_note"] = ("tg_debug_l1_fill: workgroups of 256 threads stream 16-byte loads, 8 x 4 KiB per step, two steps in flight; l2 = all walk "
                              "one megabyte (L2 hits, never L1 hits), memory = every workgroup streams its own share of a gigabyte")

    # ---- what a dependent launch and a device-wide barrier cost here; the same steps replayed from captured graphs ----
    launch_floor = None
    if not args.headline_only:
        us = C.c_double()
        flag = C.c_int32()
        launch_floor = {}
        for wgs in (256, 512):
            tg.check(L.tg_debug_launch_chain(2000, wgs, C.byref(us)))
            launch_floor[f"dependent_launch_us_{wgs}wg"] = us.value
        for wgs in (256, 64):
            for fenced in (1, 0):
                tg.check(L.tg_debug_grid_barrier(400, wgs, fenced, 1 << 16, C.byref(us), C.byref(flag)))
                launch_floor[f"grid_barrier_us_{wgs}wg_{'fences' if fenced else 'atomic_data'}"] = None if flag.value else us.value
        launch_floor["note"] = ("dependent_launch: 2000 back-to-back launches of a kernel that reads what the previous one wrote; grid_barrier: one "
                                "resident kernel, per round 64 B published per workgroup + device-wide barrier + 64 B read from a workgroup on "
                                "another XCD; fences = ordinary stores/loads + device-scope fences, atomic_data = the data moves through "
                                "device-scope atomic accesses; null = a bounded wait gave up")
        # the hand-over between resident workgroups, sharded over the 8 XCDs (tg_debug_handover): per round every workgroup
        # publishes words_per_wg floats, all hand over, every workgroup reads and checks all of them
        to, wrong = C.c_int32(), C.c_int32()
        handover = {}
        for label, bar, data in (("one_counter", 0, 0), ("tree_per_xcd", 1, 1), ("eight_counters_summed", 3, 1), ("flag_array", 4, 1),
                                 ("pairs_value_round_in_data", 0, 3), ("sentinel_in_data", 0, 4)):
            for wgs, wpw in ((64, 6), (256, 6), (256, 27)):
                tg.check(L.tg_debug_handover(400, wgs, bar, data, wpw, 1 << 16, C.byref(us), C.byref(to), C.byref(wrong), None))
                handover[f"{label}_us_{wgs}wg_{wgs * wpw}floats"] = None if (to.value or wrong.value) else us.value
        launch_floor["handover"] = handover
        launch_floor["handover_note"] = ("one resident kernel; a round = write-through stores of the data, hand-over, every workgroup reads all of it and "
                                         "checks the sum; one_counter: every workgroup adds to and polls one word; tree_per_xcd: counter per XCD -> "
                                         "8-way counter -> release flag per XCD; eight_counters_summed: counter per XCD, every workgroup polls all 8 "
                                         "(what the one-kernel decode step uses); flag_array: a word per workgroup; *_in_data: no barrier, the consumer "
                                         "polls the data itself; null = a wait gave up or a sum was wrong")
        # the one-kernel decode step (all layers in one launch of resident workgroups) against one launch per projection:
        # same bits, tested; 256 steps each on the same session
        fused = {}
        for mode in (1, 0):
            L.tg_set_fused_decode(mode, 0, 0)
            sess.decode_enqueue(8)
            tg.synchronize()
            ev.record(e0, stream)
            sess.decode_enqueue(256)
            ev.record(e1, stream)
            tg.synchronize()
            sess.read_ids(1)  # reports a wait that gave up
            fused["one_kernel_step_tok_s" if mode else "launch_per_projection_tok_s"] = 256 / (1e-3 * ev.elapsed_ms(e0, e1))
        if L.tg_set_fused_decode(1, 0, 0) == 0:
            ts = np.zeros((cfg.n_layers, 24), np.uint64)
            if L.tg_debug_fused_timestamps(sess.h, ts.ctypes.data_as(C.c_void_p), cfg.n_layers) == 0:
                t = ts.astype(np.int64)[1:-1]
                names = ("norms_qkv", "qkv_tiles", "arrive_qkv", "wait_attention", "merge", "o_tiles", "arrive_o", "wait_o", "norms_upgate",
                         "upgate_tiles", "arrive_h", "wait_h", "down_tiles", "arrive_d", "wait_d")
                fused["layer_timeline_us"] = {n: float((t[:, i + 1] - t[:, i]).mean() / 100.0) for i, n in enumerate(names)}
                fused["layer_us"] = float((t[:, 15] - t[:, 0]).mean() / 100.0)
                fused["attention_workgroup_us"] = {"sees_qkv_after_gemv_wg0_arrived": float((t[:, 16] - t[:, 3]).mean() / 100.0),
                                                   "body": float((t[:, 17] - t[:, 16]).mean() / 100.0),
                                                   "arrive": float((t[:, 18] - t[:, 17]).mean() / 100.0),
                                                   "gemv_wg0_sees_it_after": float((t[:, 4] - t[:, 18]).mean() / 100.0)}
            L.tg_set_fused_decode(0, 0, 0)
        launch_floor["one_kernel_step"] = fused
        if not args.graphs and L.tg_set_graphs(1) == 0:
            rates = {}
            for mode in (1, 0):
                L.tg_set_graphs(mode)
                sess.decode_enqueue(8)
                tg.synchronize()
                ev.record(e0, stream)
                sess.decode_enqueue(256)
                ev.record(e1, stream)
                tg.synchronize()
                rates["graph_replay_tok_s" if mode else "stream_tok_s"] = 256 / (1e-3 * ev.elapsed_ms(e0, e1))
            launch_floor.update(rates)

    # ---- long-prompt prefill (the matrix-matrix path) on a fresh session ----
    long_prefill = None
    if args.long_prefill > 0:
        s2 = model.session()
        lp = rng.integers(0, cfg.n_vocab, args.long_prefill).astype(np.int32)
        s2.prefill(lp, want_logits=False)
        s2.reset()
        tg.synchronize()
        t0 = time.perf_counter()
        s2.prefill(lp, want_logits=False)
        dt = time.perf_counter() - t0
        long_prefill = {"tokens": args.long_prefill, "ms": 1e3 * dt, "tok_s": args.long_prefill / dt}
        del s2

    # ---- the 270m shape, reported beside the headline: 64-token prompt + 256 greedy steps, and a 16384-token
    # prefill + 256 greedy steps at that context.  Its layer weights (100 MB) fit the 256 MB memory-side cache. ----
    small = None
    if args.model == "1B" and not args.headline_only:
        del sess, model
        scfg = tg.named_config("270m")
        simg = tgw.random_weight_image(scfg, args.seed + 1)
        smodel = tg.Transformer(scfg)
        smodel.read_weights_mem(simg)
        spath = None
        if args.cpu_steps > 0:  # the CPU baseline of this shape reads the same weight file
            spath = f"/tmp/tg_bench_270m_{args.seed + 1}.bin"
            simg.tofile(spath)
        del simg
        ss = smodel.session()
        s_bytes = MODELS["270m"][1]

        sprompt = rng.integers(0, scfg.n_vocab, 64).astype(np.int32)

        def run(n_prompt_s, n_steps):
            ids = sprompt if n_prompt_s == sprompt.size else rng.integers(0, scfg.n_vocab, n_prompt_s).astype(np.int32)
            ss.reset()
            ss.prefill(ids, want_logits=False)  # allocates the workspace for this length
            ss.reset()
            tg.synchronize()
            t0 = time.perf_counter()
            ss.prefill(ids, want_logits=False)
            tp = time.perf_counter() - t0
            ss.decode_enqueue(16)
            tg.synchronize()
            time.sleep(settle_ms * 1e-3)
            t0 = time.perf_counter()
            ss.decode_enqueue(n_steps)
            te = time.perf_counter() - t0
            tg.synchronize()
            td = time.perf_counter() - t0
            # host_enqueue_ms_per_step next to ms_per_step tells which side set the pace: this shape's step is 91 launches
            # of 3.6 us on the device, and the host issues a launch in 2.5 us or in 4.2 us depending on the core the
            # thread happens to run on and on what else that core is doing (2,600 or 3,070 tok/s)
            return {"prompt_tokens": n_prompt_s, "prefill_ms": 1e3 * tp, "prefill_tok_s": n_prompt_s / tp, "decode_steps": n_steps,
                    "decode_tok_s": n_steps / td, "ms_per_step": 1e3 * td / n_steps, "host_enqueue_ms_per_step": 1e3 * te / n_steps}

        # The library's own choice for this shape (tg_set_graphs(-1)): replay of a captured step whose position-dependent
        # nodes are updated before every replay, one graph launch and 36 node updates per step on the host instead of 91
        # kernel launches.  Beside it the same 256 steps as stream launches, which follow the host wherever the launching
        # thread sits on a slow core (`host_enqueue_ms_per_step` = `ms_per_step`).
        L.tg_set_graphs(-1)
        short, long_ctx = run(64, 256), run(16384, 256)
        short["launch"] = long_ctx["launch"] = "updated hipGraph replay (library default for this shape)"
        L.tg_set_graphs(0)
        short["stream_launches"] = {k: v for k, v in run(64, 256).items() if k in ("decode_tok_s", "ms_per_step", "host_enqueue_ms_per_step")}
        short["weight_stream_GBps"] = s_bytes * short["decode_tok_s"] / 1e9
        short["frac_of_hbm_roofline"] = short["weight_stream_GBps"] / HBM_PEAK_GBS
        small = {"shape": "gemma-3-270m", "weight_bytes_per_token": s_bytes, "prompt64_decode256": short,
                 "prompt16384_decode256": long_ctx}
        del ss, smodel
        if spath is not None:
            try:
                small["cpu_baseline"] = cpu_baseline(spath, "270m", sprompt, 256)
                small["cpu_baseline"]["host_cpus"] = os.cpu_count()
            finally:
                os.remove(spath)

    tok_s = args.steps / wall
    out = {
        "metric": "decode_tokens_per_s",
        "value": tok_s,
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms": settle_ms,
        "host_pace": {"steps": 32, "host_enqueue_ms_per_step": 1e3 * host_32 / 32, "ms_per_step": 1e3 * dev_32 / 32,
                      "note": "32 further steps after the timed region: time until the host had issued them / until the device had run them"},
        "ms_per_step": 1e3 * wall / args.steps,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"gemma-3-{args.model} shape, int8 weight-only, random-init N(0,0.02); {n_prompt}-token random prompt "
                        f"prefilled, then greedy decode, batch 1, GeLU LUT(-4,4,1024)",
            "prompt_tokens": n_prompt,
            "decode_position_start": n_prompt + args.warmup,
            "seed": args.seed,
            "launch": "hipGraph replay" if args.graphs else ("stream" if (args.model == "1B" or args.stream_launches) else "library default (updated hipGraph replay; stream launches under a profiler)"),
        },
        "roofline": {
            "kernel": "tg_gemv_lmhead_argmax",
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": LMHEAD_TRAFFIC_BYTES.get(args.model),
            "traffic_source": "constant from profiles/decode_1B_hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, scaled on a "
                              "256 MiB copy kernel); not measured by this run",
            "algorithmic_bytes_per_launch": lm_bytes,
            "avg_launch_us": per_kernel_us["lmhead_argmax"],
            "timing": "HIP events around every launch of the kernel inside real decode steps (includes dispatch latency)",
            "back_to_back_note": "the same launch repeated 50x on the session's one matrix: part of it is served by the memory-side cache",
            "back_to_back_us": lm_iso_us,
            "back_to_back_GBps": lm_bytes / lm_iso_us / 1e3,
        },
        "gemv_lmhead_shape": {
            "entry": "tg_qgemv_dev",
            "shape": [h, V],
            "avg_launch_us": bare_us,
            "GBps": lm_bytes / bare_us / 1e3,
            "frac": lm_bytes / bare_us / 1e3 / HBM_PEAK_GBS,
            "same_matrix_us": bare_same_us,
            "same_matrix_GBps": lm_bytes / bare_same_us / 1e3,
            "timing": "HIP events around 60 back-to-back launches of the plain GEMV (no norm prologue, no argmax epilogue) "
                      "rotating over 3 copies of the matrix, so that every launch streams from HBM; same_matrix = re-launched on "
                      "one copy, part of which the 256 MB memory-side cache still holds",
        },
        "gemv_640x2048": c1,
        "extra_rooflines": extra_rooflines,
        "launch_floor": launch_floor,
        "decode_step": {
            "gpu_ms_per_step_events": gpu_ms / args.steps,
            "blocks": {"n": n_blocks, "tok_s_median": block_tok_s[len(block_tok_s) // 2], "tok_s_min": block_tok_s[0],
                       "tok_s_max": block_tok_s[-1], "tok_s_in_order": block_order,
                       "timing": "HIP events between the blocks of the timed region"},
            "weight_bytes_per_token": step_bytes,
            "weight_stream_GBps": step_bytes * tok_s / 1e9,
            "frac_of_hbm_roofline": step_bytes * tok_s / 1e9 / HBM_PEAK_GBS,
            "avg_kernel_us": per_kernel_us,
        },
        "prefill": {"tokens": n_prompt, "tok_s_forward_only": n_prompt / t_prefill, "ms": 1e3 * t_prefill,
                    "first_call_ms": 1e3 * t_prefill_first, "long_prompt": long_prefill},
        "gemma3_270m": small,
        "setup_s": {"generate_weights": t_gen, "upload_and_retile": t_load},
        "device": dev,
    }
    if args.cpu_steps > 0:
        path = f"/tmp/tg_bench_{args.model}_{args.seed}.bin"
        image.tofile(path)
        try:
            out["cpu_baseline"] = cpu_baseline(path, args.model, prompt, args.cpu_steps)
            out["cpu_baseline"]["host_cpus"] = os.cpu_count()
        finally:
            os.remove(path)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
