#!/usr/bin/env python3
"""Benchmark of the MI355X transformer-op backend.

    python bench.py --gpus 1 --steps K --warmup W [--cases LIST] [--no-cpu]

Prints ONE JSON line. The headline `value` is the row-op throughput on the configured fp32
[8192, 4096] tensors (seed 1): one step = last-dim softmax + LayerNorm + RMSNorm + erf-GELU +
bias+residual add, each reading its inputs from HBM and writing its output once; value =
algorithmic bytes of the step / wall time, with every input already resident in HBM. The same line
carries `roofline` (dominant kernel of the step, HIP-event timed), `cpu_baseline` (the CPU checker
restating ft-kernel-cpu, timed on this host's cores), and `cases`: the other parts of the metric --
fp32 / fp64 GEMM TFLOP/s, causal SDPA TFLOP/s, pre-LN block and GPT-2-shaped forward tokens/s --
each with its own roofline fraction.

Everything runs on one GPU. `--gpus N` with N > 1 exits: this backend has no multi-GPU path.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
FP32_MFMA_PEAK_TF = 157.3    # dense fp32 matrix
FP64_MFMA_PEAK_TF = 78.6     # dense fp64 matrix

ROWS, COLS = 8192, 4096
ELEM = ROWS * COLS
# Algorithmic bytes per launch: every input read once + the output written once.
ROW_BYTES = {
    "softmax": 2 * ELEM * 4,
    "layer_norm": 2 * ELEM * 4 + 2 * COLS * 4,
    "rms_norm": 2 * ELEM * 4 + COLS * 4,
    "gelu": 2 * ELEM * 4,
    "bias_residual_add": 3 * ELEM * 4 + COLS * 4,
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


WARM_SECONDS = 0.05  # untimed launches before each timed region: the GPU's clocks take tens of ms of load to settle


def event_time_ms(device, launch, iters, warm_s=WARM_SECONDS):
    """Average duration of `launch` over `iters` back-to-back launches, by HIP events recorded on
    the stream the kernels run on (the library stream), after `warm_s` of untimed launches of the same call."""
    t_end = time.perf_counter() + warm_s
    while time.perf_counter() < t_end:
        for _ in range(4):
            launch()
        device.synchronize()
    e0, e1 = device.Event(), device.Event()
    e0.record()
    for _ in range(iters):
        launch()
    e1.record()
    e1.synchronize()
    return e0.elapsed_ms(e1) / iters


# HBM bytes per launch at fp32 [8192,4096], from two rocprofv3 --pmc runs of this file (FETCH_SIZE, then WRITE_SIZE) over the
# rotating buffer sets, each scaled by what the same counter reads for the GELU kernel, a plain copy of 2 x 128 MiB (factors
# 0.5001 and 1.0000).
# Counters cannot be read from inside the process, so these are the figures of the committed profile summary.
MEASURED_HBM_TRAFFIC = {"softmax": 268474075, "layer_norm": 268741296, "rms_norm": 268584590, "gelu": 268435456,
                        "bias_residual_add": 402771071}


ROTATE_SETS = 10  # distinct input / output buffer sets: 9 x 256 MiB (or more) are touched between two uses of one buffer


def bench_rowops(device, synth, steps, warmup, with_cpu):
    """Row ops at fp32 [8192, 4096]. The part has a 256 MB last-level cache and a 128 MiB input relaunched on the same address
    could be served from it, so every launch of the timed loops takes the next of ROTATE_SETS buffer sets (identical contents,
    distinct addresses). The same-buffer timing is reported beside it."""
    from frankentorch_amd.device import DeviceBuffer

    log("[rowops] generating fp32 [%d, %d] inputs (seed 1), %d buffer sets" % (ROWS, COLS, ROTATE_SETS))
    x = synth.normal(1, "x", (ROWS, COLS))
    gamma = synth.uniform(1, "gamma", (COLS,), 0.5, 1.5)
    beta = synth.normal(1, "beta", (COLS,), 0.0, 0.1)
    bias = synth.normal(1, "bias", (COLS,), 0.0, 0.1)
    res = synth.normal(1, "residual", (ROWS, COLS))
    dg, dbt, dbi = (DeviceBuffer.from_host(a) for a in (gamma, beta, bias))
    xs = [DeviceBuffer.from_host(x) for _ in range(ROTATE_SETS)]
    rs = [DeviceBuffer.from_host(res) for _ in range(ROTATE_SETS)]
    ys = [DeviceBuffer((ROWS, COLS)) for _ in range(ROTATE_SETS)]
    calls = {
        "softmax": lambda i: device.softmax_lastdim(xs[i], ys[i], ROWS, COLS),
        "layer_norm": lambda i: device.layer_norm(xs[i], dg, dbt, ys[i], ROWS, COLS, 1e-5),
        "rms_norm": lambda i: device.rms_norm(xs[i], dg, ys[i], ROWS, COLS, 1e-6),
        "gelu": lambda i: device.gelu(xs[i], ys[i], ELEM),
        "bias_residual_add": lambda i: device.bias_residual_add(xs[i], dbi, rs[i], ys[i], ROWS, COLS),
    }
    turn = [0]

    def rotating(call):
        def fn():
            turn[0] = (turn[0] + 1) % ROTATE_SETS
            call(turn[0])
        return fn

    launches = {k: rotating(c) for k, c in calls.items()}
    # The ceiling of a read-once / write-once kernel at this shape, measured in the same run on the same rotating sets:
    # the library's plain 128-bit streaming copy (128 MiB in, 128 MiB out). Not part of the step.
    copy_launch = rotating(lambda i: device.copy(xs[i], ys[i], ELEM))

    def step():
        for fn in launches.values():
            fn()

    # Untimed warm-up: the W steps asked for, and then more of the same step until WARM_SECONDS of load have passed (what
    # every per-kernel figure below gets too): at 0.25 ms a step, five warm-up steps end before the clocks have settled
    # and the timed steps read 4-5 % low.
    for _ in range(warmup):
        step()
    device.synchronize()
    t_end = time.perf_counter() + WARM_SECONDS
    while time.perf_counter() < t_end:
        for _ in range(8):
            step()
        device.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    device.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / steps
    step_bytes = sum(ROW_BYTES.values())
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    per_kernel = {}
    for name, fn in launches.items():
        fn()
        device.synchronize()
        ms = event_time_ms(device, fn, max(20, steps))
        ms_same = event_time_ms(device, lambda: calls[name](0), max(20, steps))
        gbs = ROW_BYTES[name] / (ms * 1e-3) / 1e9
        gbs_same = ROW_BYTES[name] / (ms_same * 1e-3) / 1e9
        per_kernel[name] = {"ms": round(ms, 5), "GB/s": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4),
                            "bytes": ROW_BYTES[name],
                            "same_buffer": {"ms": round(ms_same, 5), "GB/s": round(gbs_same, 1), "frac": round(gbs_same / HBM_PEAK_GBS, 4)}}
        log("[rowops] %-18s %.4f ms  %7.1f GB/s  %.1f%% of HBM peak over %d rotating buffer sets (same buffer: %.4f ms, %.1f%%)"
            % (name, ms, gbs, 100 * gbs / HBM_PEAK_GBS, ROTATE_SETS, ms_same, 100 * gbs_same / HBM_PEAK_GBS))
    copy_launch()
    device.synchronize()
    ms_copy = event_time_ms(device, copy_launch, max(20, steps))
    ms_copy_same = event_time_ms(device, lambda: device.copy(xs[0], ys[0], ELEM), max(20, steps))
    copy_ceiling = {"ms": round(ms_copy, 5), "GB/s": round(2 * ELEM * 4 / (ms_copy * 1e-3) / 1e9, 1),
                    "frac": round(2 * ELEM * 4 / (ms_copy * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "bytes": 2 * ELEM * 4,
                    "same_buffer": {"ms": round(ms_copy_same, 5), "frac": round(2 * ELEM * 4 / (ms_copy_same * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
                    "workload": "plain streaming copy fp32 [8192,4096] -> [8192,4096], one 128-bit vector per lane, same rotating buffer sets"}
    log("[rowops] %-18s %.4f ms  %7.1f GB/s  %.1f%% of HBM peak (the ceiling of a read-once / write-once kernel here; same buffer %.1f%%)"
        % ("copy_ceiling", ms_copy, copy_ceiling["GB/s"], 100 * copy_ceiling["frac"], 100 * copy_ceiling["same_buffer"]["frac"]))
    dominant = max(per_kernel, key=lambda k: per_kernel[k]["ms"])
    per_kernel["copy_ceiling"] = copy_ceiling
    roof = {"bound": "hbm", "kernel": dominant, "achieved": per_kernel[dominant]["GB/s"], "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": per_kernel[dominant]["frac"], "traffic": MEASURED_HBM_TRAFFIC.get(dominant),
            "buffers": "%d rotating input/output sets per kernel (no reuse from the last-level cache)" % ROTATE_SETS}
    del xs, rs, ys

    cpu = None
    if with_cpu:
        O = cpu_oracle()

        def cpu_step():
            O.softmax(x, 1)
            O.layer_norm(x, gamma, beta, 1e-5)
            O.rms_norm(x, gamma, 1e-6)
            O.gelu(x)
            O.bias_add(x, bias, res)

        cpu_step()
        best = float("inf")
        t_all = time.perf_counter()
        reps = 0
        while reps < 3 or (time.perf_counter() - t_all < 10.0 and reps < 400):
            t0 = time.perf_counter()
            cpu_step()
            best = min(best, time.perf_counter() - t0)
            reps += 1
        cpu = {"value": round(step_bytes / best / 1e9, 2), "unit": "GB/s", "cores": O.threads(), "kind": "port",
               "sample": "the full config-2 step (5 row ops on fp32 [8192,4096]), best of %d runs, %.1f s of CPU work"
                         % (reps, time.perf_counter() - t_all)}
        log("[rowops] cpu baseline %.2f GB/s on %d threads" % (cpu["value"], cpu["cores"]))
        # Context only, clearly labelled: the same five ops through PyTorch's own CPU kernels.
        try:
            import torch

            tx, tg, tb = torch.from_numpy(x), torch.from_numpy(gamma), torch.from_numpy(beta)
            tbias, tres = torch.from_numpy(bias), torch.from_numpy(res)

            def torch_step():
                torch.softmax(tx, 1)
                torch.nn.functional.layer_norm(tx, (COLS,), tg, tb, 1e-5)
                tx * torch.rsqrt(tx.pow(2).mean(1, keepdim=True) + 1e-6) * tg
                torch.nn.functional.gelu(tx)
                tx + tbias + tres

            best_t, reps_t = cpu_time(torch_step, 4.0)
            cpu["torch_cpu_context"] = {"value": round(step_bytes / best_t / 1e9, 2), "unit": "GB/s", "threads": torch.get_num_threads(),
                                        "note": "PyTorch %s CPU kernels on the same tensors, best of %d; not the reference" % (torch.__version__, reps_t)}
            log("[rowops] torch CPU context %.2f GB/s" % cpu["torch_cpu_context"]["value"])
        except Exception as exc:  # context line only
            log("[rowops] torch CPU context skipped: %s" % exc)
    return value, ms_per_step, roof, per_kernel, cpu


def cpu_oracle():
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle as O  # CPU checker restating ft-kernel-cpu: the reported baseline only

    return O


def cpu_time(fn, budget_s, min_reps=2, max_reps=50):
    """Best-of-N wall time of a CPU call inside a time budget (one untimed warm-up first)."""
    fn()
    best, reps, t_all = float("inf"), 0, time.perf_counter()
    while reps < min_reps or (time.perf_counter() - t_all < budget_s and reps < max_reps):
        t0 = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t0)
        reps += 1
    return best, reps


def bench_gemm(device, synth, steps, with_cpu):
    from frankentorch_amd.device import EPI_BIAS, DeviceBuffer

    out = {}
    a = synth.uniform(2, "A", (4096, 4096), -1, 1)
    b = synth.uniform(2, "B", (4096, 4096), -1, 1)
    da, db = DeviceBuffer.from_host(a), DeviceBuffer.from_host(b)
    dc = DeviceBuffer((4096, 4096))
    iters = max(10, steps)

    def run(name, desc, A, B, Cc, bias, flop, peak):
        fn = lambda: device.gemm(desc, A, B, Cc, bias)
        for _ in range(3):
            fn()
        device.synchronize()
        ms = event_time_ms(device, fn, iters)
        tf = flop / (ms * 1e-3) / 1e12
        out[name] = {"ms": round(ms, 4), "TFLOP/s": round(tf, 2), "frac": round(tf / peak, 4), "flop": flop,
                     "peak_TFLOP/s": peak}
        log("[gemm] %-34s %.3f ms  %6.2f TFLOP/s  %.1f%% of MFMA peak" % (name, ms, tf, 100 * tf / peak))

    run("f32_4096x4096x4096_nn", device.gemm_desc(4096, 4096, 4096), da, db, dc, None, 2 * 4096 ** 3, FP32_MFMA_PEAK_TF)
    run("f32_4096x4096x4096_nt", device.gemm_desc(4096, 4096, 4096, trans_b=True), da, db, dc, None, 2 * 4096 ** 3,
        FP32_MFMA_PEAK_TF)
    b2 = synth.uniform(2, "B2", (4096, 11008), -1, 1)
    bias = synth.uniform(2, "bias2", (11008,), -1, 1)
    db2, dbias = DeviceBuffer.from_host(b2), DeviceBuffer.from_host(bias)
    dc2 = DeviceBuffer((4096, 11008))
    run("f32_4096x11008x4096_bias", device.gemm_desc(4096, 11008, 4096, epilogue=EPI_BIAS), da, db2, dc2, dbias,
        2 * 4096 * 4096 * 11008, FP32_MFMA_PEAK_TF)
    del db2, dc2
    ba = synth.uniform(2, "ba", (32, 512, 128), -1, 1)
    bb = synth.uniform(2, "bb", (32, 128, 512), -1, 1)
    dba, dbb = DeviceBuffer.from_host(ba), DeviceBuffer.from_host(bb)
    dbc = DeviceBuffer((32, 512, 512))
    run("f32_bmm_32x512x512x128", device.gemm_desc(512, 512, 128, batch=32), dba, dbb, dbc, None, 32 * 2 * 512 * 128 * 512,
        FP32_MFMA_PEAK_TF)
    da64, db64 = DeviceBuffer.from_host(a.astype(np.float64)), DeviceBuffer.from_host(b.astype(np.float64))
    dc64 = DeviceBuffer((4096, 4096), np.float64)
    run("f64_4096x4096x4096_nn", device.gemm_desc(4096, 4096, 4096), da64, db64, dc64, None, 2 * 4096 ** 3, FP64_MFMA_PEAK_TF)
    if with_cpu:
        O = cpu_oracle()
        if O.sgemm_blocked(a[:64], b) is not None:
            best, reps = cpu_time(lambda: O.sgemm_blocked(a, b), 4.0)
            out["cpu"] = {"value": round(2 * 4096 ** 3 / best / 1e12, 3), "unit": "TFLOP/s", "cores": O.threads(), "kind": "port",
                          "sample": "fp32 4096^3 [m,k].[k,n] with the blocked AVX2 kernel that stands in for matrixmultiply, best of %d" % reps}
            log("[gemm] cpu baseline %.3f TFLOP/s on %d threads" % (out["cpu"]["value"], O.threads()))
    return out


def bench_sdpa(device, synth, steps, with_cpu):
    from frankentorch_amd.device import DeviceBuffer

    B, H, S, D = 4, 32, 2048, 128
    s = 1.0 / math.sqrt(D)
    q, k, v = (synth.normal(3, t, (B * H, S, D), 0.0, s) for t in ("Q", "K", "V"))
    dq, dk, dv = DeviceBuffer.from_host(q), DeviceBuffer.from_host(k), DeviceBuffer.from_host(v)
    do = DeviceBuffer(q.shape)
    desc = device.sdpa_desc_contiguous(B * H, S, S, D, D, True)
    fn = lambda: device.sdpa_forward(desc, s, dq, dk, dv, do)
    for _ in range(2):
        fn()
    device.synchronize()
    ms = event_time_ms(device, fn, max(5, steps // 2))
    flop = B * H * 4 * D * (S * (S + 1) // 2)  # causal count: two products over the lower triangle
    tf = flop / (ms * 1e-3) / 1e12
    log("[sdpa] B4 H32 S2048 D128 causal  %.3f ms  %.2f TFLOP/s (causal count)  %.1f%% of MFMA peak" % (ms, tf, 100 * tf / FP32_MFMA_PEAK_TF))
    res = {"ms": round(ms, 4), "TFLOP/s": round(tf, 2), "frac": round(tf / FP32_MFMA_PEAK_TF, 4), "flop": flop,
           "peak_TFLOP/s": FP32_MFMA_PEAK_TF, "workload": "B4 H32 S2048 D128 causal fp32"}
    if with_cpu:
        O = cpu_oracle()
        nh = 16  # heads of the 128 timed on the CPU (one per thread); same causal flop count per head
        best, reps = cpu_time(lambda: O.sdpa_forward(q[:nh], k[:nh], v[:nh], s, True), 4.0, min_reps=1)
        res["cpu"] = {"value": round(flop * nh / (B * H) / best / 1e12, 4), "unit": "TFLOP/s", "cores": O.threads(), "kind": "port",
                      "sample": "%d of the %d heads, best of %d" % (nh, B * H, reps)}
        log("[sdpa] cpu baseline %.4f TFLOP/s (causal count) on %d threads" % (res["cpu"]["value"], O.threads()))
    del dq, dk, dv, do
    # the same causal problem in fp64 (the reference's own SDPA precision), on the fp64 matrix cores
    q64, k64, v64 = (t.astype(np.float64) for t in (q, k, v))
    eq, ek, ev = (DeviceBuffer.from_host(t) for t in (q64, k64, v64))
    eo = DeviceBuffer(q64.shape, np.float64)
    fn64 = lambda: device.sdpa_forward(desc, s, eq, ek, ev, eo)
    ms64 = event_time_ms(device, fn64, max(5, steps // 4))
    tf64 = flop / (ms64 * 1e-3) / 1e12
    log("[sdpa] B4 H32 S2048 D128 causal fp64  %.3f ms  %.2f TFLOP/s (causal count)  %.1f%% of the fp64 MFMA peak" % (ms64, tf64, 100 * tf64 / FP64_MFMA_PEAK_TF))
    res["fp64"] = {"ms": round(ms64, 4), "TFLOP/s": round(tf64, 2), "frac": round(tf64 / FP64_MFMA_PEAK_TF, 4), "flop": flop,
                   "peak_TFLOP/s": FP64_MFMA_PEAK_TF, "workload": "B4 H32 S2048 D128 causal fp64"}
    if with_cpu:
        best, reps = cpu_time(lambda: O.sdpa_forward(q64[:nh], k64[:nh], v64[:nh], s, True), 4.0, min_reps=1)
        res["fp64"]["cpu"] = {"value": round(flop * nh / (B * H) / best / 1e12, 4), "unit": "TFLOP/s", "cores": O.threads(), "kind": "port",
                              "sample": "%d of the %d heads, best of %d" % (nh, B * H, reps)}
    del eq, ek, ev, eo, q64, k64, v64
    # grouped-query attention with an additive mask: 32 query heads on 8 K/V heads, the same S and D, a dense soft
    # mask (every key visible), so the two products run over the full [S, S] rectangle and every mask value is read
    Bg, Hq, Hkv = 2, 32, 8
    qg = synth.normal(3, "Qg", (Bg, Hq, S, D), 0.0, s)
    kg, vg = (synth.normal(3, t, (Bg, Hkv, S, D), 0.0, s) for t in ("Kg", "Vg"))
    mask = synth.normal(3, "mask", (S, S), 0.0, 0.5)
    bq, bk, bv, bm = (DeviceBuffer.from_host(t) for t in (qg, kg, vg, mask))
    bo = DeviceBuffer(qg.shape)
    gdesc = device.sdpa_desc_gqa(Bg, Hq, Hkv, S, S, D, D, False)
    gfn = lambda: device.sdpa_forward_masked(gdesc, s, bq, bk, bv, bm, 0, bo)
    for _ in range(2):
        gfn()
    device.synchronize()
    gms = event_time_ms(device, gfn, max(5, steps // 2))
    gflop = Bg * Hq * 4 * D * S * S
    gtf = gflop / (gms * 1e-3) / 1e12
    log("[sdpa] masked GQA B2 Hq32 Hkv8 S2048 D128  %.3f ms  %.2f TFLOP/s  %.1f%% of MFMA peak" % (gms, gtf, 100 * gtf / FP32_MFMA_PEAK_TF))
    res["masked_gqa"] = {"ms": round(gms, 4), "TFLOP/s": round(gtf, 2), "frac": round(gtf / FP32_MFMA_PEAK_TF, 4), "flop": gflop,
                         "workload": "B2, 32 query heads on 8 K/V heads, S2048 D128 fp32, shared additive [S,S] mask, no hidden keys"}
    if with_cpu:
        best, reps = cpu_time(lambda: O.sdpa_forward_masked_gqa(qg[:1, :16], kg[:1, :4], vg[:1, :4], np.float32(s), mask), 4.0, min_reps=1)
        res["masked_gqa"]["cpu"] = {"value": round(gflop * 16 / (Bg * Hq) / best / 1e12, 4), "unit": "TFLOP/s", "cores": O.threads(),
                                    "kind": "port", "sample": "16 of the 64 query heads, best of %d" % reps}
    return res


def bench_backward(device, synth, steps, with_cpu):
    """Backward kernels of the same ops at the forward benchmark shapes."""
    from frankentorch_amd.device import DeviceBuffer

    out = {}
    iters = max(10, steps // 2)
    O = cpu_oracle() if with_cpu else None

    def timed(fn, n=iters):
        for _ in range(3):
            fn()
        device.synchronize()
        return event_time_ms(device, fn, n)

    # LayerNorm / RMSNorm backward, fp32 [8192,4096]: read x and dy, write dx (+ weight, dweight, dbias once)
    x = synth.normal(1, "x", (ROWS, COLS))
    dy = synth.normal(1, "dy", (ROWS, COLS))
    gamma = synth.uniform(1, "gamma", (COLS,), 0.5, 1.5)
    # rotating buffer sets, as for the forward row ops: x, dy in and dx out per set
    nsets = 8
    xs_, dys, gxs = ([DeviceBuffer.from_host(x) for _ in range(nsets)], [DeviceBuffer.from_host(dy) for _ in range(nsets)],
                     [DeviceBuffer((ROWS, COLS)) for _ in range(nsets)])
    dg = DeviceBuffer.from_host(gamma)
    gw, gb = DeviceBuffer((COLS,)), DeviceBuffer((COLS,))
    ws = device.layer_norm_backward(dys[0], xs_[0], dg, gxs[0], gw, gb, ROWS, COLS, 1e-5)
    turn = [0]

    def nxt():
        turn[0] = (turn[0] + 1) % nsets
        return turn[0]

    def ln_bwd():
        i = nxt()
        device.layer_norm_backward(dys[i], xs_[i], dg, gxs[i], gw, gb, ROWS, COLS, 1e-5, workspace=ws)

    def rms_bwd():
        i = nxt()
        device.rms_norm_backward(dys[i], xs_[i], dg, gxs[i], gw, ROWS, COLS, 1e-6, workspace=ws)

    for name, nbytes, fn, cpu_fn in (
        ("layer_norm_backward", 3 * ELEM * 4 + 3 * COLS * 4, ln_bwd, lambda: O.layer_norm_backward(dy, x, gamma, np.float32(1e-5))),
        ("rms_norm_backward", 3 * ELEM * 4 + 2 * COLS * 4, rms_bwd, lambda: O.rms_norm_backward(dy, x, gamma, np.float32(1e-6))),
    ):
        ms = timed(fn)
        gbs = nbytes / (ms * 1e-3) / 1e9
        out[name] = {"ms": round(ms, 5), "GB/s": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4), "bytes": nbytes,
                     "workload": "fp32 [8192,4096], dx + dweight (+ dbias), all launches of the entry point, %d rotating buffer sets" % nsets}
        log("[backward] %-20s %.4f ms  %7.1f GB/s  %.1f%% of HBM peak" % (name, ms, gbs, 100 * gbs / HBM_PEAK_GBS))
        if with_cpu:
            best, reps = cpu_time(cpu_fn, 2.0)
            out[name]["cpu"] = {"value": round(nbytes / best / 1e9, 2), "unit": "GB/s", "cores": O.threads(), "kind": "port",
                                "sample": "the same tensors, best of %d" % reps}
    del xs_, dys, gxs
    # linear backward at the GPT-2 FC1 shape: dx and dweight products + dbias
    batch, in_f, out_f = 8192, 768, 3072
    dyl, xl = synth.normal(4, "dyl", (batch, out_f)), synth.normal(4, "xl", (batch, in_f))
    wl = synth.normal(4, "wl", (out_f, in_f), 0.0, 0.02)
    a, b, c = DeviceBuffer.from_host(dyl), DeviceBuffer.from_host(xl), DeviceBuffer.from_host(wl)
    lx, lw, lb = DeviceBuffer((batch, in_f)), DeviceBuffer((out_f, in_f)), DeviceBuffer((out_f,))
    ws2 = device.linear_backward(a, b, c, lx, lw, lb, batch, in_f, out_f)
    ms = timed(lambda: device.linear_backward(a, b, c, lx, lw, lb, batch, in_f, out_f, workspace=ws2))
    flop = 4 * batch * in_f * out_f
    tf = flop / (ms * 1e-3) / 1e12
    out["linear_backward"] = {"ms": round(ms, 4), "TFLOP/s": round(tf, 2), "frac": round(tf / FP32_MFMA_PEAK_TF, 4), "flop": flop,
                              "workload": "fp32 batch 8192, 768 -> 3072: dx = dy.W, dweight = dy^T.x, dbias"}
    log("[backward] linear_backward      %.4f ms  %6.2f TFLOP/s  %.1f%% of MFMA peak" % (ms, tf, 100 * tf / FP32_MFMA_PEAK_TF))
    if with_cpu:
        nb = 512  # rows of the batch timed on the CPU (the checker's products accumulate wide and are slow)
        best, reps = cpu_time(lambda: O.linear_backward(dyl[:nb], xl[:nb], wl, True), 3.0, min_reps=1)
        out["linear_backward"]["cpu"] = {"value": round(4 * nb * in_f * out_f / best / 1e12, 4), "unit": "TFLOP/s", "cores": O.threads(),
                                         "kind": "port", "sample": "%d of the 8192 rows, wide-accumulation products, best of %d" % (nb, reps)}
    del a, b, c, lx, lw
    # SDPA backward at the config-4 shape; flop count of the reference's five full-rectangle products per head
    B, H, S, D = 4, 32, 2048, 128
    sc = 1.0 / math.sqrt(D)
    q, k, v = (synth.normal(3, t, (B * H, S, D), 0.0, sc) for t in ("Q", "K", "V"))
    do = synth.normal(3, "dO", (B * H, S, D))
    dq, dk, dv, ddo = (DeviceBuffer.from_host(t) for t in (q, k, v, do))
    gq, gk, gv = DeviceBuffer(q.shape), DeviceBuffer(q.shape), DeviceBuffer(q.shape)
    ws3 = device.sdpa_backward(dq, dk, dv, ddo, B * H, S, S, D, D, sc, True, gq, gk, gv)
    ms = timed(lambda: device.sdpa_backward(dq, dk, dv, ddo, B * H, S, S, D, D, sc, True, gq, gk, gv, workspace=ws3), max(3, steps // 10))
    flop_full = 5 * 2 * B * H * S * S * D          # what the reference executes: five full [S,S] products per head
    flop = 5 * 2 * B * H * (S * (S + 1) // 2) * D  # the causal count, as for the forward
    tf = flop / (ms * 1e-3) / 1e12
    out["sdpa_backward"] = {"ms": round(ms, 3), "TFLOP/s": round(tf, 2), "frac": round(tf / FP32_MFMA_PEAK_TF, 4), "flop": flop,
                            "reference_count_TFLOP/s": round(flop_full / (ms * 1e-3) / 1e12, 2),
                            "workload": "B4 H32 S2048 D128 causal fp32; flop = five products over the causal half (4 D S(S+1)/2 x 2.5 per head); "
                                        "reference_count = the reference's five full [S,S] products per head"}
    log("[backward] sdpa_backward        %.3f ms  %6.2f TFLOP/s  %.1f%% of MFMA peak" % (ms, tf, 100 * tf / FP32_MFMA_PEAK_TF))
    if with_cpu:
        best, reps = cpu_time(lambda: O.sdpa_backward(q[:1], k[:1], v[:1], do[:1], np.float32(sc), True), 3.0, min_reps=1)
        out["sdpa_backward"]["cpu"] = {"value": round(flop_full / (B * H) / best / 1e12, 4), "unit": "TFLOP/s (reference count)", "cores": O.threads(),
                                       "kind": "port", "sample": "1 of the 128 heads, wide-accumulation products, best of %d" % reps}
    del dq, dk, dv, ddo, gq, gk, gv, ws3
    # log-softmax and the fused cross-entropy on the forward's logits [8192, 50257] (made on the device by the LM-head product)
    rows, vocab, width = 8192, 50257, 768
    hid = synth.normal(5, "hidden", (rows, width)) * np.float32(0.25)
    wte = synth.normal(5, "wte", (vocab, width))
    tgt = synth.token_ids(5, "target", (rows,), vocab).astype(np.int64)
    dh, dwte, dtgt = DeviceBuffer.from_host(hid), DeviceBuffer.from_host(wte), DeviceBuffer.from_host(tgt)
    lg, lo = DeviceBuffer((rows, vocab)), DeviceBuffer((rows, vocab))
    loss, dloss = DeviceBuffer((rows,)), DeviceBuffer.from_host(np.ones(rows, np.float32))
    device.gemm(device.gemm_desc(rows, vocab, width, trans_b=True), dh, dwte, lg)
    nel = rows * vocab * 4
    sample = None
    if with_cpu:
        nb = 64
        sample = (hid[:nb].astype(np.float64) @ wte.T.astype(np.float64)).astype(np.float32)
    for name, nbytes, fn, cpu_fn in (
        ("log_softmax", 2 * nel, lambda: device.log_softmax_strided(lg, lo, rows, vocab, 1), lambda: O.log_softmax(sample, 1)),
        ("cross_entropy_forward", nel + rows * 12, lambda: device.cross_entropy_forward(lg, dtgt, rows, vocab, loss),
         lambda: O.cross_entropy_forward(sample, tgt[:64])),
        ("cross_entropy_backward", 2 * nel + rows * 12, lambda: device.cross_entropy_backward(lg, dtgt, dloss, rows, vocab, lo),
         lambda: O.cross_entropy_backward(sample, tgt[:64], np.ones(64, np.float32))),
        # softmax over the vocabulary: rows that are no multiple of a 128-bit vector and far beyond 8192 vectors
        ("softmax_vocab", 2 * nel, lambda: device.softmax_lastdim(lg, lo, rows, vocab), lambda: O.softmax(sample, 1)),
    ):
        ms = timed(fn, max(5, steps // 5))
        gbs = nbytes / (ms * 1e-3) / 1e9
        out[name] = {"ms": round(ms, 4), "GB/s": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4), "bytes": nbytes,
                     "workload": "fp32 logits [8192,50257], int64 targets"}
        log("[backward] %-22s %.4f ms  %7.1f GB/s  %.1f%% of HBM peak" % (name, ms, gbs, 100 * gbs / HBM_PEAK_GBS))
        if with_cpu:
            best, reps = cpu_time(cpu_fn, 2.0)
            out[name]["cpu"] = {"value": round(nbytes * 64 / rows / best / 1e9, 2), "unit": "GB/s", "cores": O.threads(), "kind": "port",
                                "sample": "64 of the 8192 rows, best of %d" % reps}
    del lg, lo, dh, dwte
    # int8 dynamic-quantised linear: quantise x per row, integer matrix-core product, dequantise (+ bias)
    m8, k8, n8 = 8192, 4096, 4096
    x8 = synth.normal(6, "x8", (m8, k8), 0.0, 3.0)
    w8 = synth.normal(6, "w8", (n8, k8), 0.0, 0.5)
    b8 = synth.normal(6, "b8", (n8,))
    dx8, dw8f, db8 = DeviceBuffer.from_host(x8), DeviceBuffer.from_host(w8), DeviceBuffer.from_host(b8)
    dwq, dws, dy8 = DeviceBuffer((n8, k8), np.int8), DeviceBuffer((n8,)), DeviceBuffer((m8, n8))
    device.quantize_rows_i8(dw8f, n8, k8, dwq, dws)  # weights: once, outside the timed region
    ws8 = device.linear_int8_dynamic(dx8, m8, k8, dwq, dws, n8, db8, dy8)
    ms = timed(lambda: device.linear_int8_dynamic(dx8, m8, k8, dwq, dws, n8, db8, dy8, workspace=ws8))
    # the quantiser alone, over rotating buffer sets (128 MiB in, 32 MiB out per launch; see bench_rowops)
    qin = [dx8] + [DeviceBuffer.from_host(x8) for _ in range(ROTATE_SETS - 1)]
    qout = [(DeviceBuffer((m8, k8), np.int8), DeviceBuffer((m8,))) for _ in range(ROTATE_SETS)]
    qturn = [0]

    def quantise_next():
        qturn[0] = (qturn[0] + 1) % ROTATE_SETS
        device.quantize_rows_i8(qin[qturn[0]], m8, k8, qout[qturn[0]][0], qout[qturn[0]][1])

    ms_q = timed(quantise_next)
    ms_q_same = timed(lambda: device.quantize_rows_i8(dx8, m8, k8, qout[0][0], qout[0][1]))
    del qin, qout
    # The same launches on all-zero operands (LAST, so that a counter run sees the product kernel's dispatches in two
    # groups: random operands first, zeros second): the integer matrix rate of this chip depends on the operand values.
    dxz = DeviceBuffer.from_host(np.zeros((m8, k8), np.float32))
    dwqz = DeviceBuffer.from_host(np.zeros((n8, k8), np.int8))
    ms_zero = timed(lambda: device.linear_int8_dynamic(dxz, m8, k8, dwqz, dws, n8, db8, dy8, workspace=ws8))
    del dxz, dwqz
    ops = 2 * m8 * n8 * k8
    tops = ops / ((ms - ms_q_same) * 1e-3) / 1e12  # in the whole call the quantiser re-reads the same x
    qbytes = m8 * k8 * 5 + m8 * 4
    out["linear_int8_dynamic"] = {"ms": round(ms, 4), "quantize_ms": round(ms_q, 4), "product_TOP/s": round(tops, 1), "frac": round(tops / 5000.0, 4),
                                  "peak_TOP/s": 5000.0, "ops": ops, "quantize_GB/s": round(qbytes / (ms_q * 1e-3) / 1e9, 1),
                                  "quantize_same_buffer_GB/s": round(qbytes / (ms_q_same * 1e-3) / 1e9, 1),
                                  "zero_operands": {"ms": round(ms_zero, 4), "product_TOP/s": round(2 * m8 * n8 * k8 / ((ms_zero - ms_q_same) * 1e-3) / 1e12, 1)},
                                  "workload": "x fp32 [8192,4096] . int8 W[4096,4096]^T + bias; product rate = ops / (whole call - quantiser)"}
    log("[backward] linear_int8_dynamic    %.4f ms (quantiser %.4f ms = %.0f GB/s); product %.0f TOP/s  %.1f%% of the 5.0 POP/s int8 peak"
        % (ms, ms_q, qbytes / (ms_q * 1e-3) / 1e9, tops, 100 * tops / 5000.0))
    if with_cpu:
        wq_h, ws_h = O.quantize_rows_i8(w8[:512])
        best, reps = cpu_time(lambda: O.linear_int8_dynamic(x8[:256], wq_h, ws_h, b8[:512]), 3.0, min_reps=1)
        out["linear_int8_dynamic"]["cpu"] = {"value": round(2 * 256 * 512 * k8 / best / 1e12, 4), "unit": "TOP/s", "cores": O.threads(), "kind": "port",
                                             "sample": "256 rows x 512 outputs of the 8192 x 4096, scalar i32 dot products, best of %d" % reps}
    return out


def bench_index(device, synth, steps):
    """The integer-exact kernels at the config-5 shapes: fused token + position embedding gather, head split (perm [0,2,1,3]) and
    the argmax over the logits. Algorithmic bytes = every input element the kernel must read once + every output element once."""
    from frankentorch_amd.device import DeviceBuffer
    import numpy as np

    out = {}
    vocab, width, batch, seq, heads = 50257, 768, 8, 1024, 12
    tokens = batch * seq
    iters = max(10, steps // 4)
    wte = DeviceBuffer.from_host(synth.normal(4, "wte", (vocab, width)) * np.float32(0.02))
    wpe = DeviceBuffer.from_host(synth.normal(4, "wpe", (seq, width)) * np.float32(0.02))
    ids = DeviceBuffer.from_host(synth.token_ids(4, "ids", (tokens,), vocab))
    emb = DeviceBuffer((tokens, width))
    ms = event_time_ms(device, lambda: device.embedding_add(wte, vocab, wpe, seq, ids, tokens, seq, width, emb), iters)
    nbytes = tokens * 8 + 2 * tokens * width * 4 + seq * width * 4  # ids, gathered rows + output, the position table once
    out["embedding_add"] = {"ms": round(ms, 5), "GB/s": round(nbytes / ms / 1e6, 1), "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                            "bytes": nbytes, "workload": "wte[50257,768] + wpe[1024,768] gather for 8192 ids (50 MB per launch: back-to-back launches run out of the 256 MB last-level cache, so this is not an HBM rate)"}
    log("[index] embedding_add   %.4f ms  %7.1f GB/s" % (ms, nbytes / ms / 1e6))
    src, dst = DeviceBuffer((batch, seq, heads, width // heads)), DeviceBuffer((batch, heads, seq, width // heads))
    ms = event_time_ms(device, lambda: device.permute_0213(emb, dst, batch, seq, heads, width // heads), iters)
    nbytes = 2 * tokens * width * 4
    out["permute_0213"] = {"ms": round(ms, 5), "GB/s": round(nbytes / ms / 1e6, 1), "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                           "bytes": nbytes, "workload": "[8,1024,12,64] -> [8,12,1024,64] fp32 (50 MB per launch: served by the last-level cache when repeated; the block path never runs it)"}
    log("[index] permute_0213    %.4f ms  %7.1f GB/s" % (ms, nbytes / ms / 1e6))
    del src
    logits = DeviceBuffer((tokens, vocab))
    device.gemm(device.gemm_desc(tokens, vocab, width, trans_b=True), emb, wte, logits)
    am = DeviceBuffer((tokens,))
    ms = event_time_ms(device, lambda: device.argmax(logits, tokens, vocab, 1, am), iters)
    nbytes = tokens * vocab * 4 + tokens * 4
    out["argmax"] = {"ms": round(ms, 5), "GB/s": round(nbytes / ms / 1e6, 1), "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                     "bytes": nbytes, "workload": "argmax over the last dim of fp32 logits [8192,50257] (read-only stream)"}
    log("[index] argmax          %.4f ms  %7.1f GB/s  %.1f%% of HBM peak" % (ms, nbytes / ms / 1e6, 100 * nbytes / ms / 1e6 / HBM_PEAK_GBS))
    return out


def bench_tier_a(device, synth, with_cpu):
    """The host-slice entry points end to end: pageable host arrays in, a caller-owned host array out, wall clock around the
    call (host copies into pinned chunks, both DMA directions, kernels). This is the call shape ft-dispatch uses today."""
    import ctypes as C

    from frankentorch_amd import _lib
    from frankentorch_amd.core import TensorMeta, check
    from frankentorch_amd.device import DeviceBuffer

    L = _lib.load()
    out = {}
    x = synth.normal(1, "x", (ROWS, COLS))
    gamma = synth.uniform(1, "gamma", (COLS,), 0.5, 1.5)
    beta = synth.normal(1, "beta", (COLS,), 0.0, 0.1)
    y = np.zeros((ROWS, COLS), np.float32)  # caller-owned and already touched: the `_into` call shape
    meta = TensorMeta.from_shape((ROWS, COLS)).to_c()
    n_out = C.c_size_t(0)

    def wall(fn, reps=8):
        # a quarter of a second of untimed calls first: the first dozen calls after the host threads have been busy
        # elsewhere (the CPU legs of this case) run 10 % slower than the steady state
        t_end = time.perf_counter() + 0.25
        fn()
        while time.perf_counter() < t_end:
            fn()
        best = float("inf")
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            best = min(best, time.perf_counter() - t0)
        return best

    # the host link alone: one pinned 128 MiB buffer each way, both directions at once on two streams
    nbytes = ELEM * 4
    link = device.link_rates(nbytes)
    log("[tier_a] host link, pinned %d MiB: H2D %.1f GB/s, D2H %.1f GB/s, both at once %.1f + %.1f GB/s"
        % (nbytes >> 20, link["h2d"], link["d2h"], link["h2d_duplex"], link["d2h_duplex"]))
    out["host_link"] = {"bytes": nbytes, "GB/s": link,
                        "note": "hipMemcpyAsync from / to pinned memory; duplex = both directions at once on two streams"}
    link_ms = nbytes / (min(link["h2d_duplex"], link["d2h_duplex"]) * 1e9) * 1e3
    O = cpu_oracle() if with_cpu else None
    cases = (
        ("softmax_dim_tensor_contiguous_f32", 2 * nbytes,
         lambda: check(L.fth_softmax_dim_tensor_contiguous_f32(x.ctypes.data, x.size, C.byref(meta), 1, y.ctypes.data, y.size, C.byref(n_out))),
         lambda: O.softmax(x, 1)),
        ("layer_norm_forward_f32", 2 * nbytes,
         lambda: check(L.fth_layer_norm_forward_f32(x.ctypes.data, x.size, gamma.ctypes.data, beta.ctypes.data, ROWS, COLS, C.c_float(1e-5),
                                                    y.ctypes.data, y.size)),
         lambda: O.layer_norm(x, gamma, beta, 1e-5)),
    )
    for name, moved, fn, cpu_fn in cases:
        t = wall(fn)
        out[name] = {"ms": round(t * 1e3, 3), "GB/s": round(moved / t / 1e9, 2), "bytes_over_the_link": moved,
                     "link_ms": round(link_ms, 3), "vs_link": round(t * 1e3 / link_ms, 3),
                     "workload": "fp32 [8192,4096] host slice in, host buffer out (128 MiB each way)"}
        log("[tier_a] %-36s %.2f ms end to end (%.2fx the duplex link time of %.2f ms)" % (name, t * 1e3, t * 1e3 / link_ms, link_ms))
        if with_cpu:
            best, reps = cpu_time(cpu_fn, 3.0)
            out[name]["cpu"] = {"ms": round(best * 1e3, 3), "cores": O.threads(), "kind": "port", "sample": "the same call, best of %d" % reps}
            log("[tier_a] %-36s cpu port %.2f ms on %d threads" % (name, best * 1e3, O.threads()))
    # fresh output allocation per call (a new Vec per call, as the non-_into reference functions return): first-touch page faults included
    def fresh():
        z = np.empty((ROWS, COLS), np.float32)
        check(L.fth_softmax_dim_tensor_contiguous_f32(x.ctypes.data, x.size, C.byref(meta), 1, z.ctypes.data, z.size, C.byref(n_out)))
    t = wall(fresh, 3)
    out["softmax_dim_tensor_contiguous_f32"]["fresh_output_ms"] = round(t * 1e3, 3)
    log("[tier_a] softmax into a newly allocated output: %.2f ms" % (t * 1e3))
    del y
    a = synth.uniform(2, "A", (4096, 4096), -1, 1)
    b = synth.uniform(2, "B", (4096, 4096), -1, 1)
    c = np.zeros((4096, 4096), np.float32)
    m2 = TensorMeta.from_shape((4096, 4096)).to_c()
    t = wall(lambda: check(L.fth_matmul_tensor_contiguous_f32(a.ctypes.data, a.size, b.ctypes.data, b.size, C.byref(m2), C.byref(m2),
                                                              c.ctypes.data, c.size, C.byref(n_out))))
    flop = 2 * 4096 ** 3
    out["matmul_tensor_contiguous_f32"] = {"ms": round(t * 1e3, 3), "TFLOP/s": round(flop / t / 1e12, 2), "bytes_over_the_link": 3 * 4096 * 4096 * 4,
                                           "workload": "fp32 4096^3 host slices in (2 x 64 MiB), host buffer out (64 MiB)"}
    log("[tier_a] matmul_tensor_contiguous_f32 4096^3  %.2f ms end to end = %.1f TFLOP/s" % (t * 1e3, flop / t / 1e12))
    if with_cpu and O.sgemm_blocked(a[:64], b) is not None:
        best, reps = cpu_time(lambda: O.sgemm_blocked(a, b), 3.0)
        out["matmul_tensor_contiguous_f32"]["cpu"] = {"ms": round(best * 1e3, 2), "cores": O.threads(), "kind": "port",
                                                      "sample": "the same product with the blocked AVX2 kernel, best of %d" % reps}
    return out


def make_layer(synth, seed, li, d, f):
    n = lambda tag, *s: synth.normal(seed, "L%d.%s" % (li, tag), s, 0.0, 0.02)
    one, zero = (lambda m: np.ones(m, np.float32)), (lambda m: np.zeros(m, np.float32))
    return {"ln1_w": one(d), "ln1_b": zero(d), "wq": n("wq", d, d), "bq": zero(d), "wk": n("wk", d, d), "bk": zero(d),
            "wv": n("wv", d, d), "bv": zero(d), "wo": n("wo", d, d), "bo": zero(d), "ln2_w": one(d), "ln2_b": zero(d),
            "w1": n("w1", f, d), "b1": zero(f), "w2": n("w2", d, f), "b2": zero(d)}


def bench_block(device, synth, steps, with_cpu, with_graph=False):
    from frankentorch_amd import fused
    from frankentorch_amd.device import DeviceBuffer

    batch, seq, d, heads, f = 1, 128, 256, 4, 1024
    enc = fused.EncoderHip(d, heads, f, [make_layer(synth, 0, 0, d, f)], 1e-5, causal=True)
    x = synth.normal(0, "x", (batch * seq, d))
    dx, dout = DeviceBuffer.from_host(x), DeviceBuffer((batch * seq, d))
    res = {"workload": "pre-LN block B1 S128 d256 h4 ffn1024 causal fp32 (launch-latency-bound)"}
    iters = max(50, steps)
    # The HIP-graph replay is opt-in (--graph): it is no faster than the seven eager launches, and it must never run under a
    # profiler (the library refuses it there).
    for label, graph in (("eager", False),) + ((("graph", True),) if with_graph else ()):
        fn = lambda: enc.forward_dev(dx, dout, batch, seq, graph=graph)
        for _ in range(3):
            fn()
        device.synchronize()
        ms = event_time_ms(device, fn, iters)
        res[label] = {"ms": round(ms, 5), "tokens/s": round(batch * seq / (ms * 1e-3), 1)}
        log("[block] %s %.4f ms  %.0f tokens/s" % (label, ms, batch * seq / (ms * 1e-3)))
    flop = 2.10e8
    res["flop"] = flop
    res["frac"] = round(flop / (res["eager"]["ms"] * 1e-3) / 1e12 / FP32_MFMA_PEAK_TF, 5)
    if with_cpu:
        O = cpu_oracle()
        layer = make_layer(synth, 0, 0, d, f)
        best, reps = cpu_time(lambda: O.encoder_layer(layer, x, batch, seq, heads, 1e-5, True), 2.0, max_reps=200)
        res["cpu"] = {"value": round(batch * seq / best, 1), "unit": "tokens/s", "cores": O.threads(), "kind": "port",
                      "sample": "the same block and input, best of %d" % reps}
        log("[block] cpu baseline %.0f tokens/s on %d threads" % (res["cpu"]["value"], O.threads()))
    return res


def bench_gpt2(device, synth, steps):
    from frankentorch_amd import fused
    from frankentorch_amd.device import DeviceBuffer

    vocab, maxpos, d, heads, f, nl, batch, seq = 50257, 1024, 768, 12, 3072, 12, 8, 1024
    log("[gpt2] generating GPT-2-small-shaped weights (seed 4)")
    wte = synth.normal(4, "wte", (vocab, d), 0.0, 0.02)
    wpe = synth.normal(4, "wpe", (maxpos, d), 0.0, 0.02)
    layers = [make_layer(synth, 4, i, d, f) for i in range(nl)]
    ids = synth.token_ids(4, "ids", (batch * seq,), vocab)
    model = fused.Gpt2Hip(wte, wpe, layers, None, None, heads, 1e-5)
    T = batch * seq
    dids = DeviceBuffer.from_host(ids)
    dlog, dam = DeviceBuffer((T, vocab)), DeviceBuffer((T,))
    fn = lambda: model.forward_dev(dids, batch, seq, dlog, dam)
    for _ in range(2):
        fn()
    device.synchronize()
    ms = event_time_ms(device, fn, max(5, steps // 4))
    flop = 12 * 2 * T * d * (3 * d + d + 2 * f) + 12 * (batch * heads) * 4 * (d // heads) * (seq * (seq + 1) // 2) + 2 * T * d * vocab
    tf = flop / (ms * 1e-3) / 1e12
    log("[gpt2] forward (logits + argmax) %.3f ms  %.0f tokens/s  %.2f TFLOP/s  %.1f%% of MFMA peak"
        % (ms, T / (ms * 1e-3), tf, 100 * tf / FP32_MFMA_PEAK_TF))
    res = {"ms": round(ms, 3), "tokens/s": round(T / (ms * 1e-3), 1), "TFLOP/s": round(tf, 2), "frac": round(tf / FP32_MFMA_PEAK_TF, 4),
           "flop": flop, "workload": "GPT-2-small shape: 12L d768 h12 ffn3072 vocab50257 B8 S1024 fp32, logits + argmax"}
    # The head alone, the two ways the library can run it: the product with row maxima recorded in its epilogue followed by the
    # small finishing kernel (what the forward above uses), and the plain product followed by the argmax kernel over all logits.
    hx = DeviceBuffer.from_host(synth.normal(4, "head.x", (T, d), 0.0, 1.0))
    hw = DeviceBuffer.from_host(wte)
    hws = DeviceBuffer((device.linear_argmax_workspace_floats(T, vocab),))
    n_head = max(5, steps // 4)
    head_ms = {}
    for name, wsp in (("fused", hws), ("separate", None)):
        head_ms[name] = event_time_ms(device, lambda: device.linear_argmax(hx, hw, T, vocab, d, dlog, dam, workspace=wsp), n_head, warm_s=0.2)
    fn()  # dam again holds the forward's argmax
    res["lm_head_argmax"] = {"fused_ms": round(head_ms["fused"], 3), "separate_ms": round(head_ms["separate"], 3),
                             "workload": "logits [8192, 50257] = x [8192, 768] . wte^T and the row argmax, back to back"}
    log("[gpt2] LM head + argmax alone: %.3f ms with the row maxima recorded in the product's epilogue, %.3f ms as two kernels"
        % (head_ms["fused"], head_ms["separate"]))
    del hx, hw, hws
    # Weight ingestion: the same weights as a safetensors checkpoint (Hugging Face names, Conv1D [in, out] matrices) in
    # host memory, loaded straight into resident buffers (pinned staging, transposes on the GPU).
    import json
    import struct

    first = dam.to_host()
    del model
    names = {"wte.weight": wte, "wpe.weight": wpe, "ln_f.weight": np.ones(d, np.float32), "ln_f.bias": np.zeros(d, np.float32)}
    for i, L in enumerate(layers):
        h = "h.%d." % i
        names.update({h + "ln_1.weight": L["ln1_w"], h + "ln_1.bias": L["ln1_b"], h + "ln_2.weight": L["ln2_w"], h + "ln_2.bias": L["ln2_b"],
                      h + "attn.c_attn.weight": np.ascontiguousarray(np.concatenate([L["wq"], L["wk"], L["wv"]], axis=0).T),
                      h + "attn.c_attn.bias": np.concatenate([L["bq"], L["bk"], L["bv"]]),
                      h + "attn.c_proj.weight": np.ascontiguousarray(L["wo"].T), h + "attn.c_proj.bias": L["bo"],
                      h + "mlp.c_fc.weight": np.ascontiguousarray(L["w1"].T), h + "mlp.c_fc.bias": L["b1"],
                      h + "mlp.c_proj.weight": np.ascontiguousarray(L["w2"].T), h + "mlp.c_proj.bias": L["b2"]})
    hdr, off = {}, 0
    for k in sorted(names):
        hdr[k] = {"dtype": "F32", "shape": list(names[k].shape), "data_offsets": [off, off + names[k].nbytes]}
        off += names[k].nbytes
    hj = json.dumps(hdr).encode()
    blob = struct.pack("<Q", len(hj)) + hj + b"".join(np.ascontiguousarray(names[k], np.float32).tobytes() for k in sorted(names))
    best = float("inf")
    for _ in range(3):
        t0 = time.perf_counter()
        loaded = fused.Gpt2Hip.from_safetensors(blob, heads, 1e-5, gelu_tanh=False)
        device.synchronize()
        best = min(best, time.perf_counter() - t0)
    loaded.forward_dev(dids, batch, seq, None, dam)
    same = bool(np.array_equal(first, dam.to_host()))
    res["ingest"] = {"seconds": round(best, 4), "GB/s": round(off / best / 1e9, 2), "bytes": off, "same_argmax_as_host_built_model": same,
                     "workload": "GPT-2-small safetensors checkpoint (fp32, 149 tensors) from host memory into resident buffers, "
                                 "48 matrices transposed on the GPU; best of 3"}
    log("[gpt2] checkpoint ingestion %.1f MB in %.3f s = %.2f GB/s (host memory -> HBM, PCIe-bound); argmax identical: %s"
        % (off / 1e6, best, off / best / 1e9, same))
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--cases", default="all", help="comma list of: gemm,sdpa,block,gpt2,backward,index,tier_a (row ops always run); 'none' for row ops only")
    ap.add_argument("--graph", action="store_true", help="also time the HIP-graph replay of the block (never under a profiler)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend runs on ONE GPU; --gpus %d is not supported (no collectives, no sharding)" % args.gpus)

    from frankentorch_amd import device, synth

    if not device.is_available():
        sys.exit("bench.py: no usable gfx950 device; the HIP library has no CPU fallback")
    info = device.device_info()
    log("[device] %s, %d CUs, %.0f GiB HBM, engine %d MHz" % (info["arch"], info["compute_units"], info["hbm_bytes"] / 2 ** 30,
                                                               info["engine_clock_khz"] // 1000))
    cases = {"gemm", "sdpa", "block", "gpt2", "backward", "index", "tier_a"} if args.cases == "all" else set(c for c in args.cases.split(",") if c and c != "none")

    value, ms_per_step, roof, per_kernel, cpu = bench_rowops(device, synth, args.steps, args.warmup, not args.no_cpu)
    extra = {"row_ops": per_kernel}
    if "gemm" in cases:
        extra["gemm"] = bench_gemm(device, synth, args.steps, not args.no_cpu)
    if "sdpa" in cases:
        extra["sdpa_causal"] = bench_sdpa(device, synth, args.steps, not args.no_cpu)
    if "block" in cases:
        extra["block"] = bench_block(device, synth, args.steps, not args.no_cpu, args.graph)
    if "gpt2" in cases:
        extra["gpt2_forward"] = bench_gpt2(device, synth, args.steps)
    if "backward" in cases:
        extra["backward"] = bench_backward(device, synth, args.steps, not args.no_cpu)
    if "index" in cases:
        extra["index"] = bench_index(device, synth, args.steps)
    if "tier_a" in cases:
        extra["tier_a"] = bench_tier_a(device, synth, not args.no_cpu)

    line = {
        "metric": "row-op GB/s (fp32, 1 MI355X)",
        "metric_full": "GEMM TFLOP/s, row-op GB/s, fused-block tokens/s (fp32, 1 MI355X) + %roofline",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[1]: row ops on fp32 [8192,4096], seed 1: softmax + LayerNorm + RMSNorm + erf-GELU + bias+residual add",
                   "bytes_per_step": sum(ROW_BYTES.values()), "device": info["arch"], "compute_units": info["compute_units"]},
        "roofline": roof,
        "cpu_baseline": cpu,
        "cases": extra,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
