#!/usr/bin/env python3
"""Benchmark of the GGUF block-quantized linear path on one MI355X.

Default workload (`decode27b`): the full per-token mat-vec set of a Gemma-3-27B-shaped stack, all weights Q8_0 and
random-init, resident in HBM (62 layers x {q,k,v,o,gate,up,down} + lm_head = 435 mat-vecs, 28,695,625,728 weight bytes
per token).  A "step" is one token: every mat-vec of the set once, fresh N(0,1) FP32 activations, batch 1.
`value` is tokens/s; `roofline` is the Q8_0 mat-vec kernel's achieved HBM rate over the same timed region.

Other workloads (`--workload gemv|prefill|ffn|decode_loop|decode27b_chained|all`) time the single-matrix configurations,
the fused layer half, the GGUF decode loop and the 27B-shape token in dependency order; they are reported under "also".
`--workload library_gemm` (never part of "all") times the ROCm library's bfloat16 GEMM on the prefill shape through
torch.matmul, weights already decoded, as a yardstick for the machine; it does not load this library (PyTorch carries a
HIP runtime of its own, and two of them in one process do not both see the device).

One JSON line on stdout; progress on stderr.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from ctypes import c_void_p
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
BF16_PEAK_TFLOPS = 2500.0      # MI355X dense bf16 MFMA, published
COPY_KERNEL = "__amd_rocclr_copyBuffer"      # the runtime's device-to-device copy, whose true traffic is its size


def traffic_from_counters(fetch_csv, write_csv, kernel_substring, copy_bytes):
    """HBM bytes per launch of the kernel named `kernel_substring`, from two `rocprofv3 --pmc` runs of this same command
    with --copy-calibration (FETCH_SIZE in one, WRITE_SIZE in the other; both count KiB per dispatch).  Each counter is
    scaled by what it reads for the calibration copy of `copy_bytes` bytes.  Returns (bytes, details)."""
    import csv

    def per_kernel(path, counter):
        kernel, copy = [], []
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] != counter:
                    continue
                if kernel_substring in row["Kernel_Name"]:
                    kernel.append(float(row["Counter_Value"]))
                elif COPY_KERNEL in row["Kernel_Name"]:
                    copy.append(float(row["Counter_Value"]))
        if not kernel or not copy:
            raise SystemExit(f"{path}: no {counter} rows for '{kernel_substring}' and the calibration copy")
        # the calibration copy is the largest copy of the run
        return sum(kernel) / len(kernel), max(copy)

    true_kib = copy_bytes / 1024.0
    fetch, fetch_copy = per_kernel(fetch_csv, "FETCH_SIZE")
    write, write_copy = per_kernel(write_csv, "WRITE_SIZE")
    f_scale, w_scale = true_kib / fetch_copy, true_kib / write_copy
    total = int(round((fetch * f_scale + write * w_scale) * 1024.0))
    return total, {"fetch_kib_per_dispatch": fetch, "write_kib_per_dispatch": write, "fetch_scale": round(f_scale, 4),
                   "write_scale": round(w_scale, 4), "calibration_copy_bytes": copy_bytes}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def q8_bytes(out_w, in_w):
    return out_w * (in_w // 32) * 34


def stats(samples, digits=4):
    """Mean, standard deviation (n - 1), extremes and count of a list of timings, beside the median the text quotes."""
    a = np.asarray(samples, dtype=np.float64)
    return {"median": round(float(np.median(a)), digits), "mean": round(float(a.mean()), digits),
            "sd": round(float(a.std(ddof=1)) if a.size > 1 else 0.0, digits), "min": round(float(a.min()), digits),
            "max": round(float(a.max()), digits), "n": int(a.size)}


def timed_each(lane, fn, reps):
    """Device time of each of `reps` consecutive calls of fn (an event after every call), and of all of them."""
    events = [lane.event() for _ in range(reps + 1)]
    lane.synchronize()
    events[0].record()
    for i in range(reps):
        fn()
        events[i + 1].record()
    lane.synchronize()
    each = [lane.elapsed_ms(events[i], events[i + 1]) for i in range(reps)]
    total = lane.elapsed_ms(events[0], events[reps])
    for e in events:
        e.dispose()
    return each, total


def timed(lane, fn, reps):
    """Device time of `reps` calls of fn on the lane's stream (HIP events), plus host wall time around a sync."""
    e0, e1 = lane.event(), lane.event()
    lane.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    ms = lane.elapsed_ms(e0, e1)
    lane.synchronize()
    wall = (time.perf_counter() - t0) * 1e3
    e0.dispose()
    e1.dispose()
    return ms, wall


def run_decode27b(args, lane, nn, oracle):
    from nntrain_amd.native import MatvecDesc
    from nntrain_amd.synth import DeviceSynth, decode27b_tensors
    tensors = decode27b_tensors()
    total_bytes = sum(q8_bytes(o, i) for _, o, i in tensors)
    assert total_bytes == 28_695_625_728, total_bytes
    synth = DeviceSynth()
    log(f"[decode27b] generating {len(tensors)} Q8_0 tensors, {total_bytes / 1e9:.2f} GB, on the device")
    weights, xs, ys = [], [], []
    for t, (name, out_w, in_w) in enumerate(tensors):
        w = lane.allocate_bytes(q8_bytes(out_w, in_w))
        synth.q8_0(lane, w, out_w * (in_w // 32), 3000 + t)
        x = lane.allocate(in_w)
        synth.normal(lane, x, in_w, 3999_000 + t)
        y = lane.allocate(out_w)
        weights.append(w)
        xs.append(x)
        ys.append(y)
    lane.synchronize()
    lib, h = lane._lib, lane._handle

    descs = (MatvecDesc * len(tensors))()
    for t, (name, out_w, in_w) in enumerate(tensors):
        descs[t] = MatvecDesc(xs[t].ptr, weights[t].ptr, None, ys[t].ptr, nn.GGML_Q8_0, 1, in_w, out_w)

    def token_forward():
        for t, (name, out_w, in_w) in enumerate(tensors):
            rc = lib.nnhip_quant_matvec(h, nn.GGML_Q8_0, c_void_p(xs[t].ptr), c_void_p(weights[t].ptr), None,
                                        c_void_p(ys[t].ptr), 1, in_w, out_w)
            if rc:
                nn.native.check(rc, "quant_matvec")

    def token_batch():
        nn.native.check(lib.nnhip_quant_matvec_batch(h, descs, len(tensors)), "quant_matvec_batch")

    graph = None
    if args.mode == "graph":
        lane.graph_begin()
        token_forward()
        graph = lane.graph_end()

    def token():
        if args.mode == "forward":
            token_forward()
        elif args.mode == "batch":
            token_batch()
        else:
            lane.graph_launch(graph)

    def verify(tag):
        """Sampled parity against the float64 oracle on the bytes that are actually in HBM."""
        worst = 0.0
        for t in (0, 3, 6, len(tensors) - 1):
            name, out_w, in_w = tensors[t]
            rows = min(out_w, 256)
            row_bytes = (in_w // 32) * 34
            x = lane.read(xs[t], np.float32)
            y = lane.read(ys[t], np.float32)
            for r0 in (0, out_w - rows):
                raw = lane.read(weights[t], np.uint8, rows * row_bytes, r0 * row_bytes)
                ref, _ = oracle.linear_f64(nn.GGML_Q8_0, raw, x, None, 1, in_w, rows)
                worst = max(worst, oracle.rel_l2(y[r0:r0 + rows], ref[0]))
        log(f"[decode27b] parity {tag}: worst sampled rel-L2 vs float64 oracle = {worst:.3e}")
        if not worst <= 1e-5:
            raise SystemExit(f"parity failure ({tag}): rel-L2 {worst:.3e} > 1e-5")
        return worst

    calibration_bytes = weights[-1].nbytes
    if args.copy_calibration:
        # a plain device-to-device copy of known size, so that a counter run (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)
        # of this same command can scale the counters by what they read for it
        n = weights[-1].nbytes
        scratch = lane.allocate_bytes(n)
        lane.copy(scratch, weights[-1], n)
        lane.synchronize()
        scratch.dispose()
        log(f"[decode27b] calibration copy of {n} bytes done")
    for _ in range(max(args.warmup, 1)):
        token()
    lane.synchronize()
    rel = verify("before timing")
    launches_before = lane.counters()["kernel_launches"]
    ms, wall = timed(lane, token, args.steps)
    launches_per_token = (lane.counters()["kernel_launches"] - launches_before) // args.steps
    # the same number of steps once more with an event after every step, for their spread (the figure above stays the
    # one pair of events around all of them)
    each_ms, _ = timed_each(lane, token, args.steps)
    rel = max(rel, verify("after timing"))
    # The dominant kernel on its own: in batch mode the library launches once per row length; the 5376-wide matrices
    # (q, k, v, gate, up of every layer and the head: 68 % of the bytes) are one launch of the matrix-core mat-vec.
    dominant = None
    if args.mode == "batch":
        idx = [t for t, (_, _, in_w) in enumerate(tensors) if in_w == 5376]
        sub = (MatvecDesc * len(idx))(*[descs[t] for t in idx])
        sub_bytes = sum(q8_bytes(tensors[t][1], tensors[t][2]) for t in idx)

        def sub_batch():
            nn.native.check(lib.nnhip_quant_matvec_batch(h, sub, len(idx)), "quant_matvec_batch")

        for _ in range(2):
            sub_batch()
        lane.synchronize()
        before = lane.counters()["kernel_launches"]
        sub_each, sub_ms = timed_each(lane, sub_batch, args.steps)
        assert (lane.counters()["kernel_launches"] - before) == args.steps, "the 5376-wide group is one launch"
        dominant = {"ms": sub_ms / args.steps, "bytes": sub_bytes, "stats": stats(sub_each)}
        log(f"[decode27b] dominant launch (311 matrices of row length 5376, {sub_bytes} bytes): "
            f"{dominant['ms']:.3f} ms, {sub_bytes / dominant['ms'] / 1e6:.0f} GB/s")
        token()             # (the full table again, for whatever runs next)
        lane.synchronize()
    ms_per_step = ms / args.steps
    tok_s = 1e3 / ms_per_step
    gbs = total_bytes / (ms_per_step * 1e-3) / 1e9
    log(f"[decode27b] {ms_per_step:.3f} ms/token (device events), wall {wall / args.steps:.3f} ms/token, "
        f"{tok_s:.1f} tok/s, {gbs:.0f} GB/s")

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline_decode(lane, nn, oracle, tensors, weights, xs)
    if graph is not None:
        lane.graph_destroy(graph)
    for b in weights + xs + ys:
        b.dispose()
    # batch mode: the library groups the 435 matrices by row length (5376, 4096, 21504) and launches the matrix-core
    # mat-vec once per group; the figures below are per launch on average (a third of the token's bytes and time each)
    n_launch = len(tensors) if args.mode != "batch" else launches_per_token
    batch_kernel = "matvec_mfma_wide_kernel<Q8_0Task, 2, 8, 1, true, false>"
    traffic = None
    if args.traffic_from:
        if args.mode != "batch":
            raise SystemExit("--traffic-from applies to --mode batch")
        # (the counter runs hold this kernel's launches of the whole token only: every dispatch of it is the 5376 group)
        traffic, detail = traffic_from_counters(args.traffic_from[0], args.traffic_from[1], "Q8_0Task, 2, 8, 1, true", calibration_bytes)
        log(f"[decode27b] HBM traffic per launch of the dominant kernel from counters: {traffic} bytes ({detail})")
    if dominant:
        roof_gbs, roof_bytes = dominant["bytes"] / dominant["ms"] / 1e6, dominant["bytes"]
        roof_extra = {"launch_ms": round(dominant["ms"], 4), "launch_ms_stats": dominant["stats"],
                      "note": "the launch for the 311 matrices of row length 5376 (68 % of the token's bytes), timed on its own "
                              "with HIP events; the 4096- and 21504-wide groups are launches of <Q8_0Task, 1, 5, 1, false, false>",
                      "whole_token_gb_per_s": round(gbs, 1)}
    else:
        roof_gbs, roof_bytes, roof_extra = gbs, total_bytes // n_launch, {}
    return {
        "metric": "27B-shape Q8_0 decode tokens/sec", "value": round(tok_s, 2), "unit": "tokens/s",
        "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_stats": stats(each_ms),
        "config": {"workload": "decode27b: 435 Q8_0 mat-vecs of a Gemma-3-27B-shaped stack (the headline configuration), "
                               "28,695,625,728 weight bytes/token resident in HBM, batch 1, fp32 activations",
                   "launch": args.mode, "launches_per_token": n_launch},
        "roofline": {"bound": "hbm", "achieved": round(roof_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(roof_gbs / HBM_PEAK_GBS, 4),
                     "traffic": traffic,
                     "kernel": batch_kernel if args.mode == "batch" else "matvec_rowstep_kernel<Q8_0Unit>",
                     "bytes_per_launch": roof_bytes, **roof_extra},
        "cpu_baseline": cpu,
        "parity": {"rel_l2_vs_f64_oracle_sampled": rel, "bar": 1e-5},
    }


def cpu_leg(oracle, typ, w_host, x_host, in_w, out_w, budget_s):
    """The CPU restatement of the reference's operator (dequantize row + sequential FP32 FMA, Tensor.QwenQuantized.cs:
    113-165) on one matrix, compiled for this host: all threads for about budget_s seconds, then one thread on the
    first rows.  Returns seconds per pass (all threads), seconds per pass extrapolated from one thread, thread count."""
    threads = oracle.max_threads()
    reps, spent = 0, 0.0
    t_begin = time.perf_counter()
    while spent < budget_s or reps < 2:
        oracle.cpu_linear(typ, w_host, x_host, None, 1, in_w, out_w, threads, native=True)
        reps += 1
        spent = time.perf_counter() - t_begin
    per_pass = spent / reps
    rows1 = max(1, min(out_w, int(out_w * min(1.0, 0.5 / max(per_pass * threads, 1e-9)))))
    row_bytes = w_host.size // out_w
    t_begin = time.perf_counter()
    oracle.cpu_linear(typ, w_host[:rows1 * row_bytes], x_host, None, 1, in_w, rows1, 1, native=True)
    one = (time.perf_counter() - t_begin) * out_w / rows1
    return per_pass, one, threads, reps


def cpu_baseline_decode(lane, nn, oracle, tensors, weights, xs):
    """One layer's seven matrices through cpu_leg; the token rate is extrapolated by bytes to the whole set."""
    sample = list(range(7))
    sample_bytes = sum(q8_bytes(tensors[t][1], tensors[t][2]) for t in sample)
    total_bytes = sum(q8_bytes(o, i) for _, o, i in tensors)
    per_layer = one_layer = 0.0
    passes = []
    for t in sample:
        name, out_w, in_w = tensors[t]
        per_pass, one, threads, reps = cpu_leg(oracle, nn.GGML_Q8_0, lane.read(weights[t], np.uint8), lane.read(xs[t], np.float32),
                                               in_w, out_w, 1.5)
        per_layer += per_pass
        one_layer += one
        passes.append(reps)
    tok_s = 1.0 / (per_layer * total_bytes / sample_bytes)
    tok_s_one = 1.0 / (one_layer * total_bytes / sample_bytes)
    log(f"[cpu_baseline] {threads} threads: layer sample {per_layer * 1e3:.1f} ms ({sample_bytes / per_layer / 1e9:.1f} GB/s)"
        f" -> {tok_s:.3f} tok/s extrapolated; one thread {tok_s_one:.4f} tok/s")
    return {"value": round(tok_s, 4), "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"layer 0's seven Q8_0 matrices ({sample_bytes} bytes), {min(passes)}-{max(passes)} passes each; token "
                      f"rate extrapolated by weight bytes to the 435-matrix set",
            "gb_per_s": round(sample_bytes / per_layer / 1e9, 2),
            "one_thread": {"value": round(tok_s_one, 5), "gb_per_s": round(sample_bytes / one_layer / 1e9, 3),
                           "sample": "the first rows of the same matrices, extrapolated by rows"},
            "cpu_model": oracle.cpu_model(), "host_threads_available": os.cpu_count(), "build": oracle.native_lib()[1]}


GEMV_CONFIGS = [
    ("cfg1 Q8_0 21504x5376", "GGML_Q8_0", 5376, 21504, 1001, 1002),
    ("cfg2 Q4_K 17408x5120", "GGML_Q4_K", 5120, 17408, 2001, 2000),
    ("cfg2 Q5_K 17408x5120", "GGML_Q5_K", 5120, 17408, 2002, 2000),
    ("cfg2 Q6_K 17408x5120", "GGML_Q6_K", 5120, 17408, 2003, 2000),
    ("cfg5 IQ2_S 5120x17408", "GGML_IQ2_S", 17408, 5120, 5001, 5002),
    ("cfg5 shape in IQ3_S 5120x17408", "GGML_IQ3_S", 17408, 5120, 5003, 5002),
    ("down projection Q4_K 5120x17408", "GGML_Q4_K", 17408, 5120, 2004, 2005),
]
MATRIX_CORE_TYPES = ("GGML_Q8_0", "GGML_Q4_K", "GGML_Q5_K", "GGML_Q6_K", "GGML_IQ2_S", "GGML_IQ3_S")


def run_gemv(args, lane, nn, oracle):
    """Single-matrix decode mat-vecs.  Weights rotate through copies totalling >= 1 GB so every launch streams from
    HBM rather than from the 256 MB Infinity Cache; the cache-resident figure is reported beside it, and so is the
    sustained rate when all the copies go through one batched launch."""
    from nntrain_amd import synth
    from nntrain_amd.native import MatvecDesc
    out = {}
    lib, h = lane._lib, lane._handle
    for name, tname, in_w, out_w, wseed, xseed in GEMV_CONFIGS:
        typ = getattr(nn, tname)
        payload = synth.matrix(typ, out_w, in_w, wseed)
        x_host = synth.activations(1, in_w, xseed)
        nbytes = payload.size
        copies = max(2, int(np.ceil(1.0e9 / nbytes)))
        w0 = lane.upload_raw(payload)
        ring = [w0]
        for _ in range(copies - 1):
            b = lane.allocate_bytes(nbytes)
            lane.copy(b, w0, nbytes)
            ring.append(b)
        x = lane.upload_raw(x_host)
        y = lane.allocate(out_w)

        def launch(w):
            rc = lib.nnhip_quant_matvec(h, typ, c_void_p(x.ptr), c_void_p(w.ptr), None, c_void_p(y.ptr), 1, in_w, out_w)
            if rc:
                nn.native.check(rc, "quant_matvec")

        for w in ring:
            launch(w)
        lane.synchronize()
        ref, _ = oracle.linear_f64(typ, payload, x_host, None, 1, in_w, out_w)
        rel = oracle.rel_l2(lane.read(y, np.float32), ref[0])
        if not rel <= 1e-5:
            raise SystemExit(f"{name}: parity failure, rel-L2 {rel:.3e}")
        samples_ring, samples_same = [], []
        for _ in range(9):
            ms, _ = timed(lane, lambda: [launch(w) for w in ring], 1)
            samples_ring.append(ms * 1e3 / len(ring))
            ms, _ = timed(lane, lambda: [launch(w0) for _ in ring], 1)
            samples_same.append(ms * 1e3 / len(ring))
        us_ring, us_same = float(np.median(samples_ring)), float(np.median(samples_same))
        launch(w0)
        rel_after = oracle.rel_l2(lane.read(y, np.float32), ref[0])
        if not rel_after <= 1e-5:
            raise SystemExit(f"{name}: parity failure after timing, rel-L2 {rel_after:.3e}")
        rel = max(rel, rel_after)
        algo = nbytes + 4 * in_w + 4 * out_w
        # sustained rate: the same mat-vec over every rotated copy as ONE batched launch (no per-launch start-up)
        ys = [lane.allocate(out_w) for _ in ring]
        descs = (MatvecDesc * len(ring))()
        for i, w in enumerate(ring):
            descs[i] = MatvecDesc(x.ptr, w.ptr, None, ys[i].ptr, typ, 1, in_w, out_w)
        nn.native.check(lib.nnhip_quant_matvec_batch(h, descs, len(ring)), "quant_matvec_batch")
        lane.synchronize()
        # large Q8_0 / Q4_K / Q5_K / Q6_K / IQ2_S groups run on the matrix-core kernels (fixed-point activations): same bar against
        # the oracle, not the single launch's bits; the other formats share the single launch's kernel and must match bitwise
        y_batch = lane.read(ys[-1], np.float32)
        rel_batch = oracle.rel_l2(y_batch, ref[0])
        if not rel_batch <= 1e-5:
            raise SystemExit(f"{name}: batched launch parity failure, rel-L2 {rel_batch:.3e}")
        if tname not in MATRIX_CORE_TYPES and not np.array_equal(y_batch.view(np.uint32), lane.read(y, np.uint32)):
            raise SystemExit(f"{name}: batched launch differs bitwise from the single launch")
        samples_batch = []
        for _ in range(7):
            ms, _ = timed(lane, lambda: nn.native.check(lib.nnhip_quant_matvec_batch(h, descs, len(ring)), "batch"), 1)
            samples_batch.append(ms * 1e3 / len(ring))
        us_batch = float(np.median(samples_batch))
        rel_batch_after = oracle.rel_l2(lane.read(ys[0], np.float32), ref[0])
        if not rel_batch_after <= 1e-5:
            raise SystemExit(f"{name}: batched launch parity failure after timing, rel-L2 {rel_batch_after:.3e}")
        rel_batch = max(rel_batch, rel_batch_after)
        out[name] = {"us_per_launch_hbm": round(us_ring, 2), "us_per_launch_hbm_stats": stats(samples_ring, 2),
                     "us_per_launch_cache_resident_stats": stats(samples_same, 2),
                     "sustained_us_per_matvec_batched_stats": stats(samples_batch, 2), "gb_per_s_hbm": round(algo / us_ring / 1e3, 1),
                     "frac_of_8TBs": round(algo / us_ring / 1e3 / HBM_PEAK_GBS, 4),
                     "us_per_launch_cache_resident": round(us_same, 2),
                     "sustained_us_per_matvec_batched": round(us_batch, 2),
                     "sustained_gb_per_s_batched": round(algo / us_batch / 1e3, 1),
                     "sustained_frac_of_8TBs": round(algo / us_batch / 1e3 / HBM_PEAK_GBS, 4),
                     "algorithmic_bytes": algo, "rel_l2_vs_f64_oracle": rel, "rel_l2_batched_vs_f64_oracle": rel_batch,
                     "weight_copies_rotated": len(ring)}
        log(f"[gemv] {name}: single launch {us_ring:.2f} us ({algo / us_ring / 1e3:.0f} GB/s, "
            f"{100 * algo / us_ring / 1e3 / HBM_PEAK_GBS:.1f}% of 8 TB/s) HBM, {us_same:.2f} us cache-resident; batched "
            f"{us_batch:.2f} us/mat-vec ({100 * algo / us_batch / 1e3 / HBM_PEAK_GBS:.1f}%); rel-L2 {rel:.2e}")
        if not args.no_cpu_baseline:
            per_pass, one, threads, _ = cpu_leg(oracle, typ, payload, x_host, in_w, out_w, 1.0)
            out[name]["cpu_baseline"] = {"gb_per_s": round(nbytes / per_pass / 1e9, 2), "us_per_matvec": round(per_pass * 1e6, 1),
                                         "cores": threads, "one_thread_gb_per_s": round(nbytes / one / 1e9, 3), "kind": "port"}
            log(f"[gemv] {name}: CPU port {nbytes / per_pass / 1e9:.1f} GB/s on {threads} threads, {nbytes / one / 1e9:.2f} GB/s on one")
        if tname == "GGML_Q8_0" or name.startswith("cfg2") or name.startswith("cfg5") or name.startswith("down"):
            # several input rows in one call (weights rotated as above): microseconds per call, up to four rows sharing a
            # pass over the weights (Q8_0 with two rows: its row-tiled lane-per-unit kernel; otherwise the matrix cores)
            per_rows = {}
            for rows in (2, 4, 8, 16):
                xr = lane.upload_raw(synth.activations(rows, in_w, xseed + rows))
                yr = lane.allocate(rows * out_w)

                def launch_rows(w):
                    nn.native.check(lib.nnhip_quant_matvec(h, typ, c_void_p(xr.ptr), c_void_p(w.ptr), None, c_void_p(yr.ptr),
                                                           rows, in_w, out_w), "quant_matvec")

                for w in ring:
                    launch_rows(w)
                samples = []
                for _ in range(5):
                    ms, _ = timed(lane, lambda: [launch_rows(w) for w in ring], 1)
                    samples.append(ms * 1e3 / len(ring))
                per_rows[f"rows={rows}"] = round(float(np.median(samples)), 2)
                per_rows[f"rows={rows} stats"] = stats(samples, 2)
                # every input row against the oracle, after the timing
                xr_host = synth.activations(rows, in_w, xseed + rows)
                ref_rows, _ = oracle.linear_f64(typ, payload, xr_host, None, rows, in_w, out_w)
                rel_rows = oracle.rel_l2(lane.read(yr, np.float32).reshape(rows, out_w), ref_rows)
                if not rel_rows <= 1e-5:
                    raise SystemExit(f"{name}: parity failure with {rows} input rows, rel-L2 {rel_rows:.3e}")
                xr.dispose()
                yr.dispose()
            out[name]["us_per_call_with_several_input_rows"] = per_rows
            log(f"[gemv] {name}: " + ", ".join(f"{k} {v:.1f} us" for k, v in per_rows.items() if not k.endswith("stats")))
        for b in ring + ys + [x, y]:
            b.dispose()
    return out


def run_ffn(args, lane, nn, oracle):
    """Feed-forward half of a decode layer (hidden += attention; n = RMSNorm(hidden); hidden += W_down(SiLU(W_gate n) *
    W_up n), NNtrain.Core/Modules/Qwen35QuantizedModel.cs:486-498) at hidden 5120 / feed-forward 17408 in Q4_K: the six
    launches the reference issues against the three fused ones.  Eight layers' weights rotate (1.2 GB) so they stream
    from HBM.  Both forms end in the same bits."""
    from nntrain_amd import synth
    from nntrain_amd.native import FusedMatvecDesc, PRE_RMS_NORM, PRE_SILU_MULTIPLY
    import ctypes
    typ, width, ffn, layers, eps = nn.GGML_Q4_K, 5120, 17408, 8, 1e-6
    lib, h, chk = lane._lib, lane._handle, nn.native.check
    up = lane.upload_raw
    base = {"gate": up(synth.matrix(typ, ffn, width, 11)), "up": up(synth.matrix(typ, ffn, width, 12)),
            "down": up(synth.matrix(typ, width, ffn, 13))}
    weights = [base]
    for _ in range(layers - 1):
        layer = {}
        for k, b in base.items():
            layer[k] = lane.allocate_bytes(b.nbytes)
            lane.copy(layer[k], b, b.nbytes)
        weights.append(layer)
    rng = np.random.default_rng(5)
    hidden0 = (rng.standard_normal(width) * 2).astype(np.float32)
    attn, gamma = up(rng.standard_normal(width).astype(np.float32)), up(rng.uniform(0.5, 1.5, width).astype(np.float32))
    hid, hid2, norm, g, u, act, down = (lane.allocate(n) for n in (width, width, width, ffn, ffn, ffn, width))
    P = lambda b: c_void_p(b.ptr) if b is not None else None                     # noqa: E731

    def matvec(w, x, y, in_w, out_w):
        chk(lib.nnhip_quant_matvec(h, typ, P(x), P(w), None, P(y), 1, in_w, out_w), "quant_matvec")

    def fused(w, in_w, out_w, **kw):
        d = FusedMatvecDesc(struct_size=ctypes.sizeof(FusedMatvecDesc), ggml_type=typ, w=P(w), in_w=in_w, out_w=out_w,
                            **{k: (P(v) if hasattr(v, "ptr") else v) for k, v in kw.items()})
        chk(lib.nnhip_quant_matvec_fused(h, ctypes.byref(d)), "quant_matvec_fused")

    def layer_unfused(w):
        chk(lib.nnhip_add_rms_norm(h, P(hid), P(attn), P(gamma), P(norm), 1, width, width, eps), "add_rms_norm")
        matvec(w["gate"], norm, g, width, ffn)
        matvec(w["up"], norm, u, width, ffn)
        chk(lib.nnhip_silu_multiply(h, P(g), P(u), P(act), ffn), "silu_multiply")
        matvec(w["down"], act, down, ffn, width)
        chk(lib.nnhip_add_in_place(h, P(hid), P(down), width), "add_in_place")

    state = {"cur": hid, "nxt": hid2}

    def layer_fused(w):
        cur, nxt = state["cur"], state["nxt"]
        fused(w["gate"], width, ffn, pre_op=PRE_RMS_NORM, x=cur, x2=attn, norm_weight=gamma, epsilon=eps, x_out=norm, sum_out=nxt, y=g)
        matvec(w["up"], norm, u, width, ffn)
        fused(w["down"], ffn, width, pre_op=PRE_SILU_MULTIPLY, x=g, x2=u, addend=nxt, y=nxt)
        state["cur"], state["nxt"] = nxt, cur

    # gate and up stacked into one matrix: two launches per layer
    stacked = []
    for w in weights:
        b = lane.allocate_bytes(w["gate"].nbytes + w["up"].nbytes)
        lane.copy(b, w["gate"], w["gate"].nbytes)
        lane.copy(b, w["up"], w["up"].nbytes, dst_offset=w["gate"].nbytes)
        stacked.append({"gate_up": b, "down": w["down"]})
    gu = lane.allocate(2 * ffn)
    gu_up = gu.view(4 * ffn, 4 * ffn)

    def layer_stacked(w):
        cur, nxt = state["cur"], state["nxt"]
        fused(w["gate_up"], width, 2 * ffn, pre_op=PRE_RMS_NORM, x=cur, x2=attn, norm_weight=gamma, epsilon=eps, sum_out=nxt, y=gu)
        fused(w["down"], ffn, width, pre_op=PRE_SILU_MULTIPLY, x=gu, x2=gu_up, addend=nxt, y=nxt)
        state["cur"], state["nxt"] = nxt, cur

    results = {}
    spread = {}
    finals = {}
    for name, fn in (("unfused_6_launches", layer_unfused), ("fused_3_launches", layer_fused), ("fused_2_launches_gate_up_stacked", None)):
        lane.write(hid, hidden0)
        state["cur"], state["nxt"] = hid, hid2
        seq = weights
        if fn is None:
            fn, seq = layer_stacked, stacked
        for w in seq:
            fn(w)
        lane.synchronize()
        finals[name] = lane.read(state["cur"] if name.startswith("fused") else hid, np.uint32)
        samples = []
        for _ in range(9):
            ms, _ = timed(lane, lambda: [fn(w) for w in seq], 1)
            samples.append(ms * 1e3 / layers)
        results[name] = round(float(np.median(samples)), 2)
        spread[name] = stats(samples, 2)
    if any(not np.array_equal(finals["unfused_6_launches"], f) for f in finals.values()):
        raise SystemExit("ffn: fused and unfused layers differ bitwise")
    wbytes = sum(b.nbytes for b in base.values())
    out = {"config": "Q4_K, hidden 5120, feed-forward 17408, 8 layers' weights rotated", "us_per_layer": results, "us_per_layer_stats": spread,
           "weight_bytes_per_layer": wbytes,
           "gb_per_s_fused": round(wbytes / results["fused_2_launches_gate_up_stacked"] / 1e3, 1),
           "gb_per_s_unfused": round(wbytes / results["unfused_6_launches"] / 1e3, 1), "bitwise_equal": True}
    log(f"[ffn] per layer: unfused {results['unfused_6_launches']:.2f} us, fused {results['fused_3_launches']:.2f} us, "
        f"gate+up stacked {results['fused_2_launches_gate_up_stacked']:.2f} us "
        f"({wbytes / results['fused_2_launches_gate_up_stacked'] / 1e3:.0f} GB/s)")
    return out


def run_decode_loop(args, lane, nn, oracle):
    """Per-token timing of the decode loop (nntrain_amd.decoder) over a synthetic llama-style GGUF file written to a
    temporary directory and loaded through the streaming loader: 4 layers of hidden 5120 / feed-forward 17408 / 40 query
    and 8 key-value heads of 128 in Q4_K, vocabulary 32000.  Three forms of the same step, same bits: one launch per
    operation (the reference's sequence), the fused launches, and the fused launches replayed from a HIP graph."""
    import struct
    import tempfile
    from nntrain_amd import synth
    from nntrain_amd.decoder import QuantizedDecoder
    layers, emb, ffn, heads, kv, hw, vocab, typ = 4, 5120, 17408, 40, 8, 128, 32000, nn.GGML_Q4_K

    def kvp(key, value):
        if isinstance(value, str):
            b = value.encode()
            return key, 8, struct.pack("<Q", len(b)) + b
        return (key, 6, struct.pack("<f", value)) if isinstance(value, float) else (key, 4, struct.pack("<I", value))

    tensors = []
    rng = np.random.default_rng(8)

    def mat(name, out_w, in_w, seed):
        tensors.append((name, (in_w, out_w), typ, synth.matrix(typ, out_w, in_w, seed)))

    def vec(name):
        tensors.append((name, (emb,), 0, rng.uniform(0.5, 1.5, emb).astype(np.float32)))

    mat("token_embd.weight", vocab, emb, 1)
    for i in range(layers):
        p = f"blk.{i}."
        vec(p + "attn_norm.weight")
        mat(p + "attn_q.weight", heads * hw, emb, 10 + i)
        mat(p + "attn_k.weight", kv * hw, emb, 20 + i)
        mat(p + "attn_v.weight", kv * hw, emb, 30 + i)
        mat(p + "attn_output.weight", emb, heads * hw, 40 + i)
        vec(p + "ffn_norm.weight")
        mat(p + "ffn_gate.weight", ffn, emb, 50 + i)
        mat(p + "ffn_up.weight", ffn, emb, 60 + i)
        mat(p + "ffn_down.weight", emb, ffn, 70 + i)
    vec("output_norm.weight")
    mat("output.weight", vocab, emb, 2)
    kvs = [kvp("general.architecture", "llama"), kvp("llama.block_count", layers), kvp("llama.embedding_length", emb),
           kvp("llama.feed_forward_length", ffn), kvp("llama.attention.head_count", heads),
           kvp("llama.attention.head_count_kv", kv), kvp("llama.attention.key_length", hw),
           kvp("llama.attention.layer_norm_rms_epsilon", 1e-6)]

    def s(x):
        b = x.encode()
        return struct.pack("<Q", len(b)) + b

    out = {}
    with tempfile.TemporaryDirectory() as tmp:
        # GGUF v3, tensor data aligned to 32 bytes
        offsets, cursor = [], 0
        for _, _, _, payload in tensors:
            offsets.append(cursor)
            cursor = (cursor + payload.nbytes + 31) // 32 * 32
        head = struct.pack("<IIQQ", 0x46554747, 3, len(tensors), len(kvs))
        for k, t, v in kvs:
            head += s(k) + struct.pack("<I", t) + v
        for (name, shape, ttype, _), off in zip(tensors, offsets):
            head += s(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape) + struct.pack("<IQ", ttype, off)
        data_start = (len(head) + 31) // 32 * 32
        path = os.path.join(tmp, "synthetic.gguf")
        with open(path, "wb") as f:
            f.write(head + b"\0" * (data_start - len(head)))
            for (_, _, _, payload), off in zip(tensors, offsets):
                f.seek(data_start + off)
                f.write(payload.tobytes())
        file_bytes = os.path.getsize(path)
        del tensors
        t0 = time.perf_counter()
        with nn.GgufReader(path) as reader:
            plain = QuantizedDecoder(lane, reader, fused=False)
            load_s = time.perf_counter() - t0
            fused = QuantizedDecoder(lane, reader, fused=True)
        lane.synchronize()
    weight_bytes = plain.quantized_bytes - plain.embedding.storage_bytes      # streamed per token (the embedding is one row)
    tokens = [3, 1000, 31999, 17, 4242, 9, 30000, 512]
    ref = [lane.read(plain.forward_token(t), np.uint32, count=vocab) for t in tokens[:2]]
    for t, r in zip(tokens[:2], ref):
        if not np.array_equal(lane.read(fused.forward_token(t), np.uint32, count=vocab), r):
            raise SystemExit("decode loop: fused and unfused logits differ bitwise")

    def per_token(dec, label):
        samples = []
        for _ in range(5):
            ms, _ = timed(lane, lambda: [dec.forward_token(t) for t in tokens], 1)
            samples.append(ms / len(tokens))
        spread[label] = stats(samples)
        return float(np.median(samples))

    spread = {}
    ms_plain, ms_fused = per_token(plain, "one_launch_per_operation"), per_token(fused, "fused_launches")
    fused.capture_graph()
    if not np.array_equal(lane.read(fused.forward_token(tokens[0]), np.uint32, count=vocab), ref[0]):
        raise SystemExit("decode loop: graph replay differs bitwise")
    ms_graph = per_token(fused, "fused_launches_hip_graph")
    if not np.array_equal(lane.read(fused.forward_token(tokens[1]), np.uint32, count=vocab), ref[1]):
        raise SystemExit("decode loop: graph replay differs bitwise after timing")
    toks, timing = fused.generate(5, 16)
    out = {"config": f"llama-style, {layers} layers, hidden {emb}, feed-forward {ffn}, heads {heads}/{kv} x {hw}, vocabulary {vocab}, Q4_K",
           "gguf_file_bytes": file_bytes, "load_seconds_file_to_hbm": round(load_s, 2),
           "weight_bytes_streamed_per_token": weight_bytes,
           "ms_per_token": {"one_launch_per_operation": round(ms_plain, 4), "fused_launches": round(ms_fused, 4),
                            "fused_launches_hip_graph": round(ms_graph, 4)},
           "ms_per_token_stats": spread,
           "launches_per_token": {"one_launch_per_operation": 1 + 12 * layers + 2, "fused_launches": 1 + 4 * layers + 1},
           "gb_per_s_fused_graph": round(weight_bytes / ms_graph / 1e6, 1),
           "frac_of_8TBs_fused_graph": round(weight_bytes / ms_graph / 1e6 / HBM_PEAK_GBS, 4),
           "greedy_generation_with_host_argmax": {"tokens": timing.generated_tokens,
                                                  "first_token_ms": round(timing.first_token_milliseconds, 3),
                                                  "decode_tokens_per_s": round(timing.decode_tokens_per_second, 1)},
           "bitwise_equal": True}
    log(f"[decode_loop] per token: {ms_plain * 1e3:.1f} us unfused, {ms_fused * 1e3:.1f} us fused, {ms_graph * 1e3:.1f} us fused + graph "
        f"({weight_bytes / ms_graph / 1e6:.0f} GB/s); load {load_s:.1f} s for {file_bytes / 1e9:.2f} GB")
    plain.dispose()
    fused.dispose()
    return out


def run_decode27b_chained(args, lane, nn, oracle):
    """The 27B-shape Q8_0 token in its real dependency order: the decode loop of nntrain_amd.decoder (norm -> q|k|v ->
    first-token attention -> o -> norm -> gate|up -> SiLU product -> down -> ... -> head, NNtrain.Core/Modules/
    Qwen35QuantizedModel.cs:451-513) over the same 435 matrix shapes as the headline set, weights drawn on the device,
    the head tied to the embedding.  Every mat-vec consumes what the one before it produced, so nothing overlaps across
    launches: one launch per operation (the reference's sequence), the fused launches, and those replayed from a HIP
    graph.  All three end in the same logits bit for bit."""
    from nntrain_amd.decoder import DecoderDescriptor, QuantizedDecoder
    from nntrain_amd.synth import DeviceSynth
    d = DecoderDescriptor("gemma3-27b-shape", 62, 5376, 21504, 32, 16, 128, 1e-6, 262144)
    synth = DeviceSynth()
    def weights():
        seeds = iter(range(7000, 9000))

        def matrix(name, in_w, out_w):
            w = lane.allocate_bytes(q8_bytes(out_w, in_w))
            synth.q8_0(lane, w, out_w * (in_w // 32), next(seeds))
            return nn.HipQuantizedMatrix.from_device(lane, w, nn.GGML_Q8_0, out_w, in_w)

        def dense(name, width):
            import zlib
            return lane.upload_raw(np.random.default_rng(zlib.crc32(name.encode())).uniform(0.5, 1.5, width).astype(np.float32))

        return matrix, dense

    log("[decode27b_chained] generating two copies of the weights (one launch per operation / fused)")
    m1, d1 = weights()
    plain = QuantizedDecoder.from_weights(lane, d, m1, d1, has_output=False, fused=False)
    m2, d2 = weights()
    fused = QuantizedDecoder.from_weights(lane, d, m2, d2, has_output=False, fused=True)
    lane.synchronize()
    vocab = d.vocabulary
    weight_bytes = plain.quantized_bytes          # every matrix is streamed whole: the head is the tied embedding
    tokens = [3, 1000, 262143, 17]
    for t in tokens[:2]:
        a = lane.read(plain.forward_token(t), np.uint32, count=vocab)
        b = lane.read(fused.forward_token(t), np.uint32, count=vocab)
        if not np.array_equal(a, b):
            raise SystemExit("decode27b_chained: fused and unfused logits differ bitwise")
    # the head against the float64 oracle, from the hidden state the chain ended in
    hidden = lane.read(plain._hidden[plain._cur], np.float32).astype(np.float64)
    gamma = lane.read(plain.output_norm, np.float32).astype(np.float64)
    normed = (hidden / np.sqrt(np.mean(hidden * hidden) + d.rms_epsilon) * gamma).astype(np.float32)
    row_bytes = (d.embedding_length // 32) * 34
    raw = lane.read(plain.embedding.device_payload(lane), np.uint8, 256 * row_bytes, 0)
    ref, _ = oracle.linear_f64(nn.GGML_Q8_0, raw, normed, None, 1, d.embedding_length, 256)
    logits = lane.read(plain.logits, np.float32, count=256)
    rel = oracle.rel_l2(logits, ref[0])
    log(f"[decode27b_chained] head logits (first 256) vs float64 oracle from the final hidden state: rel-L2 {rel:.3e}")
    if not (np.all(np.isfinite(logits)) and rel <= 1e-4):       # the norm is recomputed here in float64: looser than 1e-5
        raise SystemExit(f"decode27b_chained: parity failure, rel-L2 {rel:.3e}")

    def per_token(dec, label):
        samples = []
        for _ in range(5):
            ms, _ = timed(lane, lambda: [dec.forward_token(t) for t in tokens], 1)
            samples.append(ms / len(tokens))
        spread[label] = stats(samples)
        return float(np.median(samples))

    spread = {}
    ms_plain, ms_fused = per_token(plain, "one_launch_per_operation"), per_token(fused, "fused_launches")
    fused.capture_graph()
    if not np.array_equal(lane.read(fused.forward_token(tokens[1]), np.uint32, count=vocab),
                          lane.read(plain.forward_token(tokens[1]), np.uint32, count=vocab)):
        raise SystemExit("decode27b_chained: graph replay differs bitwise")
    ms_graph = per_token(fused, "fused_launches_hip_graph")
    if not np.array_equal(lane.read(fused.forward_token(tokens[2]), np.uint32, count=vocab),
                          lane.read(plain.forward_token(tokens[2]), np.uint32, count=vocab)):
        raise SystemExit("decode27b_chained: graph replay differs bitwise after timing")

    def entry(ms):
        return {"ms_per_token": round(ms, 4), "tokens_per_s": round(1e3 / ms, 2), "gb_per_s": round(weight_bytes / ms / 1e6, 1),
                "frac_of_8TBs": round(weight_bytes / ms / 1e6 / HBM_PEAK_GBS, 4)}

    layers = d.layer_count
    out = {"config": "62 layers, hidden 5376, feed-forward 21504, heads 32/16 x 128, vocabulary 262144 (head tied to the "
                     "embedding), Q8_0, first-token attention (no cache)",
           "weight_bytes_streamed_per_token": weight_bytes,
           "one_launch_per_operation": entry(ms_plain), "fused_launches": entry(ms_fused),
           "fused_launches_hip_graph": entry(ms_graph), "ms_per_token_stats": spread,
           "launches_per_token": {"one_launch_per_operation": 1 + 12 * layers + 2, "fused_launches": 1 + 4 * layers + 1},
           "rel_l2_head_vs_f64_oracle": rel, "bitwise_equal": True}
    log(f"[decode27b_chained] per token: {ms_plain:.3f} ms one launch per operation, {ms_fused:.3f} ms fused, "
        f"{ms_graph:.3f} ms fused + graph ({weight_bytes / ms_graph / 1e6:.0f} GB/s, {1e3 / ms_graph:.1f} tok/s)")
    plain.dispose()
    fused.dispose()
    lane.trim()
    return out


def run_prefill(args, lane, nn, oracle):
    """Q4_K 17408x5120 bf16-MFMA prefill mat-mul at M = 128, 256, 512, 2048 (the prefill configuration of the benchmark list); the other formats
    the kernel decodes (Q5_K, Q6_K, Q8_0, IQ2_S, IQ3_S) at M = 512 under "other_formats"."""
    out = _prefill_of(lane, nn, oracle, nn.GGML_Q4_K, "Q4_K", (128, 256, 512, 2048))
    if out is not None:
        out["fp32_activations_three_products"] = _prefill_split(lane, nn, oracle, (128, 512))
        out["other_formats"] = {}
        for tname in ("Q5_K", "Q6_K", "Q8_0", "IQ2_S", "IQ3_S"):
            res = _prefill_of(lane, nn, oracle, getattr(nn, "GGML_" + tname), tname, (512,))
            if res is not None:
                out["other_formats"][tname] = res["M=512"]
    return out


def _prefill_split(lane, nn, oracle, ms_list):
    """The FP32-activation prefill at the reference's own accuracy gate (both operands as two bfloat16 parts, three
    products, nnhip_quant_matmul_split) beside the one-product entry with FP32 activations (nnhip_quant_matmul) and the
    FP32 mat-vec route the operator takes by default, on the Q4_K 17408 x 5120 matrix."""
    from nntrain_amd import synth
    typ, in_w, out_w = nn.GGML_Q4_K, 5120, 17408
    payload = synth.matrix(typ, out_w, in_w, 2001)
    out = {}
    for m in ms_list:
        x_host = synth.activations(m, in_w, 4100 + m)
        x = lane.upload_raw(x_host)
        y = lane.allocate(m * out_w)
        picked = np.arange(0, m, max(16, m // 32))
        ref, _ = oracle.linear_f64(typ, payload, np.ascontiguousarray(x_host[picked]), None, len(picked), in_w, out_w)
        # (against the product of the FP32 activations: the one-product entry rounds them too, which the 2e-3 of the
        # bfloat16-input figures above does not include)
        entry = {}
        for label, mode, bar in (("three_products", "split", 5e-5), ("one_product", True, 4e-3), ("mat_vec_passes", False, 1e-5)):
            mat = nn.HipQuantizedMatrix(payload, typ, out_w, in_w, inference_matmul_prefill=mode)
            mat.forward(lane, x, None, m, out=y)
            lane.synchronize()
            samples = []
            for _ in range(5 if mode is not False else 3):
                ms, _ = timed(lane, lambda: mat.forward(lane, x, None, m, out=y), 1)
                samples.append(ms)
            rel = oracle.rel_l2(lane.read(y, np.float32, m * out_w).reshape(m, out_w)[picked], ref)
            if not rel <= bar:
                raise SystemExit(f"prefill {label} M={m}: parity failure after timing, rel-L2 {rel:.3e} > {bar}")
            entry[label] = {"ms": round(float(np.median(samples)), 4), "ms_stats": stats(samples), "rel_l2_vs_f64_oracle": rel, "bar": bar}
            mat.dispose()
        out[f"M={m}"] = entry
        log(f"[prefill] FP32 activations M={m}: three products {entry['three_products']['ms']:.3f} ms (rel-L2 "
            f"{entry['three_products']['rel_l2_vs_f64_oracle']:.1e}), one product {entry['one_product']['ms']:.3f} ms "
            f"({entry['one_product']['rel_l2_vs_f64_oracle']:.1e}), mat-vec passes {entry['mat_vec_passes']['ms']:.3f} ms "
            f"({entry['mat_vec_passes']['rel_l2_vs_f64_oracle']:.1e})")
        x.dispose()
        y.dispose()
    return out


def _prefill_of(lane, nn, oracle, typ, tname, ms_list):
    from nntrain_amd import synth
    in_w, out_w = 5120, 17408
    payload = synth.matrix(typ, out_w, in_w, 2001)
    mat = nn.HipQuantizedMatrix(payload, typ, out_w, in_w)
    mat.device_payload(lane)
    out = {}
    for m in ms_list:
        xb = synth.to_bf16_bits(synth.activations(m, in_w, 4000))
        x = lane.upload_raw(xb)
        y = lane.allocate(m * out_w)
        try:
            mat.forward_bf16(lane, x, None, m, out=y)
        except nn.NnHipError as e:
            log(f"[prefill] unavailable: {e}")
            x.dispose()
            y.dispose()
            mat.dispose()
            return None
        lane.synchronize()
        # every 16th input row (every 64th at M = 2048: at most 32 rows) against the float64 oracle, before and after timing
        picked = np.arange(0, m, max(16, m // 32))
        ref, _ = oracle.linear_f64(typ, payload, np.ascontiguousarray(xb[picked]), None, len(picked), in_w, out_w, x_is_bf16=True)

        def check(tag):
            got = lane.read(y, np.float32, m * out_w).reshape(m, out_w)[picked]
            r = oracle.rel_l2(got, ref)
            if not (np.all(np.isfinite(got)) and r <= 2e-3):
                raise SystemExit(f"prefill {tname} M={m}: parity failure {tag}, rel-L2 {r:.3e} > 2e-3")
            return r

        rel = check("before timing")
        samples = []
        for _ in range(7):
            ms, _ = timed(lane, lambda: mat.forward_bf16(lane, x, None, m, out=y), 3)
            samples.append(ms / 3)
        ms = float(np.median(samples))
        rel = max(rel, check("after timing"))
        flops = 2.0 * m * in_w * out_w
        out[f"M={m}"] = {"ms": round(ms, 4), "ms_stats": stats(samples), "tflops": round(flops / ms / 1e9, 1),
                         "mfma_util_vs_2500_TFLOPs_bf16": round(flops / ms / 1e9 / BF16_PEAK_TFLOPS, 4),
                         "rel_l2_vs_f64_oracle": rel, "rows_checked": int(len(picked))}
        log(f"[prefill] {tname} M={m}: {ms:.3f} ms, {flops / ms / 1e9:.0f} TFLOP/s, rel-L2 {rel:.2e}")
        x.dispose()
        y.dispose()
    mat.dispose()
    return out


def library_gemm_yardstick(ms_list=(128, 256, 512, 2048)):
    """What the ROCm library GEMM (torch.matmul, bfloat16 weights already decoded and resident) reaches on the prefill
    shape on this box: a yardstick to read the prefill kernel's own figures against, nothing the product uses."""
    try:
        import torch
        if not torch.cuda.is_available():
            return {"unavailable": "torch sees no device"}
        in_w, out_w = 5120, 17408
        w = torch.randn(out_w, in_w, device="cuda", dtype=torch.bfloat16)
        out = {}
        for m in ms_list:
            x = torch.randn(m, in_w, device="cuda", dtype=torch.bfloat16)
            for _ in range(5):
                y = x @ w.t()
            torch.cuda.synchronize()
            samples = []
            for _ in range(5):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(5):
                    y = x @ w.t()
                e1.record()
                torch.cuda.synchronize()
                samples.append(e0.elapsed_time(e1) / 5)
            ms = float(np.median(samples))
            flops = 2.0 * m * in_w * out_w
            out[f"M={m}"] = {"ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 1),
                             "vs_2500_TFLOPs_bf16": round(flops / ms / 1e9 / BF16_PEAK_TFLOPS, 4)}
            log(f"[prefill] library bf16 GEMM (torch.matmul) M={m}: {ms:.3f} ms, {flops / ms / 1e9:.0f} TFLOP/s")
            del x, y
        return out
    except Exception as e:          # a yardstick only: its absence must not fail the run
        return {"unavailable": f"{type(e).__name__}: {e}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", choices=["decode27b", "decode27b_chained", "gemv", "prefill", "ffn", "decode_loop", "all", "library_gemm"],
                    default="all")
    ap.add_argument("--mode", choices=["forward", "graph", "batch"], default="batch",
                    help="decode27b: one launch per matrix, the same captured in a HIP graph, or the batched entry point")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="decode27b --mode batch: counter_collection.csv files of two rocprofv3 --pmc runs of this command "
                         "with --copy-calibration (FETCH_SIZE, WRITE_SIZE); fills roofline.traffic, which is null otherwise")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="decode27b: also run one device-to-device copy of the lm_head weights (for counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("this build measures one GPU: the quantized linear path has no collectives and every box has a "
                         "single MI355X; run with --gpus 1")

    if args.workload == "library_gemm":
        res = library_gemm_yardstick()
        at512 = res.get("M=512", {})
        print(json.dumps({"metric": "library bf16 GEMM on the prefill shape (torch.matmul), TFLOP/s at M=512", "value": at512.get("tflops"),
                          "unit": "TFLOP/s", "n_gpus": 1, "steps": 25, "warmup": 5, "ms_per_step": at512.get("ms"),
                          "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                          "config": {"workload": "library_gemm 17408x5120, M = 128 / 256 / 512 / 2048"}, "roofline": None,
                          "cpu_baseline": None, "also": {"library_bf16_gemm": res}}), flush=True)
        return

    import nntrain_amd as nn
    import oracle
    lane = nn.HipExecutionLane(0)
    log(f"device: {lane.device_name()}, {lane.compute_units} CUs, {lane.total_memory_bytes / 2**30:.0f} GiB")

    also = {}
    if args.workload in ("gemv", "all"):
        also["gemv_single_matrix"] = run_gemv(args, lane, nn, oracle)
    if args.workload in ("prefill", "all"):
        also["prefill_q4k_bf16_mfma"] = run_prefill(args, lane, nn, oracle)
    if args.workload in ("ffn", "all"):
        also["ffn_layer_half_fused_epilogues"] = run_ffn(args, lane, nn, oracle)
    if args.workload in ("decode_loop", "all"):
        also["decode_loop_gguf_file"] = run_decode_loop(args, lane, nn, oracle)
    if args.workload in ("decode27b_chained", "all"):
        also["decode27b_chained"] = run_decode27b_chained(args, lane, nn, oracle)
    if args.workload in ("decode27b", "all"):
        res = run_decode27b(args, lane, nn, oracle)
    else:
        res = {"metric": "quant GEMV GB/s", "value": None, "unit": "GB/s", "ms_per_step": None,
               "config": {"workload": args.workload}, "roofline": None, "cpu_baseline": None}
    lane.dispose()

    line = {
        "metric": res["metric"], "value": res["value"], "unit": res["unit"], "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": res["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic", "config": res["config"],
        "roofline": res["roofline"], "cpu_baseline": res["cpu_baseline"],
    }
    if "ms_per_step_stats" in res:
        line["ms_per_step_stats"] = res["ms_per_step_stats"]
    if "parity" in res:
        line["parity"] = res["parity"]
    if also:
        line["also"] = also
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
