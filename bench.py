#!/usr/bin/env python3
"""Benchmark of the quantized decode hot path on one MI355X.

A step is one pass of the Q4_K decode matvec (batch 1) over the four Llama-3-8B layer shapes
(4096x4096 q/o, 1024x4096 k/v, 14336x4096 gate/up, 4096x14336 down), activations f32 N(0,1), weights
random Q4_K super-blocks (f16 d/dmin ~ N(0, 0.02), 6-bit scales/mins, uniform nibbles), all resident in
HBM before the timed region.  Each shape rotates over enough distinct weight buffers to exceed the
256 MB last-level cache, so the bytes really come from HBM.

Prints ONE JSON line: whole-path GB/s (algorithmic bytes / device time), the roofline of the dominant
kernel and the CPU checker timed on the host cores beside it.  The same line carries, under "e2e", the second
half of the metric: tokens/s of the random-init Q4_K_M Llama-3-8B-architecture decoder (512-token prompt, 256
greedy steps, batch 1; about 10 s including the weight upload; --no-e2e skips it).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SHAPES = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)]  # (n, k)
HBM_PEAK_GBS = 8000.0
ROTATE_BYTES = 640 << 20  # > 2x the 256 MB Infinity Cache
# HBM bytes per launch (average of the four shapes) measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on this
# workload at batch 1, scaled by what the same counters read for a 256 MiB device copy (FETCH_SIZE x2.000,
# WRITE_SIZE x1.000); a measured constant, to be re-measured when the kernel changes.
TRAFFIC_BYTES_PER_LAUNCH = 19766426


def prefill_legs(dev) -> dict:
    """configs[2]: Y = X . W^T with bf16 X [m, 4096] and Q6_K / Q8_0 W [14336, 4096]; configs[3]: causal attention,
    f16, 32 query heads on 8 KV heads, head_dim 128.  Device time per call from events around 5 calls; TFLOP/s counts
    2 m n k (matmul) and 4 s^2 d h / 2 (causal attention) against the 2.5 PFLOP/s dense f16 MFMA peak."""
    from kalosm_amd import synth
    from kalosm_amd.fusor import MaskKind, QMatrix, Tensor

    res = {"matmul": [], "attention": [], "attention_decode": []}
    n, k = 14336, 4096
    for ty, name in ((synth.Q6_K, "Q6_K"), (synth.Q8_0, "Q8_0")):
        q = QMatrix.from_raw_bytes(dev, (n, k), synth.random_weight(ty, n, k, seed=7), ty)
        for m in (512, 2048):
            x = Tensor.from_slice(dev, synth.to_bf16_bits(synth.random_activation(m, k, seed=8)), dtype="bf16")
            y = Tensor(dev, (m, n), "f32")
            for _ in range(2):
                x.q_mat_mul(q, out=y)
            dev.sync()
            dev.timer_start()
            for _ in range(5):
                x.q_mat_mul(q, out=y)
            ms = dev.timer_stop() / 5
            tf = 2.0 * m * n * k / ms / 1e9
            res["matmul"].append({"weights": name, "activations": "bf16", "m": m, "n": n, "k": k,
                                  "us": round(ms * 1e3, 1), "TFLOPs": round(tf, 1),
                                  "frac_mfma_peak": round(tf / 2500.0, 4)})
            if ty == synth.Q8_0:  # the integer variant: f32 activations quantised per 32 inside the call, int8 MFMA
                xf = Tensor.from_slice(dev, synth.random_activation(m, k, seed=8))
                for _ in range(2):
                    xf.q_mat_mul_q8(q, out=y)
                dev.sync()
                dev.timer_start()
                for _ in range(5):
                    xf.q_mat_mul_q8(q, out=y)
                ms = dev.timer_stop() / 5
                tf = 2.0 * m * n * k / ms / 1e9
                res["matmul"].append({"weights": name, "activations": "Q8_0 per 32 (int8 MFMA)", "m": m, "n": n, "k": k,
                                      "us": round(ms * 1e3, 1), "TOPs": round(tf, 1),
                                      "frac_int8_mfma_peak": round(tf / 5000.0, 4)})
    # the decoder's own prefill projections with few output tiles (k split over workgroups): f32 activations
    for ty, name, n2, k2 in ((synth.Q4_K, "Q4_K", 4096, 4096), (synth.Q6_K, "Q6_K", 4096, 14336)):
        q = QMatrix.from_raw_bytes(dev, (n2, k2), synth.random_weight(ty, n2, k2, seed=9), ty)
        m = 512
        xf = Tensor.from_slice(dev, synth.random_activation(m, k2, seed=10))
        y = Tensor(dev, (m, n2), "f32")
        for _ in range(2):
            xf.q_mat_mul(q, out=y)
        dev.sync()
        dev.timer_start()
        for _ in range(5):
            xf.q_mat_mul(q, out=y)
        ms = dev.timer_stop() / 5
        tf = 2.0 * m * n2 * k2 / ms / 1e9
        res["matmul"].append({"weights": name, "activations": "f32", "m": m, "n": n2, "k": k2, "us": round(ms * 1e3, 1),
                              "TFLOPs": round(tf, 1), "frac_mfma_peak": round(tf / 2500.0, 4)})
    h, hkv, d = 32, 8, 128
    for s in (512, 2048, 8192):
        rng = np.random.default_rng(s)
        qt, kt, vt = (Tensor.from_slice(dev, rng.standard_normal((1, hh, s, d)).astype(np.float16), "f16")
                      for hh in (h, hkv, hkv))
        ot = Tensor(dev, (1, h, s, d), "f16")
        for _ in range(2):
            qt.flash_attention(kt, vt, 1 / np.sqrt(d), MaskKind.Causal, out=ot)
        dev.sync()
        dev.timer_start()
        for _ in range(5):
            qt.flash_attention(kt, vt, 1 / np.sqrt(d), MaskKind.Causal, out=ot)
        ms = dev.timer_stop() / 5
        tf = 4.0 * s * s * d * h / 2 / ms / 1e9
        res["attention"].append({"seq": s, "us": round(ms * 1e3, 1), "TFLOPs": round(tf, 1),
                                 "frac_mfma_peak": round(tf / 2500.0, 4)})
    # configs[3], decode variant: one query per head against a cache of L keys (f16 K / V), HBM bound:
    # bytes = K and V once (2 * hkv * L * d * 2) + the query and the output (2 * h * d * 2); caches rotate over
    # more than the Infinity Cache
    for L in (1024, 4096, 16384):
        rng = np.random.default_rng(L)
        kv_bytes = 2 * hkv * L * d * 2
        copies = max(2, -(-(640 << 20) // kv_bytes))
        kvs = []
        base_k = rng.standard_normal((1, hkv, L, d)).astype(np.float16)
        base_v = rng.standard_normal((1, hkv, L, d)).astype(np.float16)
        for c in range(min(copies, 160)):
            kvs.append((Tensor.from_slice(dev, base_k, "f16"), Tensor.from_slice(dev, base_v, "f16")))
        qt = Tensor.from_slice(dev, rng.standard_normal((1, h, 1, d)).astype(np.float16), "f16")
        ot = Tensor(dev, (1, h, 1, d), "f16")
        reps = 200
        for i in range(20):
            qt.flash_attention(*kvs[i % len(kvs)], 1 / np.sqrt(d), None, out=ot)
        dev.sync()
        dev.timer_start()
        for i in range(reps):
            qt.flash_attention(*kvs[i % len(kvs)], 1 / np.sqrt(d), None, out=ot)
        ms = dev.timer_stop() / reps
        nbytes = kv_bytes + 2 * h * d * 2
        res["attention_decode"].append({"kv_len": L, "us": round(ms * 1e3, 2), "bytes": nbytes,
                                        "GBps": round(nbytes / ms / 1e6, 1), "frac_hbm_peak": round(nbytes / ms / 1e6 / 8000.0, 4),
                                        "cache_copies_rotated": len(kvs)})
        del kvs
    return res


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--m", type=int, default=1, help="activation rows (decode batch)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--e2e", action="store_true", help="(default) also run the 8B-architecture decoder and report tok/s")
    ap.add_argument("--no-e2e", action="store_true", help="skip the 8B-architecture decoder leg (about 10 s)")
    ap.add_argument("--e2e-eager", action="store_true",
                    help="also run 32 decode steps of the decoder with stream launches (for a kernel tracer)")
    ap.add_argument("--prefill", action="store_true",
                    help="also time the prefill matmul (configs[2]) and the causal prefill attention (configs[3])")
    ap.add_argument("--no-graph", action="store_true", help="launch on the stream instead of replaying a recorded graph")
    ap.add_argument("--calib-copy", action="store_true", help="append 4 device copies of 256 MiB (counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (nothing in it uses a second); run with --gpus 1",
              file=sys.stderr)
        return 2

    from kalosm_amd import synth
    from kalosm_amd.fusor import Device, QMatrix, Tensor

    dev = Device.gpu(0)
    info = dev.info()
    m = args.m
    ty = synth.Q4_K

    # ---- resident inputs
    sets = []
    for si, (n, k) in enumerate(SHAPES):
        wbytes = n * (k // 256) * 144
        copies = max(2, -(-ROTATE_BYTES // wbytes))
        raw = synth.random_weight(ty, n, k, seed=1000 + si)
        qs = [QMatrix.from_raw_bytes(dev, (n, k), raw, ty) for _ in range(copies)]
        x = Tensor.from_slice(dev, synth.random_activation(m, k, seed=2000 + si))
        y = Tensor(dev, (m, n), "f32")
        sets.append(dict(n=n, k=k, qs=qs, x=x, y=y, raw=raw, bytes=synth.matvec_bytes(ty, n, k, m)))

    def run_shape(s, launches, offset=0):
        qs, x, y = s["qs"], s["x"], s["y"]
        for i in range(launches):
            x.q_mat_mul(qs[(offset + i) % len(qs)], out=y)

    # ---- warmup, then the timed steps (per shape trains inside one bracketed region)
    # The K launches of a shape are recorded once and replayed as one submission (the reference submits one
    # command buffer per resolve); host launch overhead of the Python/ctypes loop stays out of the device time.
    for s in sets:
        run_shape(s, args.warmup)
    dev.sync()
    per_shape_ms = []
    if args.no_graph:  # plain stream launches (for runs under a kernel tracer, which does not follow graph replays)
        t_wall0 = time.perf_counter()
        for s in sets:
            dev.timer_start()
            run_shape(s, args.steps, offset=args.warmup)
            per_shape_ms.append(dev.timer_stop())
    else:
        graphs = []
        for s in sets:
            dev.graph_begin()
            run_shape(s, args.steps, offset=args.warmup)
            graphs.append(dev.graph_end())
        t_wall0 = time.perf_counter()
        for g in graphs:
            dev.timer_start()
            g.launch()
            per_shape_ms.append(dev.timer_stop())
    if args.calib_copy:  # a device-to-device copy of known size, to scale the FETCH_SIZE / WRITE_SIZE counters
        nbytes = 256 << 20
        a, b = Tensor(dev, (nbytes,), "u8"), Tensor(dev, (nbytes,), "u8")
        import ctypes as C
        for _ in range(4):
            dev._lib.fh_copy(dev._h, C.c_void_p(b.ptr), C.c_void_p(a.ptr), nbytes)
    dev.sync()
    wall_ms = (time.perf_counter() - t_wall0) * 1e3
    total_ms = float(sum(per_shape_ms))
    step_bytes = sum(s["bytes"] for s in sets)
    value = step_bytes * args.steps / (total_ms * 1e-3) / 1e9
    shapes_out = []
    for s, ms in zip(sets, per_shape_ms):
        us = ms * 1e3 / args.steps
        shapes_out.append({"n": s["n"], "k": s["k"], "us_per_launch": round(us, 3),
                           "GBps": round(s["bytes"] / (us * 1e-6) / 1e9, 1),
                           "frac_hbm_peak": round(s["bytes"] / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)})
    # dominant kernel: the Q4_K MFMA matvec k_qmv_q4k_m1, one launch per matvec (activation staging is inside it);
    # its launches are the step's four, so the per-launch average is (bytes of the four shapes / 4) over
    # (device time / launches).  Device time between events includes the dispatch gap between dependent launches.
    launches = args.steps * len(sets)
    avg_us = total_ms * 1e3 / launches
    achieved = (step_bytes / len(sets)) / (avg_us * 1e-6) / 1e9
    out = {
        "metric": "Q4_K matvec GB/s (% HBM peak); Q4_K_M 8B-arch decode tok/s, batch 1, 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(total_ms / args.steps, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: Q4_K decode matvec at Llama-3-8B layer shapes "
                               "(4096x4096, 1024x4096, 14336x4096, 4096x14336), batch %d, one launch each per step" % m,
                   "batch": m, "weights_rotated_bytes_per_shape": ROTATE_BYTES, "device": info["name"],
                   "compute_units": info["compute_units"]},
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "shapes": shapes_out,
        "wall_ms_timed_region": round(wall_ms, 2),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_BYTES_PER_LAUNCH if m == 1 else None,
                     "kernel": "k_qmv_q4k_m1 (instances <1,1>, <2,1>, <1,4>: tiles, blocks per wavefront)", "avg_launch_us": round(avg_us, 3),
                     "algorithmic_bytes_per_launch": step_bytes // len(sets)},
    }

    # ---- CPU baseline: the checker's q_mat_mul (a C restatement of fusor-ml/cpu, not the Rust binary),
    # same shapes and inputs, all host cores, bounded repetitions
    if not args.no_cpu:
        from oracle import oracle

        oracle.build()
        threads = oracle.default_threads()
        t_budget, reps_done, cpu_s, cpu_bytes = 12.0, 0, 0.0, 0
        xs = [s["x"].as_slice() for s in sets]
        for s, x in zip(sets, xs):  # warm
            oracle.q_mat_mul(ty, x, s["raw"], s["n"], threads=threads)
        while cpu_s < t_budget and reps_done < 20:
            t0 = time.perf_counter()
            for s, x in zip(sets, xs):
                oracle.q_mat_mul(ty, x, s["raw"], s["n"], threads=threads)
            cpu_s += time.perf_counter() - t0
            cpu_bytes += step_bytes
            reps_done += 1
        out["cpu_baseline"] = {"value": round(cpu_bytes / cpu_s / 1e9, 3), "unit": "GB/s", "cores": threads,
                               "kind": "port",
                               "sample": "%d repetitions of the same four matvecs (same weights and activations), "
                                         "%d threads with the reference's static column split" % (reps_done, threads)}
        # parity of the timed configuration against the checker
        worst = 0.0
        for s, x in zip(sets, xs):
            s["x"].q_mat_mul(s["qs"][0], out=s["y"])
            got = s["y"].as_slice()
            want = oracle.q_mat_mul(ty, x, s["raw"], s["n"], threads=threads)
            diff = np.abs(got - want)
            ok = (diff <= 1e-2) | (diff <= 1e-3 * np.maximum(np.abs(got), np.abs(want)))
            if not ok.all():
                print("bench.py: PARITY FAILURE at shape", s["n"], s["k"], "max abs", diff.max(), file=sys.stderr)
                return 1
            worst = max(worst, float(diff.max()))
        out["parity_max_abs_err"] = worst

    if not args.no_e2e and not args.e2e_eager:
        from kalosm_amd import e2e
        out["e2e"] = e2e.run(dev)
    if args.e2e_eager:
        from kalosm_amd import e2e
        out["e2e_eager"] = e2e.run(dev, steps=32, repeats=1, use_graph=False)
    if args.prefill:
        out["prefill"] = prefill_legs(dev)

    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
