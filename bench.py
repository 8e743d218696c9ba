#!/usr/bin/env python3
"""Benchmark of the quantized decode hot path on one MI355X.

A step is one pass of the Q4_K decode matvec (batch 1) over the four Llama-3-8B layer shapes
(4096x4096 q/o, 1024x4096 k/v, 14336x4096 gate/up, 4096x14336 down), activations f32 N(0,1), weights
random Q4_K super-blocks (f16 d/dmin ~ N(0, 0.02), 6-bit scales/mins, uniform nibbles), all resident in
HBM before the timed region.  Each shape rotates over enough distinct weight buffers to exceed the
256 MB last-level cache, and a recorded train of a shape has max(K, copies, 200) launches, one after the other through
the whole pool, so a buffer is read again only after 640 MB of others: the bytes come from HBM whatever K is.  The
train is replayed `--trains` times and the median replay gives the shape's time per launch; the reported step time is
K steps at that rate (the repetitions only steady the number).

Prints ONE JSON line: whole-path GB/s (algorithmic bytes / device time), the roofline of the dominant
kernel and the CPU checker timed on the host cores beside it.  The same line carries the other benchmark
configurations, each with its own roofline entry: "batch" (configs[1] at 4 and 16 rows), "prefill"
(configs[2]: bf16 x Q6_K / Q8_0 and the Q8_0 x Q8 integer variant at 512 and 2048 rows; configs[3]: causal
attention at 512 / 2048 / 8192 and single-query attention against 1024 / 4096 / 16384 cached keys) and "e2e"
(configs[4]: tokens/s of the random-init Q4_K_M Llama-3-8B-architecture decoder, 512-token prompt, 256 greedy
steps, batch 1, with its greedy tokens checked against the CPU checker on a short prompt outside the timed
region).  --no-legs / --no-e2e skip them.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SHAPES = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)]  # (n, k)
HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
MFMA_I8_PEAK_TOPS = 5000.0
ROTATE_BYTES = 640 << 20  # > 2x the 256 MB Infinity Cache
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "q4k_matvec_m1_llama_shapes.md")


def measured_traffic():
    """HBM bytes per launch of the headline kernel as the tracked counter profile states them (rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE scaled by a copy of known size), with the commit the profile was taken at."""
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None, None
    m = re.search(r"traffic_bytes_per_launch\s*=\s*(\d+)", text)
    c = re.search(r"measured_at_commit\s*=\s*([0-9a-f]{7,40})", text)
    return (int(m.group(1)) if m else None), (c.group(1) if c else None)


def timed_trains(dev, enqueue, trains: int, use_graph: bool = True):
    """Median device milliseconds of `trains` runs of the launch sequence `enqueue()` (recorded once and replayed
    unless use_graph is off; one untimed run first)."""
    ms = []
    if use_graph:
        dev.graph_begin()
        enqueue()
        g = dev.graph_end()
        g.launch()          # one untimed replay
        dev.sync()
        for _ in range(trains):
            dev.timer_start()
            g.launch()
            ms.append(dev.timer_stop())
        del g
    else:
        enqueue()
        dev.sync()
        for _ in range(trains):
            dev.timer_start()
            enqueue()
            ms.append(dev.timer_stop())
    return statistics.median(ms), ms


def train_length(steps: int, copies: int) -> int:
    """Launches of one timed train over a pool of `copies` buffers that together exceed the memory-side cache twice
    over: at least `steps`, at least once through the whole pool, so that a buffer is read again only after 640 MB of
    others - every replay of the train then reads from HBM whatever `steps` is - and at least 200, so that what
    starting a replay costs (some 17 us between the two events) does not weigh on the figure per launch."""
    return max(steps, copies, 200)


def matvec_sets(dev, ty, m: int):
    from kalosm_amd import synth
    from kalosm_amd.fusor import QMatrix, Tensor

    sets = []
    for si, (n, k) in enumerate(SHAPES):
        wbytes = n * (k // 256) * 144
        copies = max(2, -(-ROTATE_BYTES // wbytes))
        raw = synth.random_weight(ty, n, k, seed=1000 + si)
        qs = [QMatrix.from_raw_bytes(dev, (n, k), raw, ty) for _ in range(copies)]
        x = Tensor.from_slice(dev, synth.random_activation(m, k, seed=2000 + si))
        y = Tensor(dev, (m, n), "f32")
        sets.append(dict(n=n, k=k, qs=qs, x=x, y=y, raw=raw, bytes=synth.matvec_bytes(ty, n, k, m)))
    return sets


def run_shape(s, launches, offset=0):
    qs, x, y = s["qs"], s["x"], s["y"]
    for i in range(launches):
        x.q_mat_mul(qs[(offset + i) % len(qs)], out=y)


def batch_leg(dev, sets_m1, steps: int, warmup: int, trains: int) -> list:
    """configs[1] at 4 and 16 activation rows: the same four shapes and weight rotation, HBM bound (the weights are
    still read once per call)."""
    from kalosm_amd import synth
    from kalosm_amd.fusor import Tensor

    out = []
    for m in (4, 16):
        tot_ms, tot_bytes, per = 0.0, 0, []
        for si, s in enumerate(sets_m1):
            n, k = s["n"], s["k"]
            t = dict(s, x=Tensor.from_slice(dev, synth.random_activation(m, k, seed=2100 + si)), y=Tensor(dev, (m, n), "f32"),
                     bytes=synth.matvec_bytes(synth.Q4_K, n, k, m))
            run_shape(t, warmup)
            dev.sync()
            L = train_length(steps, len(t["qs"]))
            ms, _ = timed_trains(dev, lambda: run_shape(t, L, offset=warmup), trains)
            tot_ms += ms / L
            tot_bytes += t["bytes"]
            per.append({"n": n, "k": k, "us_per_launch": round(ms * 1e3 / L, 3), "launches_per_train": L})
        gbs = tot_bytes / (tot_ms * 1e-3) / 1e9
        out.append({"rows": m, "GBps": round(gbs, 1), "shapes": per,
                    "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                 "frac": round(gbs / HBM_PEAK_GBS, 4)}})
    return out


def decoder_shapes_leg(dev, steps: int, warmup: int, trains: int) -> list:
    """The two fused matrices a decode step of the 8B architecture launches besides the four layer shapes of
    configs[1]: q|k|v (6144 x 4096) and gate|up (28672 x 4096), plain matvec, batch 1, weights rotated over 640 MB."""
    from kalosm_amd import synth
    from kalosm_amd.fusor import QMatrix, Tensor

    out = []
    for si, (n, k) in enumerate(((6144, 4096), (28672, 4096))):
        wbytes = n * (k // 256) * 144
        copies = max(2, -(-ROTATE_BYTES // wbytes))
        raw = synth.random_weight(synth.Q4_K, n, k, seed=1100 + si)
        s = dict(qs=[QMatrix.from_raw_bytes(dev, (n, k), raw, synth.Q4_K) for _ in range(copies)],
                 x=Tensor.from_slice(dev, synth.random_activation(1, k, seed=2200 + si)), y=Tensor(dev, (1, n), "f32"))
        nbytes = synth.matvec_bytes(synth.Q4_K, n, k, 1)
        run_shape(s, warmup)
        dev.sync()
        L = train_length(steps, copies)
        ms, _ = timed_trains(dev, lambda: run_shape(s, L, offset=warmup), trains)
        us = ms * 1e3 / L
        out.append({"n": n, "k": k, "us_per_launch": round(us, 3), "GBps": round(nbytes / us / 1e3, 1),
                    "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)})
        del s
    return out


def _errs(got, want):
    """Largest absolute and largest relative difference (relative to max(|got|, |want|), over the elements whose
    absolute difference exceeds 1e-2: the ones the relative bound has to cover) and the tolerance verdict."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = np.abs(got - want)
    scale = np.maximum(np.abs(got), np.abs(want))
    rel = np.where(scale > 0, d / np.where(scale > 0, scale, 1.0), 0.0)
    ok = bool(((d <= 1e-2) | (d <= 1e-3 * scale)).all())
    return {"max_abs_err": float(d.max()), "max_rel_err": float(rel.max()),
            "max_rel_err_where_abs_above_1e-2": float(rel[d > 1e-2].max()) if (d > 1e-2).any() else 0.0, "ok": ok}


def five_bit_leg(dev, steps: int, warmup: int, trains: int) -> list:
    """Q5_K and Q5_0 (the 5-bit formats of Q5_K_M / Q5_0 model files) through the single-row matrix-core kernel, beside
    Q4_K on the same two shapes in the same run: batch 1, weights rotated over 640 MB, HBM bound."""
    from kalosm_amd import synth
    from kalosm_amd.fusor import QMatrix, Tensor

    out = []
    for n, k in ((4096, 4096), (14336, 4096)):
        base = None
        for ty in (synth.Q4_K, synth.Q5_K, synth.Q5_0):
            wbytes = n * (k // synth.BLOCK_ELEMS[ty]) * synth.BLOCK_BYTES[ty]
            copies = max(2, -(-ROTATE_BYTES // wbytes))
            raw = synth.random_weight(ty, n, k, seed=1200 + ty)
            s = dict(qs=[QMatrix.from_raw_bytes(dev, (n, k), raw, ty) for _ in range(copies)],
                     x=Tensor.from_slice(dev, synth.random_activation(1, k, seed=2300)), y=Tensor(dev, (1, n), "f32"))
            nbytes = synth.matvec_bytes(ty, n, k, 1)
            run_shape(s, warmup)
            dev.sync()
            L = train_length(steps, copies)
            ms, _ = timed_trains(dev, lambda: run_shape(s, L, offset=warmup), trains)
            us = ms * 1e3 / L
            e = {"weights": synth.TYPE_NAMES[ty], "n": n, "k": k, "us_per_launch": round(us, 3), "ns_per_KB": round(us * 1e6 / nbytes, 3),
                 "roofline": {"bound": "hbm", "achieved": round(nbytes / us / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}}
            if ty == synth.Q4_K:
                base = us / nbytes
            else:
                e["time_per_byte_vs_Q4_K"] = round(us / nbytes / base, 3)
            out.append(e)
            del s
    return out


def prefill_legs(dev, trains: int, use_graph: bool = True, check: bool = False) -> dict:
    """configs[2]: Y = X . W^T with bf16 X [m, 4096] and Q6_K / Q8_0 W [14336, 4096]; configs[3]: causal attention,
    f16, 32 query heads on 8 KV heads, head_dim 128, and its decode variant.  Device time per call: the median over
    `trains` replays of a recorded train of CALLS back-to-back calls (as the headline and the decode variant are timed:
    a call in a pipeline of launches, not a lone launch between two events), all launches of a call included;
    TFLOP/s counts 2 m n k (matmul) and 4 s^2 d h / 2 (causal attention) against the 2.5 PFLOP/s dense f16 MFMA peak
    (5 POP/s for the int8 variant); the decode variant counts K and V bytes against the 8 TB/s HBM peak."""
    from kalosm_amd import synth
    from kalosm_amd.fusor import MaskKind, QMatrix, Tensor

    CALLS = 8

    def med(fn):
        # warm-up: at least three calls and 50 ms of them (the device drops its clocks while the host prepares the next
        # case's inputs; the first calls after that run slower than the steady state the figure is about)
        t0, calls = time.perf_counter(), 0
        while calls < 3 or time.perf_counter() - t0 < 0.05:
            fn()
            dev.sync()
            calls += 1
        ms, _ = timed_trains(dev, lambda: [fn() for _ in range(CALLS)], max(trains, 7), use_graph)
        return ms / CALLS

    def mfma(tf, peak=MFMA_F16_PEAK_TFLOPS, unit="TFLOP/s"):
        return {"bound": "mfma", "achieved": round(tf, 1), "peak": peak, "unit": unit, "frac": round(tf / peak, 4)}

    res = {"calls_per_train": CALLS, "matmul": [], "attention": [], "attention_decode": []}
    if check:
        from oracle import oracle
        res["parity"] = "one checked call per configuration, outside the timed trains: CPU checker on 48 sampled weight " \
                        "rows (matmul), float64 softmax attention on sampled query rows (causal), the checker's " \
                        "attention (single query); tolerance 1e-2 absolute or 1e-3 relative"
    n, k = 14336, 4096
    for ty, name in ((synth.Q6_K, "Q6_K"), (synth.Q8_0, "Q8_0")):
        raw = synth.random_weight(ty, n, k, seed=7)
        q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
        rows = (np.arange(48) * 293 + 5) % n
        bpr = len(raw) // n
        sub = np.concatenate([raw[r * bpr:(r + 1) * bpr] for r in rows]) if check else None
        for m in (512, 2048):
            xa = synth.random_activation(m, k, seed=8)
            bits = synth.to_bf16_bits(xa)
            x = Tensor.from_slice(dev, bits, dtype="bf16")
            y = Tensor(dev, (m, n), "f32")
            ms = med(lambda: x.q_mat_mul(q, out=y))
            tf = 2.0 * m * n * k / ms / 1e9
            e = {"weights": name, "activations": "bf16", "m": m, "n": n, "k": k, "us": round(ms * 1e3, 1), "roofline": mfma(tf)}
            if check:
                xb = (bits.astype(np.uint32) << 16).view(np.float32).reshape(m, k)
                e["parity"] = _errs(y.as_slice()[:, rows], oracle.q_mat_mul(ty, xb, sub, len(rows), fast=True))
            res["matmul"].append(e)
            if ty == synth.Q8_0:  # the integer variant: f32 activations quantised per 32 inside the call, int8 MFMA
                xf = Tensor.from_slice(dev, xa)
                ms = med(lambda: xf.q_mat_mul_q8(q, out=y))
                tf = 2.0 * m * n * k / ms / 1e9
                e = {"weights": name, "activations": "Q8_0 per 32 (int8 MFMA)", "m": m, "n": n, "k": k,
                     "us": round(ms * 1e3, 1), "roofline": mfma(tf, MFMA_I8_PEAK_TOPS, "TOP/s")}
                if check:
                    e["parity"] = _errs(y.as_slice()[:, rows], oracle.q8_0_matmul_q8(xa, sub, len(rows)))
                res["matmul"].append(e)
    # the decoder's own prefill projections with few output tiles (k split over workgroups): f32 activations
    for ty, name, n2, k2 in ((synth.Q4_K, "Q4_K", 4096, 4096), (synth.Q6_K, "Q6_K", 4096, 14336)):
        q = QMatrix.from_raw_bytes(dev, (n2, k2), synth.random_weight(ty, n2, k2, seed=9), ty)
        m = 512
        xf = Tensor.from_slice(dev, synth.random_activation(m, k2, seed=10))
        y = Tensor(dev, (m, n2), "f32")
        ms = med(lambda: xf.q_mat_mul(q, out=y))
        tf = 2.0 * m * n2 * k2 / ms / 1e9
        res["matmul"].append({"weights": name, "activations": "f32", "m": m, "n": n2, "k": k2, "us": round(ms * 1e3, 1),
                              "roofline": mfma(tf)})
    h, hkv, d = 32, 8, 128
    for s in (512, 2048, 8192):
        rng = np.random.default_rng(s)
        qa, ka, va = (rng.standard_normal((1, hh, s, d)).astype(np.float16) for hh in (h, hkv, hkv))
        qt, kt, vt = (Tensor.from_slice(dev, a, "f16") for a in (qa, ka, va))
        ot = Tensor(dev, (1, h, s, d), "f16")
        ms = med(lambda: qt.flash_attention(kt, vt, 1 / np.sqrt(d), MaskKind.Causal, out=ot))
        tf = 4.0 * s * s * d * h / 2 / ms / 1e9
        e = {"seq": s, "us": round(ms * 1e3, 1), "roofline": mfma(tf)}
        if check:  # float64 softmax attention on 24 sampled query rows of three heads
            got = ot.as_slice().astype(np.float32)
            rows = sorted(set([0, 1, 63, 64, 127, 128, s // 2, s - 129, s - 64, s - 1] + rng.integers(0, s, 14).tolist()))
            g, w = [], []
            for hh in (0, 5, 31):
                kf, vf = ka[0, hh // (h // hkv)].astype(np.float64), va[0, hh // (h // hkv)].astype(np.float64)
                for i in rows:
                    sc = (qa[0, hh, i].astype(np.float64) @ kf[:i + 1].T) / np.sqrt(d)
                    pr = np.exp(sc - sc.max())
                    w.append((pr / pr.sum()) @ vf[:i + 1])
                    g.append(got[0, hh, i])
            e["parity"] = _errs(np.array(g), np.array(w))
        res["attention"].append(e)
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
        reps = 100

        def train(off=0):
            for i in range(reps):
                qt.flash_attention(*kvs[(off + i) % len(kvs)], 1 / np.sqrt(d), None, out=ot)

        train()
        dev.sync()
        reps = train_length(reps, len(kvs))
        ms, _ = timed_trains(dev, lambda: train(7), trains)
        ms /= reps
        nbytes = kv_bytes + 2 * h * d * 2
        gbs = nbytes / ms / 1e6
        e = {"kv_len": L, "us": round(ms * 1e3, 2), "bytes": nbytes, "cache_copies_rotated": len(kvs),
             "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(gbs / HBM_PEAK_GBS, 4)}}
        if check:
            qa = qt.as_slice().astype(np.float32)
            qt.flash_attention(*kvs[0], 1 / np.sqrt(d), None, out=ot)
            e["parity"] = _errs(ot.as_slice().astype(np.float32),
                                oracle.flash_attention(qa, base_k.astype(np.float32), base_v.astype(np.float32), 1 / np.sqrt(d)))
        res["attention_decode"].append(e)
        del kvs
    return res


def calibration(dev, trains: int, use_graph: bool, probes: bool = True) -> dict:
    """What one dependent launch costs on this device whatever the kernel does: an empty kernel, and a plain
    streaming read of the byte counts of the benchmark's matrices (rotating like the weights do)."""
    from kalosm_amd.fusor import Tensor
    import ctypes as C

    L = 100
    out = {"launches_per_train": L, "empty_us": {}, "read": [],
           "what": "an empty kernel and a plain streaming read (k_probe_read: 16 bytes per lane and request, 4 KB per "
                   "wavefront) launched like the matvec: trains of dependent launches in a replayed graph, buffers of "
                   "the matrices' sizes rotated over 768 MB"}
    for wg, th in ((1, 64), (256, 1024)):
        ms, _ = timed_trains(dev, lambda: [dev._lib.fh_probe_empty(dev._h, wg, th) for _ in range(L)], trains, use_graph)
        out["empty_us"]["%dx%d" % (wg, th)] = round(ms * 1e3 / L, 3)
    total = 768 << 20
    buf = Tensor(dev, (total,), "u8")
    dev._lib.fh_memset(dev._h, C.c_void_p(buf.ptr), 1, total)
    for nbytes in (2359296, 9437184, 33030144, 66060288, 430940160):
        used = nbytes // 16384 * 16384
        copies = max(1, total // used)

        Lr = train_length(L, min(copies, -(-ROTATE_BYTES // used)))

        def train():
            for i in range(Lr):
                dev._lib.fh_probe_read(dev._h, C.c_void_p(buf.ptr + (i % copies) * used), used)

        train()
        dev.sync()
        ms, _ = timed_trains(dev, train, trains, use_graph)
        us = ms * 1e3 / Lr
        out["read"].append({"bytes": used, "us": round(us, 3), "GBps": round(used / us / 1e3, 1)})
    del buf
    if probes:
        out["device"] = device_probes(dev)
    return out


def device_probes(dev) -> dict:
    """fh_probe_device: the dense MFMA rate, LDS read throughput by wavefront count and address pattern, and L2 hits
    next to an HBM stream inside one compute unit."""
    from kalosm_amd.fusor import Tensor
    from kalosm_amd._lib import check
    import ctypes as C

    res = (C.c_double * 4)()

    def probe(kind, a, b, ptr=None, nbytes=0):
        check(dev._lib.fh_probe_device(dev._h, kind, a, b, C.c_void_p(ptr) if ptr else None, nbytes, res))
        return [res[i] for i in range(4)]

    out = {"mfma_32x32x16_f16": [], "lds_read_b128": [], "l2_next_to_hbm": []}
    for waves in (1, 2):
        for iters in (2000, 20000, 100000):
            r = probe(0, waves, iters)
            out["mfma_32x32x16_f16"].append({"wavefronts_per_simd": waves, "iterations": iters, "TFLOPs": round(r[0], 1),
                                              "us": round(r[1], 1)})
    names = ["linear", "operand rows, no swizzle", "operand rows, row & 7", "operand rows, tile kernels' swizzle"]
    for pattern in range(4):
        for waves in (4, 8, 16):
            r = probe(1, waves, pattern)
            out["lds_read_b128"].append({"pattern": names[pattern], "wavefronts": waves,
                                         "bytes_per_clock_per_cu": round(r[1], 1)})
    cus = dev.info()["compute_units"] if hasattr(dev, "info") else 256
    need = (256 << 10) + cus * 16 * (512 << 10)
    buf = Tensor(dev, (need,), "u8")
    dev._lib.fh_memset(dev._h, C.c_void_p(buf.ptr), 1, need)
    modes = ["all wavefronts on the shared 256 KB", "all wavefronts streaming", "even on the shared region, odd streaming"]
    for mode in range(3):
        r = probe(2, mode, 0, buf.ptr, need)
        out["l2_next_to_hbm"].append({"mode": modes[mode], "l2_bytes_per_ns_per_cu": round(r[0], 1),
                                      "hbm_bytes_per_ns_per_cu": round(r[1], 1)})
    return out


def e2e_check(model, weights, cfg, prompt_len=16, steps=8):
    """The decoder that was just timed against the CPU checker's decoder on the same weights, outside the timed
    region: logits of a short prompt within tolerance and the greedy ids that follow (a step whose two best checker
    logits are closer than 2e-2 may differ)."""
    from kalosm_amd import synth
    from oracle import oracle

    ocfg = dict(cfg, type_attn=synth.Q4_K, type_ffn_gate_up=synth.Q4_K, type_ffn_down=synth.Q6_K, type_embd=synth.Q4_K,
                type_output=synth.Q6_K)
    ref = oracle.Llama(ocfg, weights)
    prompt = np.random.default_rng(99).integers(0, cfg["vocab"], prompt_len)
    model.reset()
    lg = model.forward(prompt)
    wl = ref.forward(prompt)
    diff = np.abs(lg - wl)
    ok = bool(((diff <= 1e-2) | (diff <= 1e-3 * np.maximum(np.abs(lg), np.abs(wl)))).all())
    tok = oracle.argmax(wl)
    got, _ = model.decode_greedy(tok, steps)
    want, t, agree = [], tok, 0
    for i in range(steps):
        w2 = ref.forward([t])
        srt = np.sort(w2)
        t = oracle.argmax(w2)
        want.append(t)
        if int(got[i]) != t:
            ok = ok and float(srt[-1] - srt[-2]) < 2e-2
            break
        agree += 1
    return {"ok": ok, "prompt_len": prompt_len, "logits_max_abs_err": float(diff.max()), "greedy_steps_checked": steps,
            "greedy_steps_equal": agree, "tokens": [int(x) for x in got[:steps]], "checker_tokens": want}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--trains", type=int, default=7, help="replays of each shape's K-launch train; the median is reported")
    ap.add_argument("--m", type=int, default=1, help="activation rows (decode batch) of the headline leg")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--no-e2e", action="store_true", help="skip the 8B-architecture decoder leg")
    ap.add_argument("--no-e2e-check", action="store_true", help="skip the decoder's comparison with the CPU checker")
    ap.add_argument("--no-legs", action="store_true", help="skip the batch, prefill and attention legs")
    ap.add_argument("--e2e-eager", action="store_true",
                    help="run 32 decode steps of the decoder with stream launches instead (for a kernel tracer)")
    ap.add_argument("--prefill", action="store_true", help="(default) kept for older command lines")
    ap.add_argument("--no-graph", action="store_true", help="launch on the stream instead of replaying a recorded graph")
    ap.add_argument("--calib", action="store_true",
                    help="add the device probes (dense MFMA rate, LDS read throughput, L2 next to an HBM stream) to the calibration")
    ap.add_argument("--no-calib", action="store_true",
                    help="skip the launch-floor calibration (an empty kernel and plain streaming reads of the matrices' sizes)")
    ap.add_argument("--calib-copy", action="store_true", help="append 4 device copies of 256 MiB (counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (nothing in it uses a second); run with --gpus 1",
              file=sys.stderr)
        return 2

    from kalosm_amd import synth
    from kalosm_amd.fusor import Device, Tensor

    dev = Device.gpu(0)
    info = dev.info()
    m = args.m
    ty = synth.Q4_K
    sets = matvec_sets(dev, ty, m)

    # ---- warmup, then the timed steps.  The K launches of a shape are recorded once and replayed as one submission
    # (the reference submits one command buffer per resolve); the Python/ctypes loop stays out of the device time.
    for s in sets:
        run_shape(s, args.warmup)
    dev.sync()
    per_shape_ms, all_ms, lens = [], [], []
    t_wall0 = time.perf_counter()
    for s in sets:
        L = train_length(args.steps, len(s["qs"]))
        ms, every = timed_trains(dev, lambda: run_shape(s, L, offset=args.warmup), args.trains, not args.no_graph)
        per_shape_ms.append(ms * args.steps / L)   # device time of `steps` launches at the train's rate
        all_ms.append([e * args.steps / L for e in every])
        lens.append(L)
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
    for s, ms, every in zip(sets, per_shape_ms, all_ms):
        us = ms * 1e3 / args.steps
        shapes_out.append({"n": s["n"], "k": s["k"], "us_per_launch": round(us, 3),
                           "us_per_launch_min_max": [round(min(every) * 1e3 / args.steps, 3),
                                                     round(max(every) * 1e3 / args.steps, 3)],
                           "GBps": round(s["bytes"] / (us * 1e-6) / 1e9, 1),
                           "frac_hbm_peak": round(s["bytes"] / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)})
    # dominant kernel: the Q4_K MFMA matvec k_qmv_q4k_m1, one launch per matvec (activation staging is inside it);
    # its launches are the step's four, so the per-launch average is (bytes of the four shapes / 4) over
    # (device time / launches).  Device time between events includes the dispatch gap between dependent launches.
    launches = args.steps * len(sets)
    avg_us = total_ms * 1e3 / launches
    achieved = (step_bytes / len(sets)) / (avg_us * 1e-6) / 1e9
    traffic, traffic_commit = measured_traffic()
    out = {
        "metric": "Q4_K matvec GB/s (% HBM peak); Q4_K_M 8B-arch decode tok/s, batch 1, 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "trains": args.trains,
        "ms_per_step": round(total_ms / args.steps, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: Q4_K decode matvec at Llama-3-8B layer shapes "
                               "(4096x4096, 1024x4096, 14336x4096, 4096x14336), batch %d, one launch each per step" % m,
                   "batch": m, "weights_rotated_bytes_per_shape": ROTATE_BYTES, "device": info["name"],
                   "compute_units": info["compute_units"],
                   "timing": "median of %d replays of each shape's recorded train of max(steps, weight copies, 200) = %s launches; "
                             "the figures are per launch, scaled to %d steps" % (args.trains, lens, args.steps)},
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "shapes": shapes_out,
        "wall_ms_timed_region": round(wall_ms, 2),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic if m == 1 else None,
                     "traffic_source": ("profiles/%s at commit %s" % (os.path.basename(TRAFFIC_PROFILE), traffic_commit))
                     if traffic and m == 1 else None,
                     "kernel": "k_qmv_q4k_m1", "avg_launch_us": round(avg_us, 3),
                     "algorithmic_bytes_per_launch": step_bytes // len(sets)},
    }
    rc = 0

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
        for s, x, sh in zip(sets, xs, shapes_out):
            s["x"].q_mat_mul(s["qs"][0], out=s["y"])
            e = _errs(s["y"].as_slice(), oracle.q_mat_mul(ty, x, s["raw"], s["n"], threads=threads))
            sh["parity"] = e
            if not e["ok"]:
                print("bench.py: PARITY FAILURE at shape", s["n"], s["k"], e, file=sys.stderr)
                return 1
            worst = max(worst, e["max_abs_err"])
        out["parity_max_abs_err"] = worst

    if not args.no_calib:
        # what one dependent launch costs on this device whatever the kernel does, in the same run and launch pattern
        cal = calibration(dev, args.trains, not args.no_graph, probes=args.calib)
        out["calibration"] = cal
        floor = {r["bytes"]: r["us"] for r in cal["read"]}
        tot = 0.0
        for sh in shapes_out:
            wbytes = sh["n"] * (sh["k"] // 256) * 144 // 16384 * 16384
            sh["read_floor_us"] = floor.get(wbytes)
            if sh["read_floor_us"]:
                sh["vs_read_floor"] = round(sh["us_per_launch"] / sh["read_floor_us"], 3)
                tot += sh["read_floor_us"]
        if tot:
            cal["step_read_floor_us"] = round(tot, 3)
            cal["step_read_floor_GBps"] = round(step_bytes / tot / 1e3, 1)
            cal["step_read_floor_frac_hbm_peak"] = round(step_bytes / tot / 1e3 / HBM_PEAK_GBS, 4)
            out["roofline"]["frac_of_same_run_read_floor"] = round(value / (step_bytes / tot / 1e3), 4)
    if not args.no_legs:
        out["batch"] = batch_leg(dev, sets, args.steps, args.warmup, args.trains)
    for s in sets:
        s["qs"].clear()
    del sets
    if not args.no_legs:
        out["decoder_shapes"] = decoder_shapes_leg(dev, args.steps, args.warmup, args.trains)
        out["five_bit"] = five_bit_leg(dev, args.steps, args.warmup, args.trains)
        out["prefill"] = prefill_legs(dev, max(3, min(args.trains, 5)), not args.no_graph, check=not args.no_cpu)
        if not all(e["parity"]["ok"] for grp in ("matmul", "attention", "attention_decode") for e in out["prefill"][grp]
                   if "parity" in e):
            print("bench.py: a prefill / attention leg differs from the CPU checker beyond the tolerance", file=sys.stderr)
            rc = 1

    if args.e2e_eager:
        from kalosm_amd import e2e
        out["e2e_eager"] = e2e.run(dev, steps=32, repeats=1, use_graph=False)
    elif not args.no_e2e:
        from kalosm_amd import e2e
        check = not (args.no_e2e_check or args.no_cpu)
        weights = {}
        res, model, cfg = e2e.run(dev, keep=(lambda n_, a: weights.__setitem__(n_, a)) if check else None, return_model=True)
        res["roofline"] = {"bound": "hbm", "achieved": res["weights_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": res["frac_hbm_peak"]}
        if check:
            res["checker"] = e2e_check(model, weights, cfg)
            if not res["checker"]["ok"]:
                print("bench.py: the decoder's logits / greedy tokens differ from the CPU checker's", file=sys.stderr)
                rc = 1
        out["e2e"] = res

    print(json.dumps(out))
    return rc


if __name__ == "__main__":
    sys.exit(main())
