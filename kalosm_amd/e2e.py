"""End-to-end run of the Llama-3-8B-architecture decoder with random-init Q4_K_M weights: a 512-token prompt of
uniform-random ids, then greedy decode steps at batch 1, timed on the device."""
from __future__ import annotations

import time

import numpy as np

from . import synth
from .llama import Model


def run(dev, cfg: dict | None = None, prompt_len: int = 512, steps: int = 256, seed: int = 0, sigma: float = 1e-4,
        kv_dtype: str = "f32", repeats: int = 3, prefill_chunk: int = 512, use_graph: bool = True,
        sampled: bool = True, keep=None, return_model: bool = False):
    """`keep(name, array)` receives every weight tensor as it is generated (for a caller that checks the decoder
    against something else afterwards); with return_model the result is (report, model, cfg)."""
    cfg = dict(cfg or synth.LLAMA3_8B)
    t0 = time.perf_counter()
    m = Model.random_init(dev, cfg, seed=seed, sigma=sigma, kv_dtype=kv_dtype, use_graph=use_graph, keep=keep)
    load_s = time.perf_counter() - t0
    rng = np.random.default_rng(seed + 1)
    prompt = rng.integers(0, cfg["vocab"], prompt_len)
    import statistics
    best = None
    toks = None
    prefill_ms = None
    runs = []
    for rep in range(repeats + 1):  # the first run captures the decode step and is not counted; the others replay it
        m.reset()
        t0 = time.perf_counter()
        lg = None
        for i in range(0, prompt_len, prefill_chunk):
            lg = m.forward(prompt[i:i + prefill_chunk])
        prefill_ms = (time.perf_counter() - t0) * 1e3
        first = int(np.argmax(lg))
        out, ms = m.decode_greedy(first, steps)
        toks = out
        if rep > 0:
            runs.append(ms)
    best = statistics.median(runs)  # the reported figure is the median repeat, not the best
    wbytes = m.weight_bytes()
    tok_s = steps / (best * 1e-3)
    samp = None
    if sampled:
        # the same steps with the reference's default generation parameters (Mirostat 2: temperature 0.8, tau 5,
        # eta 0.1, mu 10, window of 64 previous ids) and a repetition penalty of 1.3 over the 64 best candidates
        from .fusor import GpuMirostat2SamplerParams
        params = GpuMirostat2SamplerParams(64, 0.8, 1.3, 5.0, 0.1, 0.0)
        sruns, stoks = [], None
        for rep in range(repeats + 1):
            m.reset()
            lg = None
            for i in range(0, prompt_len, prefill_chunk):
                lg = m.forward(prompt[i:i + prefill_chunk])
            randoms = np.random.default_rng(seed + 2).random(steps).astype(np.float32)
            out, ms, mu = m.decode_sampled(int(np.argmax(lg)), steps, params, randoms, previous_tokens=prompt,
                                           repetition_range=64, mu=10.0)
            stoks = out
            if rep > 0:
                sruns.append(ms)
        sbest = statistics.median(sruns)
        samp = {"sampler": "mirostat2 top_k 64 temperature 0.8 penalty 1.3 window 64", "tok_per_s": round(steps / (sbest * 1e-3), 1),
                "ms_per_token": round(sbest / steps, 4), "distinct_tokens": int(len(set(stoks.tolist())))}
    report = {"tok_per_s": round(tok_s, 1), "ms_per_token": round(best / steps, 4), "steps": steps, "repeats": repeats,
            "ms_per_token_repeats": [round(r / steps, 4) for r in runs], "prompt_len": prompt_len, "graph_replay": use_graph, "prefill_ms_host_clock": round(prefill_ms, 1), "kv_dtype": kv_dtype,
            "weight_bytes_per_token": wbytes, "weights_GBps": round(wbytes * tok_s / 1e9, 1),
            "frac_hbm_peak": round(wbytes * tok_s / 8e12, 4), "load_seconds": round(load_s, 1),
            "first_tokens": [int(t) for t in toks[:8]], "config": {k: cfg[k] for k in ("n_layers", "d_model", "ffn", "vocab")},
            "sampled": samp}
    return (report, m, cfg) if return_model else report
