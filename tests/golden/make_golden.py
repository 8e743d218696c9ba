"""Writes tests/golden/fusor_golden.npz: small input / expected-output vectors for the quantized-inference path.

Run from the repository root:  python tests/golden/make_golden.py

The expected values are computed by the CPU checker (oracle/) and, before anything is written, cross-checked
against independent float64 numpy forms (tests/refgen.py); the values the reference's own tests store are
entered literally with the place they come from.  The file is data only: inputs and expected outputs.
Both the CPU tests (the checker must still reproduce them) and the GPU tests (the HIP path must match them)
load it, so the two sides cannot drift together unnoticed.
"""
from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

import refgen  # noqa: E402
from kalosm_amd import synth  # noqa: E402
from oracle import oracle  # noqa: E402

Q4_0, Q8_0, Q4_K, Q6_K = 2, 8, 12, 14
NAMES = {Q4_0: "q4_0", Q8_0: "q8_0", Q4_K: "q4_k", Q6_K: "q6_k"}


def h16(v) -> np.ndarray:
    return np.frombuffer(np.float32(v).astype(np.float16).tobytes(), np.uint8)


def h16_bits(bits: int) -> np.ndarray:
    return np.frombuffer(np.uint16(bits).tobytes(), np.uint8)


def edge_blocks(ty: int) -> np.ndarray:
    """Blocks with negative, subnormal, zero and largest-finite f16 scales; sub-scales 0 and 63 (K-quants);
    all-zero and all-0xFF codes; plus the reference's deterministic generator blocks."""
    rng = np.random.default_rng(100 + ty)
    scales = [h16(1.0), h16(-0.0173), h16_bits(0x0001), h16_bits(0x83FF), h16(0.0), h16_bits(0x7BFF), h16(-2.5)]
    blocks = []
    for i, d in enumerate(scales):
        for fill in (None, 0x00, 0xFF):
            if ty == Q4_0:
                body = rng.integers(0, 256, 16, dtype=np.uint8) if fill is None else np.full(16, fill, np.uint8)
                blocks.append(np.concatenate([d, body]))
            elif ty == Q8_0:
                body = rng.integers(0, 256, 32, dtype=np.uint8) if fill is None else np.full(32, fill, np.uint8)
                blocks.append(np.concatenate([d, body]))
            elif ty == Q4_K:
                dmin = scales[(i + 3) % len(scales)]
                sc = rng.integers(0, 64, 8, dtype=np.uint8)
                mn = rng.integers(0, 64, 8, dtype=np.uint8)
                sc[0], sc[5], mn[1], mn[6] = 0, 63, 63, 0
                body = rng.integers(0, 256, 128, dtype=np.uint8) if fill is None else np.full(128, fill, np.uint8)
                blocks.append(np.concatenate([d, dmin, synth.pack_k4_scales(sc, mn), body]))
            else:
                body = rng.integers(0, 256, 192, dtype=np.uint8) if fill is None else np.full(192, fill, np.uint8)
                sc = rng.integers(-128, 128, 16, dtype=np.int8)
                sc[0], sc[7], sc[15] = 0, 127, -128
                blocks.append(np.concatenate([body, sc.view(np.uint8), d]))
    raw = np.concatenate(blocks)
    raw = np.concatenate([raw, refgen.REF_GENERATORS[ty](4)])
    assert raw.size % refgen.BLOCK_BYTES[ty] == 0
    return raw


def main() -> None:
    oracle.build()
    g: dict[str, np.ndarray] = {}

    # ---- values the reference's own tests store
    # core/src/quantized/matmul/tests.rs:1337-1397 (+528 / -528), :1399-1423 (32896), :1281-1303 (30 / 70)
    g["ref_known_528"] = np.float32([528.0, -528.0])
    g["ref_known_32896"] = np.float32([32896.0])
    g["ref_known_f32_30_70"] = np.float32([30.0, 70.0])
    # models/kalosm-llama/src/raw/rope.rs:295-310
    g["rope_cos_sextet"] = np.float32([1.0000, 0.5403, -0.4161, -0.9900, -0.6536, 0.2837])
    g["rope_sin_sextet"] = np.float32([0.0000, 0.8415, 0.9093, 0.1411, -0.7568, -0.9589])
    # conformance/src/suite/native/rope_ops.rs:238-243
    g["rope_inv_freq_8_1e4"] = np.float32([1.0, 0.1, 0.01, 0.001])

    # ---- block decode: edge blocks per format, expected bit patterns
    for ty, nm in NAMES.items():
        raw = edge_blocks(ty)
        want = oracle.dequantize(ty, raw)
        with np.errstate(over="ignore", invalid="ignore"):
            indep = refgen.np_dequantize(ty, raw)
        assert np.array_equal(want.view(np.uint32), indep.view(np.uint32)), nm
        g[f"blocks_{nm}_raw"] = raw
        g[f"blocks_{nm}_f32_bits"] = want.view(np.uint32)

    # ---- [64, 512] matvec / small matmul per format (rows 1 and 3), random and the reference's patterned bytes
    for ty, nm in NAMES.items():
        n, k = 64, 512
        nb = n * k // refgen.BLOCK_ELEMS[ty]
        for tag, raw in (("rand", synth.random_weight(ty, n, k, seed=40 + ty)), ("pattern", refgen.REF_GENERATORS[ty](nb))):
            for m in (1, 3):
                x = synth.random_activation(m, k, seed=50 + m) if tag == "rand" else \
                    np.stack([refgen.deterministic_input(k, 7 * r) for r in range(m)])
                y = oracle.q_mat_mul(ty, x, raw, n)
                y64 = refgen.np_matmul_f64(ty, x, raw, n)
                assert np.abs(y - y64).max() <= 2e-5 * max(1.0, np.abs(y64).max()), (nm, tag, m)
                g[f"matvec_{nm}_{tag}_m{m}_x"] = x
                g[f"matvec_{nm}_{tag}_m{m}_y"] = y
            g[f"matvec_{nm}_{tag}_raw"] = raw

    # ---- Q8_0 activation blocks and the integer product
    x = synth.random_activation(2, 128, seed=60) * 3
    x[0, :32] = 0.0                                   # an all-zero block
    qa = oracle.q8_0_quantize(x)
    g["q8_act_x"], g["q8_act_blocks"] = x, qa
    raw = synth.random_weight(Q8_0, 16, 128, seed=61)
    y = oracle.q8_0_matmul_q8(x, raw, 16)
    g["q8q8_raw"], g["q8q8_y"] = raw, y

    # ---- attention: grouped heads, causal with a cache offset, unmasked single query
    rng = np.random.default_rng(70)
    for tag, (h, hkv, sq, skv, d, causal) in dict(causal=(4, 2, 6, 9, 64, True), decode=(8, 2, 1, 37, 128, False),
                                                  prefill=(2, 1, 33, 33, 128, True)).items():
        q = rng.standard_normal((1, h, sq, d)).astype(np.float32)
        k = rng.standard_normal((1, hkv, skv, d)).astype(np.float32)
        v = rng.standard_normal((1, hkv, skv, d)).astype(np.float32)
        sc = np.float32(1.0 / np.sqrt(d))
        out = oracle.flash_attention(q, k, v, float(sc), 1 if causal else 0)
        assert np.abs(out - refgen.np_attention(q, k, v, float(sc), causal=causal)).max() < 2e-5, tag
        for nm_, a in (("q", q), ("k", k), ("v", v), ("out", out)):
            g[f"attn_{tag}_{nm_}"] = a
        g[f"attn_{tag}_causal"] = np.int32([int(causal)])

    # ---- RoPE rotation (both pairings, start_pos 3) on the Llama-3 tables
    cos, sin = oracle.rope_tables(128, 16, 500000.0)
    x = rng.standard_normal((1, 3, 4, 128)).astype(np.float32)
    for inter in (1, 0):
        y = oracle.rope(x, cos, sin, 3, bool(inter))
        z = (x[..., 0::2] + 1j * x[..., 1::2]) if inter else (x[..., :64] + 1j * x[..., 64:])
        w = z.astype(np.complex128) * (cos[3:7].astype(np.float64) + 1j * sin[3:7].astype(np.float64))[None, None]
        chk = np.empty(x.shape)
        if inter:
            chk[..., 0::2], chk[..., 1::2] = w.real, w.imag
        else:
            chk[..., :64], chk[..., 64:] = w.real, w.imag
        assert np.abs(y - chk).max() < 1e-6
        g[f"rope_y_interleaved{inter}"] = y
    g["rope_x"], g["rope_cos"], g["rope_sin"] = x, cos, sin

    # ---- rms_norm (plain and residual) and SwiGLU
    x = (rng.standard_normal((3, 512)) * 2).astype(np.float32)
    r = rng.standard_normal((3, 512)).astype(np.float32)
    w = (1 + (np.arange(512) % 5) * 0.25).astype(np.float32)
    g["rms_x"], g["rms_res"], g["rms_w"] = x, r, w
    g["rms_y"] = oracle.rms_norm(x, w, 1e-5)
    g["rms_y_res"] = oracle.rms_norm(x, w, 1e-5, residual=r)
    t = x.astype(np.float64) + r
    assert np.abs(g["rms_y_res"] - t / np.sqrt((t * t).mean(1, keepdims=True) + 1e-5) * w).max() < 1e-5
    gate = (rng.standard_normal(1024) * 4).astype(np.float32)
    up = rng.standard_normal(1024).astype(np.float32)
    g["swiglu_gate"], g["swiglu_up"], g["swiglu_y"] = gate, up, oracle.swiglu(gate, up)
    g64 = gate.astype(np.float64)
    assert np.abs(g["swiglu_y"] - g64 / (1 + np.exp(-g64)) * up).max() < 1e-5

    # ---- a tiny decoder (weights regenerate from the seed: synth.llama_random_tensor): prompt logits and greedy ids
    cfg = dict(n_layers=2, d_model=256, n_heads=4, n_kv_heads=2, head_dim=64, ffn=512, vocab=320, ctx=64, eps=1e-5,
               theta=500000.0)
    weights = {name: synth.llama_random_tensor(name, ty, n, k, 21, 0.02) for name, ty, n, k in synth.llama_tensor_specs(cfg)}
    ref = oracle.Llama(dict(cfg, type_attn=Q4_K, type_ffn_gate_up=Q4_K, type_ffn_down=Q6_K, type_embd=Q4_K,
                            type_output=Q6_K), weights)
    prompt = np.random.default_rng(22).integers(0, cfg["vocab"], 9).astype(np.uint32)
    logits = ref.forward(prompt)
    toks, t = [], oracle.argmax(logits)
    first = t
    for _ in range(8):
        t = oracle.argmax(ref.forward([t]))
        toks.append(t)
    g["llama_cfg"] = np.float64([cfg[k_] for k_ in ("n_layers", "d_model", "n_heads", "n_kv_heads", "head_dim", "ffn", "vocab",
                                                    "ctx", "eps", "theta")])
    g["llama_seed_sigma"] = np.float64([21, 0.02])
    g["llama_prompt"], g["llama_logits"] = prompt, logits
    g["llama_first"], g["llama_greedy"] = np.uint32([first]), np.uint32(toks)

    out = os.path.join(HERE, "fusor_golden.npz")
    np.savez_compressed(out, **g)
    print(f"wrote {out}: {len(g)} arrays, {os.path.getsize(out)} bytes")


if __name__ == "__main__":
    main()
