"""The CPU checker against the committed vectors of tests/golden/: the checker of today must still give what
the fixture generator wrote (and cross-checked against float64 numpy) when the file was made."""
import numpy as np
import pytest

import refgen
from refgen import Q4_0, Q4_K, Q6_K, Q8_0
from kalosm_amd import synth

NAMES = {Q4_0: "q4_0", Q8_0: "q8_0", Q4_K: "q4_k", Q6_K: "q6_k"}


def h16(v):
    return np.frombuffer(np.float32(v).astype(np.float16).tobytes(), np.uint8)


def test_reference_stored_values(oracle, golden):
    """The numbers the reference's tests store: +528 / -528 (core/src/quantized/matmul/tests.rs:1337-1397), 30 / 70 for
    f32 weights (:1281-1303), 32896 for the unit-scale K-quant block (:1399-1423)."""
    x = np.arange(1, 33, dtype=np.float32)[None, :]
    raw = np.concatenate([h16(1.0), np.full(16, 0x99, np.uint8), h16(1.0), np.full(16, 0x77, np.uint8)])
    assert np.array_equal(oracle.q_mat_mul(Q4_0, x, raw, 2)[0], golden["ref_known_528"])
    raw = np.concatenate([h16(1.0), np.full(32, 1, np.uint8), h16(1.0), np.full(32, 0xFF, np.uint8)])
    assert np.array_equal(oracle.q_mat_mul(Q8_0, x, raw, 2)[0], golden["ref_known_528"])
    raw = np.concatenate([h16(1.0), h16(0.0), np.uint8([1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1]), np.full(128, 0x11, np.uint8)])
    y = oracle.q_mat_mul(Q4_K, np.arange(1, 257, dtype=np.float32)[None, :], raw, 1)
    assert y[0, 0] == golden["ref_known_32896"][0]
    w = np.float32([[1, 2, 3, 4], [5, 6, 7, 8]])           # rows of an F32 "quantized" matrix, x = 1..4
    y = oracle.q_mat_mul(synth.W_F32, np.float32([[1, 2, 3, 4]]), w.view(np.uint8).reshape(-1), 2)
    assert np.array_equal(y[0], golden["ref_known_f32_30_70"])


@pytest.mark.parametrize("ty", list(NAMES))
def test_edge_blocks(oracle, golden, ty):
    raw = golden[f"blocks_{NAMES[ty]}_raw"]
    assert np.array_equal(oracle.dequantize(ty, raw).view(np.uint32), golden[f"blocks_{NAMES[ty]}_f32_bits"])


@pytest.mark.parametrize("ty", list(NAMES))
@pytest.mark.parametrize("tag", ["rand", "pattern"])
def test_matvec(oracle, golden, ty, tag):
    raw = golden[f"matvec_{NAMES[ty]}_{tag}_raw"]
    for m in (1, 3):
        x, y = golden[f"matvec_{NAMES[ty]}_{tag}_m{m}_x"], golden[f"matvec_{NAMES[ty]}_{tag}_m{m}_y"]
        got = oracle.q_mat_mul(ty, x, raw, 64)
        assert np.abs(got - y).max() <= 1e-6 * max(1.0, np.abs(y).max())
        assert np.abs(refgen.np_matmul_f64(ty, x, raw, 64) - y).max() <= 2e-5 * max(1.0, np.abs(y).max())


def test_q8_activation_path(oracle, golden):
    assert np.array_equal(oracle.q8_0_quantize(golden["q8_act_x"]), golden["q8_act_blocks"])
    assert np.array_equal(oracle.q8_0_matmul_q8(golden["q8_act_x"], golden["q8q8_raw"], 16), golden["q8q8_y"])


@pytest.mark.parametrize("tag", ["causal", "decode", "prefill"])
def test_attention(oracle, golden, tag):
    q, k, v, out = (golden[f"attn_{tag}_{n}"] for n in "q k v out".split())
    causal = int(golden[f"attn_{tag}_causal"][0])
    got = oracle.flash_attention(q, k, v, float(np.float32(1.0 / np.sqrt(q.shape[-1]))), causal)
    assert np.abs(got - out).max() < 1e-6
    assert np.abs(refgen.np_attention(q, k, v, 1.0 / np.sqrt(q.shape[-1]), causal=bool(causal)) - out).max() < 2e-5


def test_rope_rms_swiglu(oracle, golden):
    for inter in (1, 0):
        got = oracle.rope(golden["rope_x"], golden["rope_cos"], golden["rope_sin"], 3, bool(inter))
        assert np.array_equal(got, golden[f"rope_y_interleaved{inter}"])
    cos, sin = oracle.rope_tables(128, 16, 500000.0)
    assert np.abs(cos - golden["rope_cos"]).max() < 1e-6 and np.abs(sin - golden["rope_sin"]).max() < 1e-6
    assert np.abs(oracle.rms_norm(golden["rms_x"], golden["rms_w"], 1e-5) - golden["rms_y"]).max() < 1e-6
    got = oracle.rms_norm(golden["rms_x"], golden["rms_w"], 1e-5, residual=golden["rms_res"])
    assert np.abs(got - golden["rms_y_res"]).max() < 1e-6
    assert np.abs(oracle.swiglu(golden["swiglu_gate"], golden["swiglu_up"]) - golden["swiglu_y"]).max() < 1e-6


def llama_from_golden(golden):
    keys = ("n_layers", "d_model", "n_heads", "n_kv_heads", "head_dim", "ffn", "vocab", "ctx", "eps", "theta")
    vals = golden["llama_cfg"]
    cfg = {k: (float(v) if k in ("eps", "theta") else int(v)) for k, v in zip(keys, vals)}
    seed, sigma = int(golden["llama_seed_sigma"][0]), float(golden["llama_seed_sigma"][1])
    return cfg, seed, sigma


def test_tiny_decoder(oracle, golden):
    cfg, seed, sigma = llama_from_golden(golden)
    weights = {name: synth.llama_random_tensor(name, ty, n, k, seed, sigma) for name, ty, n, k in synth.llama_tensor_specs(cfg)}
    ref = oracle.Llama(dict(cfg, type_attn=Q4_K, type_ffn_gate_up=Q4_K, type_ffn_down=Q6_K, type_embd=Q4_K,
                            type_output=Q6_K), weights)
    lg = ref.forward(golden["llama_prompt"])
    assert np.abs(lg - golden["llama_logits"]).max() <= 1e-5 * max(1.0, np.abs(lg).max())
    t = oracle.argmax(lg)
    assert t == int(golden["llama_first"][0])
    for want in golden["llama_greedy"]:
        t = oracle.argmax(ref.forward([t]))
        assert t == int(want)
