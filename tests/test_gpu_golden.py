"""The HIP path against the committed vectors of tests/golden/ (the same file the CPU checker is held to)."""
import numpy as np
import pytest

from refgen import Q4_0, Q4_K, Q6_K, Q8_0, assert_close
from kalosm_amd import synth
from kalosm_amd.fusor import MaskKind, QMatrix, RopeCache, Tensor
from kalosm_amd.llama import Model
from test_golden import NAMES, h16, llama_from_golden

pytestmark = pytest.mark.gpu


def test_reference_stored_values(dev, golden):
    """+528 / -528, 30 / 70 and 32896 (core/src/quantized/matmul/tests.rs:1281-1423) through the C ABI."""
    x = Tensor.from_slice(dev, np.arange(1, 33, dtype=np.float32)[None, :])
    raw = np.concatenate([h16(1.0), np.full(16, 0x99, np.uint8), h16(1.0), np.full(16, 0x77, np.uint8)])
    assert np.array_equal(x.q_mat_mul(QMatrix.from_raw_bytes(dev, (2, 32), raw, Q4_0)).as_slice()[0], golden["ref_known_528"])
    raw = np.concatenate([h16(1.0), np.full(32, 1, np.uint8), h16(1.0), np.full(32, 0xFF, np.uint8)])
    assert np.array_equal(x.q_mat_mul(QMatrix.from_raw_bytes(dev, (2, 32), raw, Q8_0)).as_slice()[0], golden["ref_known_528"])
    raw = np.concatenate([h16(1.0), h16(0.0), np.uint8([1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1]), np.full(128, 0x11, np.uint8)])
    x = Tensor.from_slice(dev, np.arange(1, 257, dtype=np.float32)[None, :])
    assert x.q_mat_mul(QMatrix.from_raw_bytes(dev, (1, 256), raw, Q4_K)).as_slice()[0, 0] == golden["ref_known_32896"][0]
    w = np.float32([[1, 2, 3, 4], [5, 6, 7, 8]])
    x = Tensor.from_slice(dev, np.float32([[1, 2, 3, 4]]))
    got = x.q_mat_mul(QMatrix.from_raw_bytes(dev, (2, 4), w.view(np.uint8).reshape(-1), synth.W_F32)).as_slice()[0]
    assert np.array_equal(got, golden["ref_known_f32_30_70"])


@pytest.mark.parametrize("ty", list(NAMES))
def test_edge_blocks_bit_exact(dev, golden, ty):
    raw = golden[f"blocks_{NAMES[ty]}_raw"]
    nb = raw.size // synth.BLOCK_BYTES[ty]
    k = synth.BLOCK_ELEMS[ty]
    got = QMatrix.from_raw_bytes(dev, (nb, k), raw, ty).dequantize().as_slice()
    assert np.array_equal(got.reshape(-1).view(np.uint32), golden[f"blocks_{NAMES[ty]}_f32_bits"])


@pytest.mark.parametrize("ty", list(NAMES))
@pytest.mark.parametrize("tag", ["rand", "pattern"])
def test_matvec(dev, golden, ty, tag):
    q = QMatrix.from_raw_bytes(dev, (64, 512), golden[f"matvec_{NAMES[ty]}_{tag}_raw"], ty)
    for m in (1, 3):
        x, y = golden[f"matvec_{NAMES[ty]}_{tag}_m{m}_x"], golden[f"matvec_{NAMES[ty]}_{tag}_m{m}_y"]
        assert_close(Tensor.from_slice(dev, x).q_mat_mul(q).as_slice(), y, what=f"{NAMES[ty]} {tag} m={m}")


def test_q8_activation_path(dev, golden):
    x = Tensor.from_slice(dev, golden["q8_act_x"])
    assert np.array_equal(x.quantize_q8_0().as_slice().reshape(-1), golden["q8_act_blocks"].reshape(-1))
    q = QMatrix.from_raw_bytes(dev, (16, 128), golden["q8q8_raw"], Q8_0)
    # exact integer block sums; the f32 block terms are added as fma(f32(isum) * d_a, d_w, acc), the checker's
    # acc + f32(isum) * (d_w * d_a) differs by roundings only
    got, want = x.q_mat_mul_q8(q).as_slice(), golden["q8q8_y"]
    assert np.abs(got - want).max() <= 4e-6 * np.abs(want).max()


@pytest.mark.parametrize("tag", ["causal", "decode", "prefill"])
def test_attention(dev, golden, tag):
    q, k, v, out = (golden[f"attn_{tag}_{n}"] for n in "q k v out".split())
    causal = int(golden[f"attn_{tag}_causal"][0])
    qt, kt, vt = (Tensor.from_slice(dev, a) for a in (q, k, v))
    got = qt.flash_attention(kt, vt, 1.0 / np.sqrt(q.shape[-1]), MaskKind.Causal if causal else None).as_slice()
    assert_close(got, out, abs_tol=1e-4, rel_tol=1e-3, what=f"attention {tag}")


def test_rope_rms_swiglu(dev, golden):
    rc = RopeCache.from_parts(Tensor.from_slice(dev, golden["rope_cos"]), Tensor.from_slice(dev, golden["rope_sin"]))
    x = golden["rope_x"]
    xt = Tensor.from_slice(dev, x)
    kt = Tensor.from_slice(dev, x[:, :1].copy())
    for inter in (1, 0):
        qo, ko = (rc.forward_interleaved if inter else rc.forward)(xt, kt, 3)
        want = golden[f"rope_y_interleaved{inter}"]
        assert np.array_equal(qo.as_slice().view(np.uint32), want.view(np.uint32))
        assert np.array_equal(ko.as_slice().view(np.uint32), want[:, :1].view(np.uint32))
    built = RopeCache.new(128, 16, 500000.0, dev)
    assert np.array_equal(built.cos.as_slice().view(np.uint32), golden["rope_cos"].view(np.uint32))
    assert np.array_equal(built.sin.as_slice().view(np.uint32), golden["rope_sin"].view(np.uint32))
    xt, wt = Tensor.from_slice(dev, golden["rms_x"]), Tensor.from_slice(dev, golden["rms_w"])
    assert_close(xt.rms_norm_fused(wt, None, 1e-5).as_slice(), golden["rms_y"], abs_tol=1e-5, rel_tol=1e-5, what="rms_norm")
    got = xt.rms_norm_residual_fused(Tensor.from_slice(dev, golden["rms_res"]), wt, None, 1e-5).as_slice()
    assert_close(got, golden["rms_y_res"], abs_tol=1e-5, rel_tol=1e-5, what="rms_norm + residual")
    got = Tensor.from_slice(dev, golden["swiglu_gate"]).silu_mul(Tensor.from_slice(dev, golden["swiglu_up"])).as_slice()
    assert_close(got, golden["swiglu_y"], abs_tol=1e-6, rel_tol=1e-6, what="swiglu")


def test_tiny_decoder(dev, golden):
    cfg, seed, sigma = llama_from_golden(golden)
    m = Model.random_init(dev, cfg, seed=seed, sigma=sigma)
    lg = m.forward(golden["llama_prompt"])
    assert_close(lg, golden["llama_logits"], what="decoder logits")
    dev.set_option("deterministic", 1)  # stored tokens, no logits to judge a near tie by: no float atomics in the steps
    try:
        got, _ = m.decode_greedy(int(golden["llama_first"][0]), len(golden["llama_greedy"]))
    finally:
        dev.set_option("deterministic", 0)
    assert got.tolist() == golden["llama_greedy"].tolist()
