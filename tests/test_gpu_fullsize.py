"""GPU parity at the full sizes of the benchmark configurations: direct comparison with the CPU checker where it
finishes in seconds, size-independent properties where it does not."""
import numpy as np
import pytest

import refgen
from refgen import Q4_0, Q4_K, Q6_K, Q8_0, assert_close, assert_greedy_follows
from kalosm_amd import synth
from kalosm_amd.fusor import MaskKind, QMatrix, Tensor
from kalosm_amd.llama import Model

pytestmark = pytest.mark.gpu
NAMES = synth.TYPE_NAMES
LLAMA_SHAPES = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)]


def test_config0_q4_0_single_matvec(dev, oracle):
    """configs[0]: 4096 x 4096 Q4_0, f16 scales N(0, 0.02), uniform nibbles, x ~ N(0, 1), batch 1."""
    n = k = 4096
    raw = synth.random_weight(Q4_0, n, k, seed=1)
    x = synth.random_activation(1, k, seed=2)
    got = Tensor.from_slice(dev, x).q_mat_mul(QMatrix.from_raw_bytes(dev, (n, k), raw, Q4_0)).as_slice()
    assert_close(got, oracle.q_mat_mul(Q4_0, x, raw, n), what="Q4_0 4096x4096")


@pytest.mark.parametrize("m", [1, 4, 16])
@pytest.mark.parametrize("n,k", LLAMA_SHAPES)
def test_config1_q4k_llama_shapes(dev, oracle, n, k, m):
    """configs[1]: Q4_K at the four Llama-3-8B layer shapes, batch 1, 4 and 16, against the checker."""
    raw = synth.random_weight(Q4_K, n, k, seed=n + k)
    x = synth.random_activation(m, k, seed=m)
    out = Tensor.filled_bytes(dev, (m, n), 0xFF)
    got = Tensor.from_slice(dev, x).q_mat_mul(QMatrix.from_raw_bytes(dev, (n, k), raw, Q4_K), out=out).as_slice()
    assert_close(got, oracle.q_mat_mul(Q4_K, x, raw, n, fast=True), what=f"Q4_K {n}x{k} m={m}")


@pytest.mark.parametrize("ty", [Q6_K, Q8_0], ids=lambda t: NAMES[t])
def test_config1_other_formats_down_shape(dev, oracle, ty):
    """The long-k shape (4096 x 14336) in the other formats of a Q4_K_M / Q8_0 file, batch 1 and 16."""
    n, k = 4096, 14336
    raw = synth.random_weight(ty, n, k, seed=77)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    for m in (1, 16):
        x = synth.random_activation(m, k, seed=m)
        got = Tensor.from_slice(dev, x).q_mat_mul(q).as_slice()
        assert_close(got, oracle.q_mat_mul(ty, x, raw, n, fast=True), what=f"{NAMES[ty]} m={m}")


@pytest.mark.parametrize("s", [512, 2048, 8192])
def test_config3_causal_attention_long(dev, oracle, s):
    """configs[3] at seq 512, 2048 and 8192 (32 / 8 heads, d = 128, f16).  The checker would need minutes, so: 24 sampled
    query rows per length (first, last, tile and block boundaries, random) against the float64 textbook form computed
    for those rows only, plus the exact property that causal row 0 returns v_0."""
    h, hkv, d = 32, 8, 128
    rng = np.random.default_rng(s)
    q = rng.standard_normal((1, h, s, d)).astype(np.float16)
    k = rng.standard_normal((1, hkv, s, d)).astype(np.float16)
    v = rng.standard_normal((1, hkv, s, d)).astype(np.float16)
    scale = 1 / np.sqrt(d)
    qt, kt, vt = (Tensor.from_slice(dev, a, "f16") for a in (q, k, v))
    got = qt.flash_attention(kt, vt, scale, MaskKind.Causal).as_slice().astype(np.float32)
    assert np.isfinite(got).all()
    rows = sorted(set([0, 1, 31, 32, 63, 64, 127, 128, 129, s // 2 - 1, s // 2, s - 129, s - 128, s - 65, s - 64, s - 2,
                       s - 1] + rng.integers(0, s, 7).tolist()))
    kf, vf = k.astype(np.float64), v.astype(np.float64)
    for hh in (0, 5, 31):
        kh = hh // (h // hkv)
        for i in rows:
            sc = (q[0, hh, i].astype(np.float64) @ kf[0, kh, :i + 1].T) * scale
            p = np.exp(sc - sc.max())
            want = (p / p.sum()) @ vf[0, kh, :i + 1]
            assert_close(got[0, hh, i], want.astype(np.float32), abs_tol=1e-2, rel_tol=1e-3, what=f"s={s} head {hh} row {i}")
    assert_close(got[0, :, 0], np.repeat(v[0, :, 0].astype(np.float32), h // hkv, axis=0), abs_tol=1e-3, rel_tol=1e-3,
                 what="row 0 sees v_0 only")


@pytest.mark.parametrize("L", [1024, 4096, 16384])
def test_config3_decode_attention_long_cache(dev, oracle, L):
    """configs[3] decode variant: one query against 1024 / 4096 / 16384 cached keys (f16, 32 / 8 heads, d = 128)."""
    h, hkv, d = 32, 8, 128
    rng = np.random.default_rng(L)
    q = rng.standard_normal((1, h, 1, d)).astype(np.float16)
    k = rng.standard_normal((1, hkv, L, d)).astype(np.float16)
    v = rng.standard_normal((1, hkv, L, d)).astype(np.float16)
    qt, kt, vt = (Tensor.from_slice(dev, a, "f16") for a in (q, k, v))
    got = qt.flash_attention(kt, vt, 1 / np.sqrt(d)).as_slice().astype(np.float32)
    want = oracle.flash_attention(*(a.astype(np.float32) for a in (q, k, v)), 1 / np.sqrt(d))
    assert_close(got, want, abs_tol=1e-2, rel_tol=1e-3, what=f"decode L={L}")


def test_config4_decoder_full_width(dev, oracle):
    """configs[4] at the real layer widths (d_model 4096, ffn 14336, 32 / 8 heads of 128, vocab 128256, Q4_K attention
    and gate / up, Q6_K down and output) with 2 layers instead of 32 so that the checker's decoder runs in seconds:
    prefill logits of a 40-token prompt, 12 greedy steps on the device, and the logits after them."""
    cfg = dict(synth.LLAMA3_8B, n_layers=2, ctx=1024)
    weights = {}
    m = Model.random_init(dev, cfg, seed=3, sigma=2e-4, keep=lambda n, a: weights.__setitem__(n, a))
    ocfg = dict(cfg, type_attn=synth.Q4_K, type_ffn_gate_up=synth.Q4_K, type_ffn_down=synth.Q6_K, type_embd=synth.Q4_K,
                type_output=synth.Q6_K)
    ref = oracle.Llama(ocfg, weights)
    prompt = np.random.default_rng(4).integers(0, cfg["vocab"], 40)
    lg = m.forward(prompt)
    wl = ref.forward(prompt)
    assert_close(lg, wl, what="prefill logits, full width")
    tok = int(np.argmax(wl))
    got, _ = m.decode_greedy(tok, 12)
    assert_greedy_follows(ref, tok, got)
    last = int(got[-1])
    assert_close(m.forward([last]), ref.forward([last]), what="logits after 12 device-side steps")


def test_config4_prompt_and_step_counts_of_the_benchmark(dev, oracle):
    """configs[4] at the lengths the benchmark times - a 512-token prompt in ONE forward pass (256-row tiles, k split
    over workgroups, plane sums, split-operand f32 attention) and 256 greedy steps on the device (cache positions
    512 .. 767: every boundary of the attention's key splits in that range) - on 2 layers at the real widths and a
    vocabulary of 16384 (the 128256-row output matrix is covered by the tests above), so that the checker's decoder
    finishes in a minute: prefill logits, every one of the 256 picks against the checker fed with the same tokens,
    and the logits after them."""
    cfg = dict(synth.LLAMA3_8B, n_layers=2, ctx=1024, vocab=16384)
    weights = {}
    m = Model.random_init(dev, cfg, seed=11, sigma=2e-4, keep=lambda n, a: weights.__setitem__(n, a))
    ocfg = dict(cfg, type_attn=synth.Q4_K, type_ffn_gate_up=synth.Q4_K, type_ffn_down=synth.Q6_K, type_embd=synth.Q4_K,
                type_output=synth.Q6_K)
    ref = oracle.Llama(ocfg, weights)
    prompt = np.random.default_rng(12).integers(0, cfg["vocab"], 512)
    lg = m.forward(prompt)
    wl = ref.forward(prompt)
    assert_close(lg, wl, what="logits of the 512-token prompt")
    tok = oracle.argmax(wl)
    got, _ = m.decode_greedy(tok, 256)
    same = assert_greedy_follows(ref, tok, got, what="256 steps after a 512-token prompt")
    assert same >= 200, f"only {same} of 256 picks were the checker's own"
    last = int(got[-1])
    assert_close(m.forward([last]), ref.forward([last]), what="logits at position 768")


def test_decoder_from_gguf_file_full_width(dev, oracle, tmp_path):
    """The model-file path at real tensor sizes: a 1 GB GGUF file (2 layers at Llama-3-8B widths, vocabulary 128256,
    the per-layer type mix of a Q4_K_M file, rope_freqs.weight) written to disk, mapped and loaded by the library,
    against the checker's decoder fed from the same bytes."""
    from test_gguf_reader import llama_file
    from kalosm_amd.gguf import GgufMetadata
    cfg = {k: synth.LLAMA3_8B[k] for k in ("d_model", "n_heads", "n_kv_heads", "head_dim", "ffn", "vocab", "eps", "theta")}
    cfg.update(n_layers=2, ctx=8192)
    data, weights, types = llama_file(cfg, seed=6)
    path = tmp_path / "llama_2_layers.gguf"
    path.write_bytes(data)
    assert len(data) > 900_000_000
    del data
    g = GgufMetadata.read(str(path))
    assert g.get_value(".context_length") == 8192 and len(g.tensor_infos) == 3 + 1 + 9 * 2
    m = Model.from_gguf(dev, g, ctx=512)
    assert m.cfg["vocab"] == 128256 and m.cfg["ffn"] == 14336 and m.cfg["ctx"] == 512
    ocfg = dict(m.cfg, type_attn=synth.Q4_K, type_ffn_gate_up=synth.Q4_K, type_ffn_down=synth.Q6_K,
                type_embd=types["token_embd.weight"], type_output=types["output.weight"], tensor_types=types)
    ref = oracle.Llama(ocfg, weights)
    prompt = np.random.default_rng(7).integers(0, cfg["vocab"], 24)
    lg, wl = m.forward(prompt), ref.forward(prompt)
    assert_close(lg, wl, what="prefill logits from the model file")
    tok = oracle.argmax(wl)
    got, _ = m.decode_greedy(tok, 8)
    assert_greedy_follows(ref, tok, got, what="decoder from the model file")


def test_config4_decoder_all_32_layers(dev, oracle):
    """configs[4] at its real depth and widths: the 32-layer Llama-3-8B-architecture decoder with random-init Q4_K_M
    weights against the checker's decoder on the same weights: prefill logits of a 48-token prompt, 16 greedy steps
    replayed on the device, and the logits after them.  The checker needs about a second per token."""
    cfg = dict(synth.LLAMA3_8B, ctx=1024)
    weights = {}
    m = Model.random_init(dev, cfg, seed=0, sigma=1e-4, keep=lambda n, a: weights.__setitem__(n, a))
    ocfg = dict(cfg, type_attn=synth.Q4_K, type_ffn_gate_up=synth.Q4_K, type_ffn_down=synth.Q6_K, type_embd=synth.Q4_K,
                type_output=synth.Q6_K)
    ref = oracle.Llama(ocfg, weights)
    prompt = np.random.default_rng(1).integers(0, cfg["vocab"], 32)
    lg = m.forward(prompt)
    wl = ref.forward(prompt)
    assert_close(lg, wl, what="prefill logits, 32 layers")
    tok = oracle.argmax(wl)
    steps = 12
    got, _ = m.decode_greedy(tok, steps)
    want, t = [], tok
    margins = []
    for _ in range(steps):
        wl = ref.forward([t])
        srt = np.sort(wl)
        margins.append(float(srt[-1] - srt[-2]))
        t = oracle.argmax(wl)
        want.append(t)
    # a greedy pick is only defined up to the logit tolerance: a step whose two best logits are closer than 2e-2
    # may legitimately differ, and every later token with it
    for i, (g, w_) in enumerate(zip(got.tolist(), want)):
        if g != w_:
            assert margins[i] < 2e-2, f"step {i}: {g} != {w_} with a margin of {margins[i]}"
            break
    else:
        assert_close(m.forward([want[-1]]), ref.forward([want[-1]]), what="logits after 12 device-side steps, 32 layers")
