"""Pins the CPU checker's composites (RoPE rotation, silu / SwiGLU, embedding gather, causal mask, attention,
rms_norm, greedy pick, the decoder) against closed forms, library routines and an independent float64 numpy
decoder.  Nothing here shares code with the C checker: a dropped term, a swapped pair or a wrong sign in it fails
one of these."""
import numpy as np
import pytest

import refgen
from refgen import Q4_K, Q6_K, Q8_0, Q4_0
from kalosm_amd import synth


# ------------------------------------------------------------------------------------------- RoPE rotation
def _angles(ctx, half, rng):
    """Arbitrary (not geometric) angles, so a wrong pair index cannot hide behind equal frequencies."""
    return rng.uniform(-3.0, 3.0, (ctx, half))


@pytest.mark.parametrize("interleaved", [True, False], ids=["interleaved", "half-split"])
@pytest.mark.parametrize("start_pos", [0, 5])
def test_rope_is_complex_multiplication(oracle, interleaved, start_pos):
    """fusor/src/composite/rope.rs:46-108: the pair (x0, x1) at angle t becomes (x0 + i x1) * e^{it}; interleaved pairs
    are (2i, 2i+1), half-split pairs are (i, i + d/2); rows start_pos .. start_pos + s of the tables."""
    rng = np.random.default_rng(3)
    b, h, s, d, ctx = 2, 3, 4, 16, 12
    ang = _angles(ctx, d // 2, rng)
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    x = rng.standard_normal((b, h, s, d)).astype(np.float32)
    y = oracle.rope(x, cos, sin, start_pos, interleaved)
    x64 = x.astype(np.float64)
    if interleaved:
        z = x64[..., 0::2] + 1j * x64[..., 1::2]
    else:
        z = x64[..., : d // 2] + 1j * x64[..., d // 2:]
    rot = (cos[start_pos:start_pos + s].astype(np.float64) + 1j * sin[start_pos:start_pos + s].astype(np.float64))
    w = z * rot[None, None]
    want = np.empty_like(x64)
    if interleaved:
        want[..., 0::2], want[..., 1::2] = w.real, w.imag
    else:
        want[..., : d // 2], want[..., d // 2:] = w.real, w.imag
    assert np.abs(y - want).max() < 1e-6
    # the rotation preserves each pair's length and depends on the position
    assert np.allclose(np.abs(w), np.abs(z))
    assert not np.allclose(y[:, :, 0], y[:, :, 1] if s > 1 else 0)


def test_rope_unit_vectors_fix_signs_and_pairing(oracle):
    """(1, 0) at angle t -> (cos t, sin t); (0, 1) -> (-sin t, cos t): fixes the sign of the sine terms and which
    element is the pair's partner in both layouts."""
    d, half = 8, 4
    ang = np.array([[0.3, 0.7, 1.1, 1.9]])
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    for interleaved in (True, False):
        for i in range(half):
            a, bidx = (2 * i, 2 * i + 1) if interleaved else (i, i + half)
            x = np.zeros((1, 1, 1, d), np.float32)
            x[..., a] = 1.0
            y = oracle.rope(x, cos, sin, 0, interleaved).reshape(d)
            want = np.zeros(d, np.float32)
            want[a], want[bidx] = cos[0, i], sin[0, i]
            assert np.array_equal(y, want), (interleaved, i)
            x = np.zeros((1, 1, 1, d), np.float32)
            x[..., bidx] = 1.0
            y = oracle.rope(x, cos, sin, 0, interleaved).reshape(d)
            want = np.zeros(d, np.float32)
            want[a], want[bidx] = -sin[0, i], cos[0, i]
            assert np.array_equal(y, want), (interleaved, i)


def test_rope_matches_the_reference_host_forms(oracle):
    """conformance/src/common/mod.rs:593-653 (rope_normal_4d, rope_interleaved_4d) restated in f32 with the same
    operation order: bit-equal, since each product is rounded before the add / sub in both."""
    rng = np.random.default_rng(8)
    b, h, s, d = 1, 2, 5, 12
    cos = rng.uniform(-1, 1, (s, d // 2)).astype(np.float32)
    sin = rng.uniform(-1, 1, (s, d // 2)).astype(np.float32)
    x = rng.standard_normal((b, h, s, d)).astype(np.float32)
    c, sn = cos[None, None], sin[None, None]
    x0, x1 = x[..., 0::2], x[..., 1::2]
    want = np.empty_like(x)
    want[..., 0::2] = x0 * c - x1 * sn
    want[..., 1::2] = x0 * sn + x1 * c
    assert np.array_equal(oracle.rope(x, cos, sin, 0, True), want)
    half = d // 2
    x0, x1 = x[..., :half], x[..., half:]
    want[..., :half] = x0 * c - x1 * sn
    want[..., half:] = x1 * c + x0 * sn
    assert np.array_equal(oracle.rope(x, cos, sin, 0, False), want)


def test_rope_tables_goldens(oracle, golden):
    """models/kalosm-llama/src/raw/rope.rs:295-310 (head_dim 2, theta 5000, six positions; summed abs error < 1e-2
    there) and conformance rope_ops.rs:238-243 (base_inverse_frequency(8, 1e4), compared exactly there)."""
    cos, sin = oracle.rope_tables(2, 6, 5000.0)
    assert np.abs(cos.reshape(-1) - golden["rope_cos_sextet"]).sum() < 1e-3
    assert np.abs(sin.reshape(-1) - golden["rope_sin_sextet"]).sum() < 1e-3
    inv = oracle.rope_inverse_frequency(8, 10000.0)
    want = np.float32(1.0) / np.power(np.float32(10000.0), np.float32([0, 2, 4, 6]) / np.float32(8))
    assert np.abs(inv - want).max() <= 1e-7 and inv[0] == 1.0
    assert np.allclose(inv, golden["rope_inv_freq_8_1e4"], rtol=1e-6)


def test_rope_tables_compose(oracle):
    """Angle of position p is p * inv: rotating by the rows of positions a then b equals the row of a + b."""
    cos, sin = oracle.rope_tables(64, 40, 500000.0)
    z = cos.astype(np.float64) + 1j * sin.astype(np.float64)
    assert np.abs(z[7] * z[13] - z[20]).max() < 2e-6
    assert np.abs(np.abs(z) - 1).max() < 1e-6


# ------------------------------------------------------------------------------------------- activations
def test_silu_and_swiglu_closed_form(oracle):
    """fusor/src/composite/activations.rs:47-65, conformance common/mod.rs:417-419: x / (1 + exp(-x))."""
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(4000) * 4, [0.0, 1.0, -1.0, 30.0, -30.0, 88.0, -88.0, 100.0, -100.0]]).astype(np.float32)
    y = oracle.silu(x)
    x64 = x.astype(np.float64)
    with np.errstate(over="ignore"):
        want = x64 / (1.0 + np.exp(-x64))
    assert np.abs(y - want).max() <= 2e-6 * max(1.0, np.abs(want).max())
    i = {v: int(np.where(x == np.float32(v))[0][0]) for v in (0.0, 1.0, -1.0, 100.0, -100.0)}
    assert y[i[0.0]] == 0.0 and y[i[100.0]] == 100.0 and y[i[-100.0]] == 0.0
    assert y[i[1.0]] == pytest.approx(0.7310585786, abs=1e-7) and y[i[-1.0]] == pytest.approx(-0.2689414214, abs=1e-7)
    up = rng.standard_normal(x.size).astype(np.float32)
    g = oracle.swiglu(x, up)
    assert np.array_equal(g, y * up)          # raw/attention_layer.rs:186-196: silu(gate) * up, one rounding each
    assert not np.allclose(g, oracle.swiglu(up, x))   # gate and up are not interchangeable


def test_add3_order(oracle):
    a = np.float32([1e8, 1.0]); b = np.float32([-1e8, 1e8]); c = np.float32([1.0, -1e8])
    assert oracle.add3(a, b, c).tolist() == [1.0, 0.0]        # (a + b) + c, raw/mod.rs:1036


# ------------------------------------------------------------------------------------------- gather, masks, argmax
@pytest.mark.parametrize("ty", [Q4_0, Q8_0, Q4_K, Q6_K])
def test_embed_rows_are_dequantized_rows(oracle, ty):
    n, k = 40, 512
    raw = synth.random_weight(ty, n, k, seed=ty)
    ids = np.array([0, 39, 7, 7, 13], np.uint32)
    table = refgen.np_dequantize(ty, raw).reshape(n, k)
    got = oracle.embed_rows(ty, raw, n, k, ids)
    assert np.array_equal(got.view(np.uint32), table[ids].view(np.uint32))
    with pytest.raises(ValueError):
        oracle.embed_rows(ty, raw, n, k, [40])


def test_causal_mask_is_triu(oracle):
    """fusor/src/cache/attention_mask.rs:46-66 and the zero left padding of mask_cache.rs:73-88."""
    for s, p in ((1, 0), (5, 0), (4, 3), (7, 9)):
        m = oracle.causal_mask(s, p)
        want = np.where(np.triu(np.ones((s, p + s), bool), k=p + 1), -np.inf, 0.0).astype(np.float32)
        assert m.shape == (s, p + s) and np.array_equal(m, want)


def test_argmax_rule(oracle):
    """fusor/src/lib.rs:416-447 with k = 1: ties go to the larger id, non-finite values are skipped."""
    assert oracle.argmax(np.float32([1, 3, 3, 2])) == 2
    assert oracle.argmax(np.float32([np.nan, np.inf, -5, -np.inf])) == 2
    assert oracle.argmax(np.float32([np.nan, np.inf])) == -1
    x = np.random.default_rng(1).standard_normal(5000).astype(np.float32)
    assert oracle.argmax(x) == int(np.argmax(x))


# ------------------------------------------------------------------------------------------- attention
def _qkv(rng, b, h, hkv, sq, skv, d):
    return (rng.standard_normal((b, h, sq, d)).astype(np.float32), rng.standard_normal((b, hkv, skv, d)).astype(np.float32),
            rng.standard_normal((b, hkv, skv, d)).astype(np.float32))


@pytest.mark.parametrize("shape", [(1, 4, 2, 9, 9, 16), (2, 6, 2, 5, 12, 8), (1, 8, 8, 1, 33, 64), (1, 3, 1, 17, 17, 32)])
@pytest.mark.parametrize("mask", ["none", "causal", "additive", "batch-key"])
def test_attention_matches_float64_and_torch(oracle, shape, mask):
    """fusor/src/composite/flash_attention.rs:113-236 against the textbook float64 form (core/tests/attention.rs:25-81
    restated in refgen.np_attention) and torch's scaled_dot_product_attention (a library routine) with the KV heads
    repeated for the groups."""
    import torch
    b, h, hkv, sq, skv, d = shape
    rng = np.random.default_rng(sum(shape))
    q, k, v = _qkv(rng, b, h, hkv, sq, skv, d)
    scale = 1.0 / np.sqrt(d)
    kind, m, m64, tm = 0, None, None, None
    if mask == "causal":
        kind = 1
        i, j = np.arange(sq)[:, None], np.arange(skv)[None, :]
        tm = torch.from_numpy(j <= i + (skv - sq))
    elif mask == "additive":
        kind = 2
        m = np.where(rng.random((sq, skv)) < 0.3, -np.inf, rng.standard_normal((sq, skv))).astype(np.float32)
        m[:, 0] = 0.25                       # no fully masked row
        m64, tm = m.astype(np.float64), torch.from_numpy(m.astype(np.float64))
    elif mask == "batch-key":
        kind = 3
        m = np.where(rng.random((b, skv)) < 0.3, -np.inf, 0.0).astype(np.float32)
        m[:, 0] = 0.0
        tm = torch.from_numpy(m.astype(np.float64))[:, None, None, :]
    got = oracle.flash_attention(q, k, v, scale, kind, m)
    if mask == "batch-key":
        want = np.stack([refgen.np_attention(q[i:i + 1], k[i:i + 1], v[i:i + 1], scale, mask=m[i].astype(np.float64)[None, :])[0]
                         for i in range(b)])
    else:
        want = refgen.np_attention(q, k, v, scale, causal=mask == "causal", mask=m64)
    assert np.abs(got - want).max() < 2e-5
    g = h // hkv
    tq, tk, tv = (torch.from_numpy(t.astype(np.float64)) for t in (q, np.repeat(k, g, 1), np.repeat(v, g, 1)))
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=tm, scale=float(scale)).numpy()
    assert np.abs(got - ref).max() < 2e-5


def test_attention_invariants(oracle):
    rng = np.random.default_rng(5)
    q, k, v = _qkv(rng, 1, 4, 2, 6, 6, 16)
    out = oracle.flash_attention(q, k, v, 0.25, 1)
    assert np.allclose(out[0, :, 0], np.repeat(v[0, :, 0], 2, 0), atol=1e-6)      # causal row 0 sees key 0 only
    ku = np.broadcast_to(k[:, :, :1], k.shape).copy()                              # equal keys -> mean of V
    out = oracle.flash_attention(q, ku, v, 0.25, 0)
    assert np.allclose(out, np.repeat(v.mean(2, keepdims=True), 2, 1).repeat(6, 2), atol=1e-6)
    # grouped heads == the KV heads repeated (flash_attention.rs:139-174): head h reads KV head h // groups
    full = oracle.flash_attention(q, np.repeat(k, 2, 1), np.repeat(v, 2, 1), 0.25, 1)
    assert np.array_equal(full, oracle.flash_attention(q, k, v, 0.25, 1))
    with pytest.raises(ValueError):
        oracle.flash_attention(q[:, :3], k, v, 0.25)                               # 3 heads on 2 KV heads


def test_attention_f16_semantics(oracle):
    """What the reference's f16 CPU instantiation yields (a rounding to f16 after every op, the row sum rounded
    after every add).  On short rows it agrees with the f32 composite on the same f16 inputs to f16 precision; on
    long rows the f16 running sum stalls (spacing 0.25 above 256 swallows addends below 0.125), which is a property
    of that instantiation, not of attention: the f32-accumulating form is the one the device path is held to."""
    rng = np.random.default_rng(2)
    q, k, v = (t.astype(np.float16) for t in _qkv(rng, 1, 4, 2, 24, 24, 32))
    scale = 1.0 / np.sqrt(32)
    h16 = oracle.flash_attention_f16(q, k, v, scale, causal=True).astype(np.float32)
    f32 = oracle.flash_attention(q.astype(np.float32), k.astype(np.float32), v.astype(np.float32), scale, 1)
    assert np.abs(h16 - f32).max() < 6e-3
    # hand-checkable case: one key -> the output is v itself, bit for bit
    one = oracle.flash_attention_f16(q[:, :, :1], k[:, :, :1], v[:, :, :1], scale)
    assert np.array_equal(one.view(np.uint16), np.repeat(v[:, :, :1], 2, 1).view(np.uint16))
    # equal scores: weights 1/n rounded to f16, so the output is n * f16(1/n) * v up to the final rounding
    n = 3
    kk = np.broadcast_to(k[:, :, :1], (1, 2, n, 32)).copy()
    vv = np.broadcast_to(v[:, :, :1], (1, 2, n, 32)).copy()
    out = oracle.flash_attention_f16(q[:, :, :2], kk, vv, scale).astype(np.float32)
    w = np.float32(np.float16(np.float32(1) / np.float32(3)))
    want = ((w * vv[0, :, 0].astype(np.float32)) * 3).astype(np.float16).astype(np.float32)
    assert np.abs(out[0, ::2, 0] - want).max() <= 2e-3 * np.abs(want).max()
    # the stall: 4096 equal keys -> the f16 denominator stops at 2048, every weight doubles
    L = 4096
    kz = np.zeros((1, 1, L, 8), np.float16)
    vz = np.ones((1, 1, L, 8), np.float16)
    out = oracle.flash_attention_f16(np.zeros((1, 1, 1, 8), np.float16), kz, vz, 1.0).astype(np.float32)
    assert out.min() > 1.9            # the exact answer is 1.0


# ------------------------------------------------------------------------------------------- rms_norm
def test_rms_norm_float64(oracle):
    """fusor/src/composite/normalization.rs:404-460; host form conformance common/mod.rs:426-449; weights
    1 + (i % 5) * 0.25 as normalization_ops.rs:45-49."""
    rng = np.random.default_rng(4)
    for rows, cols in ((3, 64), (2, 257), (1, 4096)):
        x = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
        r = rng.standard_normal((rows, cols)).astype(np.float32)
        w = (1 + (np.arange(cols) % 5) * 0.25).astype(np.float32)
        bias = rng.standard_normal(cols).astype(np.float32)
        for res, bb in ((None, None), (r, None), (r, bias)):
            t = x.astype(np.float64) + (0 if res is None else res.astype(np.float64))
            want = t / np.sqrt((t * t).mean(1, keepdims=True) + 1e-5) * w + (0 if bb is None else bb)
            got = oracle.rms_norm(x, w, 1e-5, residual=res, bias=bb)
            assert np.abs(got - want).max() < 5e-6 * max(1, np.abs(want).max())
    # eps matters when the row is tiny; an all-zero row stays zero
    z = oracle.rms_norm(np.zeros((1, 8), np.float32), np.ones(8, np.float32), 1e-5)
    assert np.array_equal(z, np.zeros((1, 8), np.float32))
    tiny = oracle.rms_norm(np.full((1, 8), 1e-3, np.float32), np.ones(8, np.float32), 1e-5)
    assert tiny[0, 0] == pytest.approx(1e-3 / np.sqrt(1e-6 + 1e-5), rel=1e-5)


# ------------------------------------------------------------------------------------------- the decoder
class NumpyLlama:
    """An independent float64 decoder from textbook operations: dequantised weights (refgen.np_dequantize), rms_norm,
    projections, interleaved RoPE as a complex rotation, a growing KV list, causal softmax attention with grouped
    heads, SwiGLU, the residual sums of models/kalosm-llama/src/raw/mod.rs:961-1041."""

    def __init__(self, cfg, weights, types):
        self.c = cfg
        deq = lambda name, n, k: refgen.np_dequantize(types[name], weights[name]).reshape(n, k).astype(np.float64)
        D, H, HK, hd, F, V = (cfg[x] for x in ("d_model", "n_heads", "n_kv_heads", "head_dim", "ffn", "vocab"))
        self.embd = deq("token_embd.weight", V, D)
        self.out = deq("output.weight", V, D)
        self.out_norm = weights["output_norm.weight"].astype(np.float64)
        self.layers = []
        for l in range(cfg["n_layers"]):
            p = f"blk.{l}."
            self.layers.append(dict(
                wq=deq(p + "attn_q.weight", H * hd, D), wk=deq(p + "attn_k.weight", HK * hd, D),
                wv=deq(p + "attn_v.weight", HK * hd, D), wo=deq(p + "attn_output.weight", D, H * hd),
                gate=deq(p + "ffn_gate.weight", F, D), up=deq(p + "ffn_up.weight", F, D), down=deq(p + "ffn_down.weight", D, F),
                an=weights[p + "attn_norm.weight"].astype(np.float64), fn=weights[p + "ffn_norm.weight"].astype(np.float64),
                k=np.zeros((HK, 0, hd)), v=np.zeros((HK, 0, hd))))
        inv = 1.0 / cfg["theta"] ** (np.arange(0, hd, 2) / hd)
        self.rot = np.exp(1j * np.outer(np.arange(cfg["ctx"]), inv))
        self.pos = 0

    def _norm(self, x, w):
        return x / np.sqrt((x * x).mean(-1, keepdims=True) + self.c["eps"]) * w

    def _rope(self, x, pos):  # x [heads, s, hd]
        z = (x[..., 0::2] + 1j * x[..., 1::2]) * self.rot[pos:pos + x.shape[1]][None]
        y = np.empty_like(x)
        y[..., 0::2], y[..., 1::2] = z.real, z.imag
        return y

    def forward(self, tokens):
        c = self.c
        H, HK, hd = c["n_heads"], c["n_kv_heads"], c["head_dim"]
        s = len(tokens)
        x = self.embd[np.asarray(tokens)]
        for L in self.layers:
            xn = self._norm(x, L["an"])
            q = (xn @ L["wq"].T).reshape(s, H, hd).transpose(1, 0, 2)
            k = (xn @ L["wk"].T).reshape(s, HK, hd).transpose(1, 0, 2)
            v = (xn @ L["wv"].T).reshape(s, HK, hd).transpose(1, 0, 2)
            q, k = self._rope(q, self.pos), self._rope(k, self.pos)
            L["k"], L["v"] = np.concatenate([L["k"], k], 1), np.concatenate([L["v"], v], 1)
            att = refgen.np_attention(q[None], L["k"][None], L["v"][None], 1.0 / np.sqrt(hd), causal=s > 1)[0]
            a = att.transpose(1, 0, 2).reshape(s, H * hd) @ L["wo"].T
            h = self._norm(a + x, L["fn"])
            g = h @ L["gate"].T
            with np.errstate(over="ignore"):
                ff = ((g / (1 + np.exp(-g))) * (h @ L["up"].T)) @ L["down"].T
            x = ff + a + x
        self.pos += s
        hid = self._norm(x[-1], self.out_norm)
        return hid @ self.out.T, hid


@pytest.mark.parametrize("heads,kv_heads", [(4, 2), (12, 4), (4, 4)], ids=["g2", "g3", "g1"])
def test_decoder_matches_independent_float64_decoder(oracle, heads, kv_heads):
    cfg = dict(n_layers=2, d_model=256, n_heads=heads, n_kv_heads=kv_heads, head_dim=64, ffn=512, vocab=300, ctx=32, eps=1e-5,
               theta=10000.0)
    specs = synth.llama_tensor_specs(cfg)
    weights = {name: synth.llama_random_tensor(name, ty, n, k, 11, 0.02) for name, ty, n, k in specs}
    types = {name: ty for name, ty, _, _ in specs}
    ref = oracle.Llama(dict(cfg, type_attn=Q4_K, type_ffn_gate_up=Q4_K, type_ffn_down=Q6_K, type_embd=Q4_K, type_output=Q6_K),
                       weights)
    mine = NumpyLlama(cfg, weights, types)
    rng = np.random.default_rng(6)
    scale = None
    for tokens in (rng.integers(0, 300, 7), [5], [299], rng.integers(0, 300, 3), [0]):   # prefill, steps, a second chunk
        lg, hid = ref.forward(tokens, want_hidden=True)
        wl, wh = mine.forward(list(tokens))
        scale = max(np.abs(wl).max(), 1.0)
        assert np.abs(hid - wh).max() < 2e-4 * max(np.abs(wh).max(), 1.0)
        assert np.abs(lg - wl).max() < 2e-4 * scale
        assert oracle.argmax(lg) == int(np.argmax(wl)) or np.sort(wl)[-1] - np.sort(wl)[-2] < 1e-3 * scale
    assert np.abs(wl).max() > 1e-2          # the logits are not degenerate
    # the cache matters: the same token from an empty cache gives other logits
    ref.reset()
    assert np.abs(ref.forward([0]) - lg).max() > 1e-3 * scale
