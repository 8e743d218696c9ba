"""GPU parity of the row / pointwise operators, attention and the KV cache against the CPU checker."""
import numpy as np
import pytest

import refgen
from refgen import assert_close
from kalosm_amd.fusor import Device, FusorHipError, KvCache, MaskKind, RopeCache, Tensor

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


# ----------------------------------------------------------------------------- rms_norm
@pytest.mark.parametrize("shape", [(1, 4096), (3, 17, 257), (2, 16, 255), (5, 64)])
@pytest.mark.parametrize("residual", [False, True])
def test_rms_norm(dev, oracle, shape, residual):
    """conformance normalization_ops.rs:45-80: weights 1 + (i % 5) * 0.25, eps 1e-5, tol 1e-4; fuzz shapes
    [2..3, 16..17, 255..257]."""
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal(shape).astype(np.float32)
    r = rng.standard_normal(shape).astype(np.float32) if residual else None
    w = (1 + (np.arange(shape[-1]) % 5) * 0.25).astype(np.float32)
    xt, wt = Tensor.from_slice(dev, x), Tensor.from_slice(dev, w)
    got = (xt.rms_norm_residual_fused(Tensor.from_slice(dev, r), wt, None, 1e-5) if residual
           else xt.rms_norm_fused(wt, None, 1e-5)).as_slice()
    want = oracle.rms_norm(x, w, 1e-5, residual=r)
    assert_close(got, want, abs_tol=1e-4, rel_tol=1e-4, what="rms_norm")
    # the formula of the reference's host check (conformance common/mod.rs:426-449) in float64
    t = (x + r if residual else x).astype(np.float64)
    ref = t / np.sqrt((t * t).mean(-1, keepdims=True) + 1e-5) * w
    assert_close(got, ref, abs_tol=1e-4, rel_tol=1e-4, what="rms_norm vs float64 formula")


def test_rms_norm_bias(dev, oracle):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((4, 300)).astype(np.float32)
    w = rng.standard_normal(300).astype(np.float32)
    b = rng.standard_normal(300).astype(np.float32)
    got = Tensor.from_slice(dev, x).rms_norm_fused(Tensor.from_slice(dev, w), Tensor.from_slice(dev, b), 1e-6).as_slice()
    assert_close(got, oracle.rms_norm(x, w, 1e-6, bias=b), abs_tol=1e-4, rel_tol=1e-4, what="rms_norm + bias")


# ----------------------------------------------------------------------------- rope
def test_rope_tables_golden(dev, oracle):
    """models/kalosm-llama/src/raw/rope.rs:295-310: head_dim 2, theta 5000, 6 positions."""
    rc = RopeCache.new(2, 6, 5000.0, dev)
    cos, sin = rc.cos.as_slice().reshape(-1), rc.sin.as_slice().reshape(-1)
    assert np.abs(cos - np.float32([1.0000, 0.5403, -0.4161, -0.9900, -0.6536, 0.2837])).max() < 1e-4
    assert np.abs(sin - np.float32([0.0000, 0.8415, 0.9093, 0.1411, -0.7568, -0.9589])).max() < 1e-4
    oc, os_ = oracle.rope_tables(128, 512, 500000.0)
    rc = RopeCache.new(128, 512, 500000.0, dev)
    assert np.array_equal(bits(rc.cos.as_slice()), bits(oc)) and np.array_equal(bits(rc.sin.as_slice()), bits(os_))


def test_rope_tables_scaled(dev, oracle):
    """Long-context scaling and rope_freqs.weight factors (models/kalosm-llama/src/raw/rope.rs:9-50)."""
    w = np.linspace(1.0, 0.5, 64).astype(np.float32)
    for scaling, fw in [((8.0, 4.0, 1.0, 8192), None), (None, w), ((8.0, 4.0, 1.0, 8192), w), ((32.0, 4.0, 1.0, 8192), None)]:
        rc = RopeCache.scaled(128, 300, 500000.0, dev, scaling=scaling, freq_weight=fw)
        oc, os_ = oracle.rope_tables_scaled(128, 300, 500000.0, scaling, fw)
        assert np.array_equal(bits(rc.cos.as_slice()), bits(oc)) and np.array_equal(bits(rc.sin.as_slice()), bits(os_))
    plain = RopeCache.new(128, 300, 500000.0, dev).cos.as_slice()
    assert not np.array_equal(plain, oc)


@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("start_pos", [0, 5])
def test_rope_pair(dev, oracle, interleaved, start_pos):
    """conformance rope_ops.rs: both pairings, a start position, and q arriving as the transposed view
    [b, s, h, d] -> [b, h, s, d] (attention_layer.rs:371-374)."""
    b, hq, hk, s, d = 2, 8, 2, 7, 64
    rng = np.random.default_rng(start_pos + 10 * interleaved)
    q_bshd = rng.standard_normal((b, s, hq, d)).astype(np.float32)
    k_bshd = rng.standard_normal((b, s, hk, d)).astype(np.float32)
    cos, sin = oracle.rope_tables(d, 32, 10000.0)
    rc = RopeCache.from_parts(Tensor.from_slice(dev, cos), Tensor.from_slice(dev, sin))
    qt = Tensor.from_slice(dev, q_bshd).reshape((b, hq, s, d))   # logical shape; physical layout is [b, s, h, d]
    kt = Tensor.from_slice(dev, k_bshd).reshape((b, hk, s, d))
    fn = rc.forward_interleaved if interleaved else rc.forward
    qo, ko = fn(qt, kt, start_pos, q_strides=(s * hq * d, d, hq * d), k_strides=(s * hk * d, d, hk * d))
    wq = oracle.rope(q_bshd.transpose(0, 2, 1, 3), cos, sin, start_pos, interleaved)
    wk = oracle.rope(k_bshd.transpose(0, 2, 1, 3), cos, sin, start_pos, interleaved)
    assert np.array_equal(bits(qo.as_slice()), bits(wq)) and np.array_equal(bits(ko.as_slice()), bits(wk))
    with pytest.raises(FusorHipError):
        fn(qt, kt, 30)  # positions beyond the table


# ----------------------------------------------------------------------------- pointwise
def test_swiglu_add_argmax_casts(dev, oracle):
    rng = np.random.default_rng(5)
    g = (rng.standard_normal(5000) * 4).astype(np.float32)
    u = rng.standard_normal(5000).astype(np.float32)
    got = Tensor.from_slice(dev, g).silu_mul(Tensor.from_slice(dev, u)).as_slice()
    assert_close(got, oracle.swiglu(g, u), abs_tol=1e-6, rel_tol=1e-6, what="silu*up")
    a, b, c = (rng.standard_normal(777).astype(np.float32) for _ in range(3))
    got = Tensor.from_slice(dev, a).add(Tensor.from_slice(dev, b), Tensor.from_slice(dev, c)).as_slice()
    assert np.array_equal(bits(got), bits(oracle.add3(a, b, c)))
    x = rng.standard_normal((6, 5, 8)).astype(np.float32)
    assert np.array_equal(Tensor.from_slice(dev, x).transpose_shd().as_slice(), x.transpose(1, 0, 2))
    h = Tensor.from_slice(dev, g).cast("f16").as_slice()
    assert np.array_equal(h.view(np.uint16), g.astype(np.float16).view(np.uint16))
    from kalosm_amd import synth
    bf = Tensor.from_slice(dev, g).cast("bf16").as_slice()
    assert np.array_equal(bf, synth.to_bf16_bits(g))
    # greedy pick: ties go to the larger id, non-finite values are skipped (fusor/src/lib.rs:416-447)
    v = rng.standard_normal(128256).astype(np.float32)
    assert Tensor.from_slice(dev, v).top_k_pairs_1() == oracle.argmax(v) == int(np.argmax(v))
    v[[7, 70000, 128255]] = v.max() + 1
    assert Tensor.from_slice(dev, v).top_k_pairs_1() == oracle.argmax(v) == 128255
    v[128255] = np.inf
    v[3] = np.nan
    assert Tensor.from_slice(dev, v).top_k_pairs_1() == oracle.argmax(v) == 70000
    assert Tensor.from_slice(dev, np.full(100, np.nan, np.float32)).top_k_pairs_1() == oracle.argmax(np.full(100, np.nan)) == -1


# ----------------------------------------------------------------------------- attention
def run_attn(dev, q, k, v, scale, mask=None, dtype="f32"):
    cast = (lambda a: a.astype(np.float16)) if dtype == "f16" else (lambda a: a)
    qt, kt, vt = (Tensor.from_slice(dev, cast(a), dtype) for a in (q, k, v))
    return qt.flash_attention(kt, vt, scale, mask).as_slice().astype(np.float32)


@pytest.mark.parametrize("L", [129, 192, 256, 257, 384, 511, 512, 569, 1025])
def test_attention_decode_tile_boundaries(dev, oracle, L):
    """conformance flash_attention_ops.rs:310-343: H=16, H_kv=2, d=128, one query, KV lengths around the tile
    sizes, each run 4 times (races show as run-to-run differences)."""
    h, hkv, d = 16, 2, 128
    q = refgen.attn_pattern(h * d, 0.1).reshape(1, h, 1, d)
    k = refgen.attn_pattern(hkv * L * d, -0.15).reshape(1, hkv, L, d)
    v = refgen.attn_pattern(hkv * L * d, 0.35).reshape(1, hkv, L, d)
    want = oracle.flash_attention(q, k, v, 1 / np.sqrt(d))
    first = None
    for _ in range(4):
        got = run_attn(dev, q, k, v, 1 / np.sqrt(d))
        assert_close(got, want, abs_tol=1e-4, rel_tol=1e-4, what=f"decode L={L}")
        first = got if first is None else first
        assert np.array_equal(got, first)


@pytest.mark.parametrize("sq,skv,d", [(64, 64, 8), (72, 80, 16), (65, 35, 8), (128, 128, 24), (96, 100, 64), (5, 3000, 128)])
@pytest.mark.parametrize("kind", ["none", "causal", "additive"])
def test_attention_prefill_shapes(dev, oracle, sq, skv, d, kind):
    """core/tests/attention.rs:152-325 and flash_attention_ops.rs:761-828: sin inputs, GQA, causal (with a
    KV longer or shorter than the queries), additive mask i % 7 == 0 ? -1.5 : 0.25, long-KV streaming."""
    if kind == "causal" and skv < sq:
        pytest.skip("a causal mask with fewer keys than queries leaves fully masked rows (NaN in the reference too)")
    h, hkv = 4, 2
    q = refgen.attn_sin(h * sq * d, 0.13).reshape(1, h, sq, d)
    k = refgen.attn_sin(hkv * skv * d, 0.07).reshape(1, hkv, skv, d)
    v = refgen.attn_sin(hkv * skv * d, 0.11).reshape(1, hkv, skv, d)
    scale = 1 / np.sqrt(d)
    mask_np, mask, okind = None, None, oracle.MASK_NONE
    if kind == "causal":
        mask, okind = MaskKind.Causal, oracle.MASK_CAUSAL
    elif kind == "additive":
        mask_np = np.where(np.arange(sq * skv) % 7 == 0, -1.5, 0.25).astype(np.float32).reshape(sq, skv)
        mask, okind = (Tensor.from_slice(dev, mask_np), MaskKind.QKMask), oracle.MASK_ADDITIVE
    got = run_attn(dev, q, k, v, scale, mask)
    want = oracle.flash_attention(q, k, v, scale, okind, mask_np)
    assert_close(got, want, abs_tol=1e-4, rel_tol=1e-4, what=f"attention {kind} {sq}x{skv}x{d}")
    ref = refgen.np_attention(q, k, v, scale, causal=(kind == "causal"), mask=mask_np)
    assert_close(got, ref, abs_tol=1e-4, rel_tol=1e-4, what="attention vs float64 textbook")


def test_attention_invariants(dev, oracle):
    """rows of P sum to 1 (V = const -> out = const), causal row 0 -> out = v_0, uniform K -> mean(V),
    GQA == repeated KV heads, all-zero additive mask == no mask (flash_attention_ops.rs:640-647)."""
    rng = np.random.default_rng(8)
    h, hkv, s, d = 32, 8, 10, 128
    q = rng.standard_normal((1, h, s, d)).astype(np.float32)
    k = rng.standard_normal((1, hkv, s, d)).astype(np.float32)
    v = rng.standard_normal((1, hkv, s, d)).astype(np.float32)
    sc = 1 / np.sqrt(d)
    out = run_attn(dev, q, k, np.full_like(v, 0.75), sc)
    assert np.abs(out - 0.75).max() < 1e-5
    out = run_attn(dev, q, k, v, sc, MaskKind.Causal)
    assert np.abs(out[0, :, 0, :] - np.repeat(v[0, :, 0, :], h // hkv, axis=0)).max() < 1e-6
    out = run_attn(dev, q, np.ones_like(k), v, sc)
    assert np.abs(out - np.repeat(v.mean(2, keepdims=True), h // hkv, axis=1)).max() < 1e-5
    rep = run_attn(dev, q, np.repeat(k, h // hkv, axis=1), np.repeat(v, h // hkv, axis=1), sc)
    assert_close(run_attn(dev, q, k, v, sc), rep, abs_tol=1e-6, rel_tol=1e-6, what="GQA vs repeated heads")
    zero = Tensor.zeros(dev, (s, s))
    assert_close(run_attn(dev, q, k, v, sc, (zero, MaskKind.QKMask)), run_attn(dev, q, k, v, sc), abs_tol=1e-6,
                 rel_tol=1e-6, what="zero mask")
    with pytest.raises(FusorHipError, match="divisible"):
        Tensor.from_slice(dev, q[:, :30]).flash_attention(Tensor.from_slice(dev, k), Tensor.from_slice(dev, v), sc)


@pytest.mark.parametrize("L", [200, 1024, 4096])
def test_attention_f16_decode(dev, oracle, L):
    """Benchmark configuration 3 (decode): f16 Q/K/V ~ N(0,1), 32 / 8 heads, d = 128.  The checker works in f32 on
    the f16-rounded inputs; the GPU result is rounded to f16 on output (tolerance 1e-2 as the reference's f16 cases)."""
    rng = np.random.default_rng(L)
    h, hkv, d = 32, 8, 128
    q, k, v = (rng.standard_normal(s).astype(np.float16).astype(np.float32) for s in ((1, h, 1, d), (1, hkv, L, d), (1, hkv, L, d)))
    got = run_attn(dev, q, k, v, 1 / np.sqrt(d), dtype="f16")
    want = oracle.flash_attention(q, k, v, 1 / np.sqrt(d))
    assert_close(got, want, abs_tol=1e-2, rel_tol=1e-3, what=f"f16 decode L={L}")


def test_attention_transposed_q(dev, oracle):
    """flash_attention_ops.rs:354-419: q given as a [b, s, h, d] buffer viewed as [b, h, s, d]."""
    rng = np.random.default_rng(9)
    b, h, hkv, s, d = 1, 8, 2, 6, 64
    q_bshd = rng.standard_normal((b, s, h, d)).astype(np.float32)
    k = rng.standard_normal((b, hkv, 40, d)).astype(np.float32)
    v = rng.standard_normal((b, hkv, 40, d)).astype(np.float32)
    qt = Tensor.from_slice(dev, q_bshd).reshape((b, h, s, d))
    got = qt.flash_attention(Tensor.from_slice(dev, k), Tensor.from_slice(dev, v), 0.125, MaskKind.Causal,
                             q_strides=(s * h * d, d, h * d)).as_slice()
    want = oracle.flash_attention(q_bshd.transpose(0, 2, 1, 3), k, v, 0.125, oracle.MASK_CAUSAL)
    assert_close(got, want, abs_tol=1e-4, rel_tol=1e-4, what="transposed q")


# ----------------------------------------------------------------------------- KV cache
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_kv_cache_growth_append_reset(dev, dtype):
    """conformance cache_ops.rs:83-268 and tensor_cache.rs:315-338: capacity 256 -> 512 ..., contents preserved
    across growth, reset, max_len cap and overflow."""
    layers, hk, d = 2, 2, 64
    c = KvCache(dev, layers, hk, d, max_len=600, dtype=dtype)
    rng = np.random.default_rng(11)
    hist = [[np.zeros((hk, 0, d), np.float32) for _ in range(2)] for _ in range(layers)]
    expected_caps = []
    for s in (1, 64, 191, 1, 300):
        for l in range(layers):
            k = rng.standard_normal((hk, s, d)).astype(np.float32)
            v = rng.standard_normal((hk, s, d)).astype(np.float32)
            c.append(l, Tensor.from_slice(dev, k), Tensor.from_slice(dev, v))
            hist[l][0] = np.concatenate([hist[l][0], k], 1)
            hist[l][1] = np.concatenate([hist[l][1], v], 1)
        ln, cap, kt, vt = c.view(0)
        expected_caps.append(cap)
        for l in range(layers):
            ln, cap, kt, vt = c.view(l)
            assert ln == hist[l][0].shape[1]
            want_k = hist[l][0].astype(np.float16).astype(np.float32) if dtype == "f16" else hist[l][0]
            assert np.array_equal(kt.as_slice()[:, :ln].astype(np.float32), want_k)
            want_v = hist[l][1].astype(np.float16).astype(np.float32) if dtype == "f16" else hist[l][1]
            assert np.array_equal(vt.as_slice()[:, :ln].astype(np.float32), want_v)
    assert expected_caps == [256, 256, 256, 512, 600]  # gpu_allocation_seq_len: pow2, min 256, capped at max_len
    with pytest.raises(FusorHipError, match="overflow"):
        c.append(0, Tensor.zeros(dev, (hk, 100, d)), Tensor.zeros(dev, (hk, 100, d)))
    c.reset()
    assert c.view(0)[0] == 0


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_kv_cache_sliding_window(dev, dtype):
    """TensorCache sliding window (tensor_cache.rs:175-202): past max_len the cache is the last max_len positions of
    [cached | new], also when one append is longer than the window."""
    layers, hk, d, window = 2, 2, 64, 300
    c = KvCache(dev, layers, hk, d, max_len=window, dtype=dtype, sliding_window=True)
    rng = np.random.default_rng(12)
    hist = [[np.zeros((hk, 0, d), np.float32) for _ in range(2)] for _ in range(layers)]
    for s in (200, 99, 1, 1, 7, 150, 299, 300, 1, 450, 3):
        for l in range(layers):
            k = rng.standard_normal((hk, s, d)).astype(np.float32)
            v = rng.standard_normal((hk, s, d)).astype(np.float32)
            c.append(l, Tensor.from_slice(dev, k), Tensor.from_slice(dev, v))
            hist[l][0] = np.concatenate([hist[l][0], k], 1)[:, -window:]
            hist[l][1] = np.concatenate([hist[l][1], v], 1)[:, -window:]
        for l in range(layers):
            ln, cap, kt, vt = c.view(l)
            assert ln == hist[l][0].shape[1] <= window
            for got, want in ((kt, hist[l][0]), (vt, hist[l][1])):
                want = want.astype(np.float16).astype(np.float32) if dtype == "f16" else want
                assert np.array_equal(got.as_slice()[:, :ln].astype(np.float32), want), (s, l)


# ----------------------------------------------------------------------------- prefill attention on the matrix cores
@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("sq,skv,causal", [(128, 128, True), (200, 200, True), (64, 300, True), (160, 97, False),
                                           (512, 512, True), (33, 33, True)])
def test_attention_prefill_f16(dev, oracle, sq, skv, causal, d):
    """f16 Q/K/V, 8 query heads on 2 KV heads, query blocks and key tiles with ragged ends, causal with the queries
    aligned to the end of a longer KV.  The checker gets the f32 values of the same f16 inputs; the output is f16
    (2^-11 relative) and P is rounded to f16 before the second product: 1e-3 relative or 1e-2 absolute."""
    h, hkv = 8, 2
    rng = np.random.default_rng(sq * 1000 + skv + d)
    q = rng.standard_normal((1, h, sq, d)).astype(np.float16)
    k = rng.standard_normal((1, hkv, skv, d)).astype(np.float16)
    v = rng.standard_normal((1, hkv, skv, d)).astype(np.float16)
    scale = 1 / np.sqrt(d)
    got = run_attn(dev, q, k, v, scale, MaskKind.Causal if causal else None, dtype="f16")
    qf, kf, vf = (a.astype(np.float32) for a in (q, k, v))
    want = oracle.flash_attention(qf, kf, vf, scale, oracle.MASK_CAUSAL if causal else oracle.MASK_NONE, None)
    assert_close(got, want, abs_tol=1e-2, rel_tol=1e-3, what=f"f16 prefill {sq}x{skv}x{d}")
    ref = refgen.np_attention(qf, kf, vf, scale, causal=causal, mask=None)
    assert_close(got, ref, abs_tol=1e-2, rel_tol=1e-3, what="vs float64 textbook")


@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("sq,skv,causal", [(128, 128, True), (200, 200, True), (64, 300, True), (160, 97, False),
                                           (512, 512, True), (33, 33, True)])
def test_attention_prefill_f32_split(dev, oracle, sq, skv, causal, d):
    """All-f32 Q/K/V take the matrix-core kernel with split operands (every value as the exact two-term f16 split,
    three MFMAs per product): f32 accuracy, so the tolerance is a tenth of the north star's; inputs of magnitude up
    to ~10 (scores up to a few tens) and the same ragged shapes as the f16 test; compared with the checker and with
    the exact row kernel."""
    h, hkv = 8, 2
    rng = np.random.default_rng(sq * 1000 + skv + d + 7)
    q = (rng.standard_normal((1, h, sq, d)) * 2.5).astype(np.float32)
    k = (rng.standard_normal((1, hkv, skv, d)) * 2.5).astype(np.float32)
    v = (rng.standard_normal((1, hkv, skv, d)) * 3.0).astype(np.float32)
    scale = 1 / np.sqrt(d)
    mask = MaskKind.Causal if causal else None
    got = run_attn(dev, q, k, v, scale, mask)
    want = oracle.flash_attention(q, k, v, scale, oracle.MASK_CAUSAL if causal else oracle.MASK_NONE, None)
    assert_close(got, want, abs_tol=1e-3, rel_tol=1e-4, what=f"f32 split prefill {sq}x{skv}x{d}")
    dev.set_option("attn_kernel", 1)
    try:
        rows = run_attn(dev, q, k, v, scale, mask)
    finally:
        dev.set_option("attn_kernel", 0)
    assert_close(got, rows, abs_tol=1e-3, rel_tol=1e-4, what="vs the exact row kernel")


@pytest.mark.parametrize("force", [6, 7, 8, 9])
@pytest.mark.parametrize("sq,skv,causal,d", [(300, 300, True, 128), (129, 700, True, 128), (257, 190, False, 128),
                                             (64, 65, True, 64), (384, 384, True, 64), (33, 200, True, 128)])
def test_attention_prefill_workgroup_shapes(dev, oracle, force, sq, skv, causal, d):
    """The four workgroup shapes of the matrix-core kernel on the same ragged inputs, whatever the dispatch would
    pick for the size (attn_kernel = 6: two heads of a KV group share the staged tiles; 7: the key tiles of a query
    block shared out over two groups of wavefronts and merged; 8: four wavefronts, one head; 9: query blocks of 64 rows,
    two key groups of two wavefronts): f16 and f32 queries on an
    f16 cache, causal with the queries at the end of a longer cache, odd tile counts (a group without a tile in the last
    step), a single query block."""
    h, hkv = 8, 2
    rng = np.random.default_rng(sq * 31 + skv * 7 + d + force)
    scale = 1 / np.sqrt(d)
    q = rng.standard_normal((1, h, sq, d)).astype(np.float16)
    k = rng.standard_normal((1, hkv, skv, d)).astype(np.float16)
    v = rng.standard_normal((1, hkv, skv, d)).astype(np.float16)
    qf, kf, vf = (a.astype(np.float32) for a in (q, k, v))
    want = oracle.flash_attention(qf, kf, vf, scale, oracle.MASK_CAUSAL if causal else oracle.MASK_NONE, None)
    dev.set_option("attn_kernel", force)
    try:
        got = run_attn(dev, q, k, v, scale, MaskKind.Causal if causal else None, dtype="f16")
    finally:
        dev.set_option("attn_kernel", 0)
    assert_close(got, want, abs_tol=1e-2, rel_tol=1e-3, what=f"f16 prefill shape {force}: {sq}x{skv}x{d}")


def test_attention_prefill_f32_on_request(dev, oracle):
    """f32 operands through the same kernel (rounded to f16 inside, f32 out), and the invariants that do not depend
    on the rounding: V constant -> output constant, causal row 0 -> v_0."""
    h, hkv, sq, d = 4, 1, 96, 128
    rng = np.random.default_rng(5)
    q, k, v = (rng.standard_normal((1, n, sq, d)).astype(np.float32) for n in (h, hkv, hkv))
    dev.set_option("attn_kernel", 2)
    try:
        got = run_attn(dev, q, k, v, 1 / np.sqrt(d), MaskKind.Causal)
        want = oracle.flash_attention(q, k, v, 1 / np.sqrt(d), oracle.MASK_CAUSAL, None)
        assert_close(got, want, abs_tol=1e-2, rel_tol=1e-3, what="f32 prefill on the matrix cores")
        assert_close(got[0, :, 0], np.broadcast_to(v[0, 0, 0], (h, d)), abs_tol=1e-3, rel_tol=1e-3, what="row 0 sees v_0 only")
        vc = np.full_like(v, 0.75)
        got = run_attn(dev, q, k, vc, 1 / np.sqrt(d), None)
        assert_close(got, np.full_like(got, 0.75), abs_tol=1e-3, rel_tol=1e-3, what="constant V")
    finally:
        dev.set_option("attn_kernel", 0)


@pytest.mark.parametrize("n", [5, 1000, 1024, 1025, 128256])
def test_top_k_pairs(dev, oracle, n):
    """Tensor::top_k_pairs(k) (fusor/src/lib.rs:416-447) at vocabulary size and at the pass boundaries: bit-equal
    pairs in the reference's order (descending logit, ties to the larger id, non-finite skipped)."""
    rng = np.random.default_rng(n)
    for variant in range(3):
        if variant == 0:
            x = rng.standard_normal(n).astype(np.float32)
        elif variant == 1:
            x = rng.integers(-3, 4, n).astype(np.float32)      # almost everything ties
            x[rng.integers(0, n, max(1, n // 50))] = np.nan
            x[rng.integers(0, n, 2)] = [np.inf, -np.inf]
            x[rng.integers(0, n, 2)] = [0.0, -0.0]
        else:
            x = np.full(n, np.nan, np.float32)                 # fewer finite values than k
            x[rng.integers(0, n, 3)] = [1.5, -2.0, 1.5]
        t = Tensor.from_slice(dev, x)
        for k in (1, 5, 64, 256):
            got = t.top_k_pairs(k)
            want = oracle.top_k(x, k)
            assert [g[0] for g in got] == [w[0] for w in want], (n, variant, k)
            assert np.array_equal(np.float32([g[1] for g in got]).view(np.uint32), np.float32([w[1] for w in want]).view(np.uint32))
    assert t.top_k_pairs(0) == []
    with pytest.raises(Exception):
        t.top_k_pairs(257)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_attention_batch_key_mask(dev, oracle, dtype):
    """MaskKind::BatchKeyMask (flash_attention.rs:12-24, :199-213): an additive [batch, kv_len] mask for every head
    and query of a batch entry (padding masks); masked keys of entry 1 must not influence its output."""
    b, h, hkv, sq, skv, d = 3, 4, 2, 37, 50, 64
    rng = np.random.default_rng(21)
    npdt = np.float16 if dtype == "f16" else np.float32
    q = rng.standard_normal((b, h, sq, d)).astype(npdt)
    k = rng.standard_normal((b, hkv, skv, d)).astype(npdt)
    v = rng.standard_normal((b, hkv, skv, d)).astype(npdt)
    mask = np.zeros((b, skv), np.float32)
    mask[1, 30:] = -np.inf
    mask[2, ::3] = -0.75
    got = Tensor.from_slice(dev, q, dtype).flash_attention(Tensor.from_slice(dev, k, dtype), Tensor.from_slice(dev, v, dtype),
                                                           0.125, (Tensor.from_slice(dev, mask), MaskKind.BatchKeyMask)).as_slice()
    want = oracle.flash_attention(q.astype(np.float32), k.astype(np.float32), v.astype(np.float32), 0.125, 3, mask)
    tol = dict(abs_tol=2e-3, rel_tol=2e-3) if dtype == "f16" else dict(abs_tol=1e-4, rel_tol=1e-4)
    assert_close(got.astype(np.float32), want, what="BatchKeyMask", **tol)
    k2 = k.copy(); k2[1, :, 30:] = 9.0
    got2 = Tensor.from_slice(dev, q, dtype).flash_attention(Tensor.from_slice(dev, k2, dtype), Tensor.from_slice(dev, v, dtype),
                                                            0.125, (Tensor.from_slice(dev, mask), MaskKind.BatchKeyMask)).as_slice()
    assert np.array_equal(got[1], got2[1])


def test_sample_token_reference_answers(dev):
    """The answers the reference's sampler tests store (fusor-ml/core/src/sampling/tests.rs:192-318,
    models/kalosm-llama/src/sampler.rs:384-441), through the library."""
    from kalosm_amd.fusor import GpuMirostat2Sampler, GpuMirostat2SamplerParams, GpuStandardSamplerParams
    flat = Tensor.from_slice(dev, np.ones(4, np.float32))
    s = GpuMirostat2Sampler(dev, 10.0)
    tok, ids, vals = flat.sample_mirostat2_token(s, [], GpuMirostat2SamplerParams(4, 1.0, 1.0, 5.0, 0.1, 0.8), want_candidates=True)
    assert tok == 0 and ids.tolist() == [3, 2, 1, 0] and vals.tolist() == [1.0] * 4
    assert s.mu == pytest.approx(10.0 - 0.1 * (2.0 - 5.0), rel=1e-6)      # four equal candidates: surprise 2 bits
    assert flat.sample_standard_token([], GpuStandardSamplerParams(4, 1.0, 1.0, 0.5, 0.0, 0.8)) == 2
    t = Tensor.from_slice(dev, np.array([9.0, 8.5, 7.0, 6.0, 2.5, 0.25, -1.0, -3.0], np.float32))
    assert t.sample_mirostat2_token(GpuMirostat2Sampler(dev, 10.0), [], GpuMirostat2SamplerParams(4, 1.0, 1.0, 5.0, 0.1, 0.0)) == 0
    t = Tensor.from_slice(dev, np.array([-5.0, -4.0, -3.0, 0.0], np.float32))
    for rnd in (0.0, 0.5, 0.999):
        assert t.sample_standard_token([], GpuStandardSamplerParams(4, 1.0, 1.0, 1.0, 0.1, rnd)) == 3
    t = Tensor.from_slice(dev, np.array([9.0, 7.5, 7.0, 4.0, 3.5, 1.0], np.float32))
    assert t.sample_mirostat2_token(GpuMirostat2Sampler(dev, 3.0), [], GpuMirostat2SamplerParams(5, 1.0, 1.0, 5.0, 0.1, 0.65)) == 0
    # processors: temperature 0.5, penalty 2, previous {0, 3, 9} (tests.rs:61-136)
    values = np.array([4.0, -2.0, 3.5, 8.0, np.nan, 1.0, 5.0, -1.5, 6.5, 7.0, -np.inf, 0.5], np.float32)
    _, ids, vals = Tensor.from_slice(dev, values).sample_standard_token(
        [0, 3, 9], GpuStandardSamplerParams(5, 0.5, 2.0, 1.0, 0.0, 0.0), want_candidates=True)
    assert ids.tolist() == [8, 6, 3, 9, 2] and vals.tolist() == [13.0, 10.0, 8.0, 7.0, 7.0]
    none = Tensor.from_slice(dev, np.array([np.nan, np.inf, -np.inf], np.float32))
    assert none.sample_standard_token([], GpuStandardSamplerParams(2, 1.0, 1.0, 1.0, 0.0, 0.5)) is None
    with pytest.raises(Exception):
        flat.sample_standard_token([], GpuStandardSamplerParams(257, 1.0, 1.0, 1.0, 0.0, 0.5))
    with pytest.raises(Exception):
        flat.sample_standard_token([], GpuStandardSamplerParams(0, 1.0, 1.0, 1.0, 0.0, 0.5))


@pytest.mark.parametrize("n", [12, 1000, 5000, 128256])
def test_sample_token_matches_checker(dev, oracle, n):
    """Both device samplers against the checker on random logits: the processed top-k candidates are bit-equal; the
    sampled id is equal wherever the checker's deciding comparisons have a relative gap above 1e-4 (exp and log2
    come from different libraries on the two sides); the Mirostat state follows to 1e-5.  Values are compared as
    numbers: the candidates' values are rebuilt from the sort keys, which hold -0.0 as 0.0."""
    from kalosm_amd.fusor import GpuMirostat2Sampler, GpuMirostat2SamplerParams, GpuStandardSamplerParams
    rng = np.random.default_rng(n)
    compared = 0
    for case in range(40):
        x = (rng.standard_normal(n) * rng.choice([0.5, 2.0, 6.0])).astype(np.float32)
        if case % 5 == 0:
            x[rng.integers(0, n, max(1, n // 20))] = [np.nan, np.inf, -np.inf][case % 3]
        if case % 7 == 0:
            x = np.round(x)                                            # ties
        k = int(rng.choice([1, 2, 7, 40, 64, 256]))
        temp = float(rng.choice([0.0, 0.7, 1.0, 1.3]))
        pen = float(rng.choice([1.0, 1.1, 1.5, 0.5]))
        n_prev = int(rng.choice([0, 1, 30, 64, 100]))
        prev = rng.integers(0, n, n_prev)
        if n_prev:
            prev[: min(n_prev, 8)] = np.argsort(-np.nan_to_num(x, nan=-1e30, posinf=-1e30))[: min(n_prev, 8)]  # hit candidates
            rng.shuffle(prev)
        rnd = float(rng.random()) if case % 9 else 0.0
        t = Tensor.from_slice(dev, x)
        used = prev[-64:]
        if case % 2 == 0:
            top_p, min_p = float(rng.choice([1.0, 0.9, 0.5, 0.1])), float(rng.choice([0.0, 0.05, 0.3]))
            got, ids, vals = t.sample_standard_token(prev, GpuStandardSamplerParams(k, temp, pen, top_p, min_p, rnd), want_candidates=True)
            want = oracle.sample_token(x, 0, k, temp, pen, top_p, min_p, random=rnd, previous=used)
        else:
            mu0, tau, eta = float(rng.choice([1.0, 3.0, 10.0])), float(rng.choice([3.0, 5.0])), float(rng.choice([0.1, 0.3]))
            s = GpuMirostat2Sampler(dev, mu0)
            got, ids, vals = t.sample_mirostat2_token(s, prev, GpuMirostat2SamplerParams(k, temp, pen, tau, eta, rnd), want_candidates=True)
            want = oracle.sample_token(x, 1, k, temp, pen, tau=tau, eta=eta, random=rnd, previous=used, mu=mu0)
        what = (n, case, k, temp, pen, n_prev, rnd)
        assert ids.tolist() == want["ids"].tolist(), what
        live = want["ids"] != 0xFFFFFFFF
        assert np.array_equal(vals[live], want["values"][live]), what        # a processed -0.0 comes back as 0.0
        if want["margin"] > 1e-4:
            compared += 1
            assert got == want["token"], what
            if case % 2 and want["token"] is not None:
                assert s.mu == pytest.approx(want["mu"], rel=1e-5, abs=1e-5), what
    assert compared >= 30


def test_sample_token_previous_gpu_token(dev, oracle):
    """The id another kernel left in device memory joins the previous tokens as their last entry
    (fixed_previous_tokens_data_with_gpu_tail, fusor-ml/core/src/sampling/processors.rs:45-81): 63 host ids + 1."""
    from kalosm_amd.fusor import GpuStandardSamplerParams
    rng = np.random.default_rng(3)
    x = rng.standard_normal(500).astype(np.float32) * 3
    order = np.argsort(-x)
    tail = Tensor.from_slice(dev, np.array([order[0]], np.uint32), "u32")
    host = np.concatenate([[order[1]], rng.integers(400, 500, 70), [order[2]]]).astype(np.uint32)   # order[1] falls out of the 63
    p = GpuStandardSamplerParams(16, 1.0, 1.8, 1.0, 0.0, 0.4)
    got, ids, vals = Tensor.from_slice(dev, x).sample_standard_token(host, p, previous_gpu_token=tail, want_candidates=True)
    want = oracle.sample_token(x, 0, 16, 1.0, 1.8, random=0.4, previous=np.concatenate([host[-63:], [order[0]]]))
    assert ids.tolist() == want["ids"].tolist() and np.array_equal(vals, want["values"])
    assert got == want["token"]
    seen = dict(zip(ids.tolist(), vals.tolist()))
    assert seen[int(order[1])] == x[order[1]]                       # outside the window: not penalised
    assert seen.get(int(order[0]), None) != x[order[0]]             # the device-side id is penalised


@pytest.mark.parametrize("n", [1, 1000, 70001, 3_000_000])
def test_check_finite_counts_and_first_indices(dev, n):
    """debug_check_nan_f32 (models/kalosm-llama/src/raw/mod.rs:9-58): counts, largest finite magnitude and the first
    four NaN indices, against numpy; clean tensors, NaNs in several scan segments, fewer than four NaNs."""
    from kalosm_amd.fusor import Tensor
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    for variant in range(4):
        a = x.copy()
        if variant >= 1:
            a[rng.integers(0, n, min(n, 3))] = np.inf
            a[rng.integers(0, n, min(n, 2))] = -np.inf
        if variant == 2:
            a[rng.integers(0, n, min(n, 2))] = np.nan  # at most two NaNs
        if variant == 3:
            a[rng.integers(0, n, min(n, 50))] = np.nan
            a[n - 1] = np.float32(np.nan)
        got = Tensor.from_slice(dev, a).check_finite()
        nan_idx = np.flatnonzero(np.isnan(a))
        fin = a[np.isfinite(a)]
        assert got["nan"] == nan_idx.size
        assert got["pos_inf"] == int(np.sum(a == np.inf)) and got["neg_inf"] == int(np.sum(a == -np.inf))
        assert got["max_abs"] == (np.abs(fin).max() if fin.size else 0.0)
        assert got["first_nan_indices"] == nan_idx[:4].tolist()
