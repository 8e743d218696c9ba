"""End-to-end decoder parity: the HIP decoder against the CPU checker's decoder on the same seeded random-init
weights (the reference stores no logits for any model, so this is pinned by the checker only)."""
import numpy as np
import pytest

from refgen import assert_close, assert_greedy_follows
from kalosm_amd import synth
from kalosm_amd.llama import Model

pytestmark = pytest.mark.gpu

SMALL = dict(n_layers=2, d_model=512, n_heads=8, n_kv_heads=2, head_dim=64, ffn=1024, vocab=1024, ctx=256, eps=1e-5,
             theta=500000.0)
# head_dim 128 with four query heads per KV head: the shapes the decode-step attention kernel is written for
HD128 = dict(n_layers=2, d_model=512, n_heads=4, n_kv_heads=1, head_dim=128, ffn=1024, vocab=1024, ctx=512, eps=1e-5,
             theta=500000.0)


def build_pair(dev, oracle, cfg, seed=0, sigma=2e-4, **kw):
    weights = {}
    m = Model.random_init(dev, cfg, seed=seed, sigma=sigma, keep=lambda n, a: weights.__setitem__(n, a), **kw)
    ocfg = dict(cfg, type_attn=synth.Q4_K, type_ffn_gate_up=synth.Q4_K, type_ffn_down=synth.Q6_K, type_embd=synth.Q4_K,
                type_output=synth.Q6_K)
    return m, oracle.Llama(ocfg, weights)


@pytest.mark.parametrize("variant", [dict(fuse_qkv=True, fuse_gate_up=True, use_graph=True),
                                     dict(fuse_qkv=False, fuse_gate_up=False, use_graph=False),
                                     dict(fuse_qkv=True, fuse_gate_up=True, use_graph=True, kv_dtype="f16")],
                         ids=["fused+graph", "separate+eager", "f16-kv"])
@pytest.mark.parametrize("cfg", [SMALL, HD128], ids=["hd64", "hd128"])
def test_decoder_matches_checker(dev, oracle, variant, cfg):
    m, ref = build_pair(dev, oracle, cfg, **variant)
    rng = np.random.default_rng(1)
    prompt = rng.integers(0, cfg["vocab"], 9)
    # an f16 KV cache is an option of this library (the reference caches f32): its rounding sets the tolerance there
    tol = dict(abs_tol=5e-2, rel_tol=5e-3) if variant.get("kv_dtype") == "f16" else dict(abs_tol=1e-2, rel_tol=1e-3)
    # prefill
    lg, hid = m.forward(prompt, want_hidden=True)
    wl, wh = ref.forward(prompt, want_hidden=True)
    assert_close(hid, wh, what="prefill hidden", **tol)
    assert_close(lg, wl, what="prefill logits", **tol)
    # token-by-token decode through forward()
    tok = int(np.argmax(wl))
    for step in range(3):
        lg = m.forward([tok])
        wl = ref.forward([tok])
        assert_close(lg, wl, what=f"decode step {step} logits", **tol)
        tok = int(np.argmax(wl))
    # greedy decode on the device (graph replay when enabled) against the checker's greedy loop
    steps = 6
    got, ms = m.decode_greedy(tok, steps)
    assert_greedy_follows(ref, tok, got)
    # a second greedy run after a reset replays the captured step from position 0
    m.reset(); ref.reset()
    lg = m.forward(prompt); wl = ref.forward(prompt)
    assert_close(lg, wl, what="prefill logits after reset", **tol)
    got2, _ = m.decode_greedy(int(np.argmax(wl)), 4)
    assert_greedy_follows(ref, int(np.argmax(wl)), got2, what="after reset")
    # a longer run crosses the key ranges of the attention splits; afterwards the cache the device-side steps wrote
    # must give the checker's logits through the eager path
    got3, _ = m.decode_greedy(int(got2[-1]), 40)
    assert_greedy_follows(ref, int(got2[-1]), got3, what="40 more steps")
    last = int(got3[-1])
    if variant.get("kv_dtype") == "f16":  # 60 cached positions rounded to f16 (the checker's cache is f32)
        tol = dict(abs_tol=5e-2, rel_tol=5e-3)
    assert_close(m.forward([last]), ref.forward([last]), what="logits after 40 device-side steps", **tol)


@pytest.mark.parametrize("heads,kv_heads", [(4, 1), (4, 2), (8, 1), (2, 2), (6, 2)], ids=["g4", "g2", "g8", "g1", "g3"])
@pytest.mark.parametrize("opts", [{}, dict(attn_heads=2), dict(attn_heads=4, attn_waves=8), dict(attn_splits=4, wo_tiles=1),
                                  dict(wo_tiles=2, down_tiles=2, matvec_tiles=2), dict(matvec_per=2, down_tiles=4),
                                  dict(attn_kernel=4), dict(attn_kernel=4, attn_heads=4, attn_waves=8)],
                         ids=["default", "heads2", "heads4-waves8", "splits4-wo1", "tiles2", "per2-down4", "twopass",
                              "twopass-heads4"])
def test_decode_step_kernel_variants(dev, oracle, heads, kv_heads, opts):
    """The fused decode step (head_dim 128) with other groupings of query heads per KV head and with the kernel
    shapes the options select: 70 greedy steps on the device (five granules of 16 keys, so every attention split
    owns keys and the blind prefetch reads past the length) against the checker's greedy loop, then the logits
    through the eager path on the cache the device-side steps wrote."""
    cfg = dict(HD128, n_heads=heads, n_kv_heads=kv_heads, d_model=128 * heads)
    m, ref = build_pair(dev, oracle, cfg, seed=3)
    for k, v in opts.items():
        dev.set_option(k, v)
    try:
        prompt = np.random.default_rng(5).integers(0, cfg["vocab"], 11)
        lg, wl = m.forward(prompt), ref.forward(prompt)
        assert_close(lg, wl, what="prefill logits")
        t = int(np.argmax(wl))
        got, _ = m.decode_greedy(t, 70)
        assert_greedy_follows(ref, t, got)
        last = int(got[-1])
        assert_close(m.forward([last]), ref.forward([last]), what="logits after 70 device-side steps")
    finally:
        for k in opts:
            dev.set_option(k, 0)


@pytest.mark.parametrize("variant", [dict(), dict(fuse_qkv=False, fuse_gate_up=False, use_graph=False), dict(five_bit=True)],
                         ids=["fused+graph", "separate+eager", "q5_0+q5_k+f16"])
def test_decoder_from_gguf_file(dev, oracle, variant, tmp_path):
    """Model::from_gguf (raw/mod.rs:284-648) on a small random-init file with what model files really hold:
    block types that change from layer to layer (so q|k|v and gate|up cannot always be fused), f32 and f16 norm
    vectors, a rope_freqs.weight tensor, tokenizer metadata beside the model keys.  The checker's decoder is fed
    from the same file through the plain-Python reader."""
    from test_gguf_reader import TINY, llama_file
    from oracle import gguf_ref
    variant = dict(variant)
    data, weights, types = llama_file(TINY, seed=5, five_bit=variant.pop("five_bit", False))
    path = tmp_path / "tiny.gguf"
    path.write_bytes(data)
    m = Model.from_gguf(dev, str(path), ctx=80, **variant)
    assert m.cfg == {**TINY, "ctx": 80, "eps": float(np.float32(1e-5))}
    r = gguf_ref.GgufRef(data)
    rw = {}
    for name, (ty, shape, off) in r.tensors.items():
        raw = r.tensor_bytes(name)
        if ty == 0 and len(shape) == 1:
            raw = raw.view(np.float32)
        elif ty == 1 and len(shape) == 1:  # vectors are widened at load (norm weights); matrices stay f16 rows
            raw = raw.view(np.float16).astype(np.float32)
        rw[name.decode()] = raw
    ocfg = dict(m.cfg, type_attn=synth.Q4_K, type_ffn_gate_up=synth.Q4_K, type_ffn_down=synth.Q6_K,
                type_embd=types["token_embd.weight"], type_output=types["output.weight"],
                tensor_types={n.decode(): t for n, (t, _, _) in r.tensors.items()})
    ref = oracle.Llama(ocfg, rw)
    rng = np.random.default_rng(2)
    prompt = rng.integers(0, TINY["vocab"], 11)
    lg, hid = m.forward(prompt, want_hidden=True)
    wl, wh = ref.forward(prompt, want_hidden=True)
    assert_close(hid, wh, what="prefill hidden")
    assert_close(lg, wl, what="prefill logits")
    tok = oracle.argmax(wl)
    got, _ = m.decode_greedy(tok, 30)
    assert_greedy_follows(ref, tok, got)
    last = int(got[-1])
    assert_close(m.forward([last]), ref.forward([last]), what="logits after 30 device-side steps")
    # the rope_freqs factors matter: the same file without them gives other logits
    cos, sin = oracle.rope_tables_weighted(64, 4, 500000.0, weights["rope_freqs.weight"])
    c0, s0 = oracle.rope_tables(64, 4, 500000.0)
    assert not np.allclose(cos[3], c0[3]) and np.array_equal(cos[0], c0[0])
    # weights by name through the VarBuilder
    from kalosm_amd.gguf import VarBuilder
    vb = VarBuilder.from_gguf(str(path))
    q = vb.pp("blk").pp(0).get("attn_v.weight", dev)
    assert q.shape() == (128, 256) and q.ggml_type == synth.Q6_K
    want_w = oracle.dequantize(synth.Q6_K, weights["blk.0.attn_v.weight"]).reshape(128, 256)
    assert np.array_equal(q.dequantize().as_slice().view(np.uint32), want_w.view(np.uint32))
    with pytest.raises(Exception) as e:
        vb.get("blk.9.attn_v.weight", dev)
    assert "not found" in str(e.value)
    # parts of different block types do not concatenate (None in the reference, core/src/quantized/mod.rs:329-337)
    from kalosm_amd.fusor import QMatrix
    assert QMatrix.concat_rows([vb.get("blk.0.attn_k.weight", dev), q]) is None


def test_decoder_from_gguf_refuses_other_variants(dev):
    """Tensors of attention / norm variants this decoder does not implement are refused, not skipped."""
    from test_gguf_reader import TINY, llama_file
    from kalosm_amd.gguf import GgufMetadata
    bias = np.zeros(256, np.float32).view(np.uint8)
    data, _, _ = llama_file(TINY, extra_tensors=[("blk.0.attn_q.bias", 0, (256,), bias)])
    with pytest.raises(Exception) as e:
        Model.from_gguf(dev, GgufMetadata.read_bytes(data))
    assert "attn_q.bias" in str(e.value)


def test_decoder_errors(dev):
    from kalosm_amd.fusor import FusorHipError
    m = Model(dev, SMALL)
    with pytest.raises(FusorHipError, match="missing"):
        m.finalize()
    with pytest.raises(FusorHipError, match="expected"):
        m.load_tensor("blk.0.attn_q.weight", synth.Q4_K, 16, 256, synth.random_weight(synth.Q4_K, 16, 256, 1))
    with pytest.raises(FusorHipError, match="unknown tensor"):
        m.load_tensor("blk.0.nope.weight", synth.Q4_K, 16, 256, synth.random_weight(synth.Q4_K, 16, 256, 1))


@pytest.mark.parametrize("use_graph", [True, False], ids=["graph", "eager"])
@pytest.mark.parametrize("kind", ["standard", "mirostat2"])
def test_sampled_decode_matches_checker(dev, oracle, use_graph, kind):
    """Sampled decode with the token resident on the device (models/kalosm-llama/src/model/inference.rs:38-173)
    against the checker fed the same tokens: at every step the checker's sampler, on the checker's logits, with the
    same window of previous ids and the same random number, must pick the id the device picked, unless its own
    deciding comparison is closer than the logit tolerance allows (relative gap below 2e-2) or the two ids' processed
    logits are within 1e-2 of each other."""
    from kalosm_amd.fusor import GpuMirostat2SamplerParams, GpuStandardSamplerParams
    cfg = HD128
    m, ref = build_pair(dev, oracle, cfg, sigma=2e-2, fuse_qkv=True, fuse_gate_up=True, use_graph=use_graph)
    rng = np.random.default_rng(11)
    prompt = rng.integers(0, cfg["vocab"], 12)
    wl = ref.forward(prompt)
    m.forward(prompt)
    history = prompt.tolist()
    first = int(np.argmax(wl))
    rounds = [(10, 24, 1.3, 16), (10, 24, 1.3, 16), (7, 40, 1.6, 5)]        # steps, top_k, penalty, window
    mu = 6.0
    close = 0
    for rnd_i, (steps, k, pen, window) in enumerate(rounds):
        randoms = rng.random(steps).astype(np.float32)
        if kind == "standard":
            p = GpuStandardSamplerParams(k, 0.9, pen, 0.95, 0.01, 0.0)
        else:
            p = GpuMirostat2SamplerParams(k, 0.9, pen, 4.0, 0.2, 0.0)
        got, ms, mu_after = m.decode_sampled(first, steps, p, randoms, previous_tokens=history, repetition_range=window, mu=mu)
        t, mu_ref, exact = first, mu, True
        for i in range(steps):
            history.append(t)
            wl = ref.forward([t])
            prev = history[-window:]
            if kind == "standard":
                want = oracle.sample_token(wl, 0, k, 0.9, pen, 0.95, 0.01, random=float(randoms[i]), previous=prev)
            else:
                want = oracle.sample_token(wl, 1, k, 0.9, pen, tau=4.0, eta=0.2, random=float(randoms[i]), previous=prev, mu=mu_ref)
                mu_ref = want["mu"]
            g = int(got[i])
            if g != want["token"]:
                vals = dict(zip(want["ids"].tolist(), want["values"].tolist()))
                near = g in vals and abs(vals[g] - vals[want["token"]]) < 1e-2
                assert want["margin"] < 2e-2 or near, (rnd_i, i, g, want["token"], want["margin"])
                close += 1
                exact = False
            t = g
        if kind == "mirostat2" and exact:
            assert mu_after == pytest.approx(mu_ref, rel=1e-3, abs=1e-3)
        mu = mu_after
        first = t
    assert close <= 3
    # the cache the sampled steps wrote gives the checker's logits through the eager path
    assert_close(m.forward([first]), ref.forward([first]), what="logits after the sampled steps", abs_tol=1e-2, rel_tol=1e-3)


@pytest.mark.parametrize("rope_freqs", [True, False], ids=["with-rope_freqs", "plain"])
def test_decoder_with_rope_scaling(dev, oracle, tmp_path, rope_freqs):
    """The `rope_scaling` argument of Model::from_gguf (models/kalosm-llama/src/raw/mod.rs:264-285): the decoder's
    RoPE tables use the scaled inverse frequencies (raw/rope.rs:20-38), then the rope_freqs.weight factors.  With
    original_max_position_embeddings 32 and low_freq_factor 1 every frequency whose wavelength exceeds 32
    positions is divided by 8, so the logits differ from the unscaled decoder's from position 1 on."""
    from test_gguf_reader import TINY, llama_file
    from oracle import gguf_ref
    scaling = (8.0, 4.0, 1.0, 32)
    data, weights, types = llama_file(TINY, seed=7, rope_freqs=rope_freqs)
    m = Model.from_gguf(dev, _bytes_source(data, tmp_path), ctx=80, rope_scaling=scaling)
    plain = Model.from_gguf(dev, _bytes_source(data, tmp_path), ctx=80)
    r = gguf_ref.GgufRef(data)
    rw = {}
    for name, (ty, shape, off) in r.tensors.items():
        raw = r.tensor_bytes(name)
        if len(shape) == 1:
            raw = raw.view(np.float32) if ty == 0 else raw.view(np.float16).astype(np.float32)
        rw[name.decode()] = raw
    ocfg = dict(m.cfg, type_attn=synth.Q4_K, type_ffn_gate_up=synth.Q4_K, type_ffn_down=synth.Q6_K,
                type_embd=types["token_embd.weight"], type_output=types["output.weight"],
                tensor_types={n.decode(): t for n, (t, _, _) in r.tensors.items()}, rope_scaling=scaling)
    ref = oracle.Llama(ocfg, rw)
    prompt = np.random.default_rng(4).integers(0, TINY["vocab"], 40)
    lg = m.forward(prompt)
    wl = ref.forward(prompt)
    assert_close(lg, wl, what="prefill logits with scaled RoPE")
    assert np.abs(plain.forward(prompt) - wl).max() > 50 * np.abs(lg - wl).max()    # the scaling is not a no-op
    tok = oracle.argmax(wl)
    got, _ = m.decode_greedy(tok, 12)
    assert_greedy_follows(ref, tok, got, what="scaled RoPE")
    with pytest.raises(Exception):
        m.set_rope_scaling(*scaling)            # the tables are built: too late


def test_forward_trims_the_context_when_it_is_full(dev, oracle):
    """Model::forward with a full context (raw/mod.rs:769-801): the cache is cleared and the last context_length - 32
    tokens of everything seen so far, the new ones included, are run again from position 0.  48 + 12 device-side steps
    fill a context of 64; the next 7 tokens overflow it; the logits must be the checker's for the 32 most recent ids
    alone, and decoding goes on from position 32."""
    cfg = dict(HD128, ctx=64)
    m, ref = build_pair(dev, oracle, cfg, seed=13)
    rng = np.random.default_rng(14)
    prompt = rng.integers(0, cfg["vocab"], 48)
    first = int(np.argmax(m.forward(prompt)))
    got, _ = m.decode_greedy(first, 12)                      # cache: prompt, first, got[:-1] = 60 positions
    seen = prompt.tolist() + [first] + got.tolist()[:-1]
    more = rng.integers(0, cfg["vocab"], 7).tolist()         # 60 + 7 > 64
    lg = m.forward(more)
    tail = (seen + more)[-32:]
    want = ref.forward(tail)
    assert_close(lg, want, what="logits after the context was trimmed")
    t = int(np.argmax(want))
    got2, _ = m.decode_greedy(t, 5)
    assert_greedy_follows(ref, t, got2, what="steps after the trim")
    with pytest.raises(Exception, match="context overflow"):
        m.decode_greedy(int(got2[-1]), 64)                   # the device-side loop does not trim


def _bytes_source(data, tmp_path):
    p = tmp_path / f"m{len(list(tmp_path.iterdir()))}.gguf"
    p.write_bytes(data)
    return str(p)


def test_graph_decode_survives_scratch_reallocation(oracle):
    """A captured decode step holds the device's scratch buffers as kernel arguments.  A larger call between two
    decodes (here a 100-token prompt and a 300-row matmul whose k-split planes, activation planes and partial sums
    outgrow the buffers the capture saw) reallocates them; the next decode must capture again instead of replaying
    kernels that point at freed memory.  Own device handle, so the buffers start at their minimum size."""
    from kalosm_amd.fusor import Device, FusorHipError, GpuStandardSamplerParams, QMatrix, Tensor
    d = Device.gpu(0)
    cfg = dict(n_layers=2, d_model=1024, n_heads=8, n_kv_heads=2, head_dim=128, ffn=2048, vocab=2048, ctx=512, eps=1e-5,
               theta=500000.0)
    m, ref = build_pair(d, oracle, cfg, seed=9)
    rng = np.random.default_rng(3)


    # a user graph over a small matvec, captured while the scratch is small
    w = QMatrix.from_raw_bytes(d, (64, 512), synth.random_weight(synth.Q8_0, 64, 512, 1), synth.Q8_0)
    xs = Tensor.from_slice(d, synth.random_activation(8, 512, 2))
    ys = Tensor.zeros(d, (8, 64))
    xs.q_mat_mul(w, out=ys)          # eager first: sizes what the capture needs
    d.graph_begin()
    xs.q_mat_mul(w, out=ys)
    g = d.graph_end()
    g.launch()
    d.sync()

    prompt = rng.integers(0, cfg["vocab"], 6)
    wl = ref.forward(prompt)
    m.forward(prompt)
    first = oracle.argmax(wl)
    p = GpuStandardSamplerParams(1, 1.0, 1.0, 1.0, 0.0, 0.0)      # top_k 1: the sampled step picks the argmax
    got, _, _ = m.decode_sampled(first, 5, p, np.full(5, 0.5, np.float32), repetition_range=0)
    assert_greedy_follows(ref, first, got, what="sampled steps with top_k 1")
    last = int(got[-1])
    got, _ = m.decode_greedy(last, 5)
    assert_greedy_follows(ref, last, got)
    # larger calls on the same device: every scratch buffer is outgrown
    m.reset(); ref.reset()
    long_prompt = rng.integers(0, cfg["vocab"], 100)
    wl = ref.forward(long_prompt)
    assert_close(m.forward(long_prompt), wl, what="100-token prefill logits")
    big = QMatrix.from_raw_bytes(d, (2048, 4096), synth.random_weight(synth.Q4_K, 2048, 4096, 4), synth.Q4_K)
    Tensor.from_slice(d, synth.random_activation(300, 4096, 5)).q_mat_mul(big).as_slice()
    Tensor.from_slice(d, synth.random_activation(16, 4096, 6)).q_mat_mul(big).as_slice()
    # same parameters, same cache capacity: only the reallocation can trigger the new capture
    first = oracle.argmax(wl)
    got, _, _ = m.decode_sampled(first, 6, p, np.full(6, 0.5, np.float32), repetition_range=0)
    assert_greedy_follows(ref, first, got, what="sampled steps after the reallocation")
    got2, _ = m.decode_greedy(int(got[-1]), 6)
    assert_greedy_follows(ref, int(got[-1]), got2, what="greedy steps after the reallocation")
    # the user graph is refused with an error that says why
    with pytest.raises(FusorHipError, match="captured"):
        g.launch()
    del g, m
    d.sync()


def test_deterministic_option_gives_identical_bits(dev, oracle):
    """The default decode step adds the k-split partial sums of the output projection and of the Q6_K down projection
    with float atomics, so the last bits of its hidden state depend on the arrival order.  With the `deterministic`
    option the step uses the ordered kernels: three runs of 24 replayed steps must give bit-identical logits and the
    checker's tokens; afterwards the default step is captured again (options are part of the capture key)."""
    cfg = dict(HD128, n_heads=8, n_kv_heads=2, d_model=1024, ffn=2048)
    m, ref = build_pair(dev, oracle, cfg, seed=12)
    prompt = np.random.default_rng(8).integers(0, cfg["vocab"], 10)
    wl = ref.forward(prompt)
    first = oracle.argmax(wl)
    want, t = [], first
    for _ in range(24):
        t = oracle.argmax(ref.forward([t]))
        want.append(t)

    def run():
        m.reset()
        m.forward(prompt)
        got, _ = m.decode_greedy(first, 24)
        return got.tolist(), m.forward([int(got[-1])])

    dev.set_option("deterministic", 1)
    try:
        runs = [run() for _ in range(3)]
    finally:
        dev.set_option("deterministic", 0)
    for toks, lg in runs:
        assert toks == want
        assert np.array_equal(lg.view(np.uint32), runs[0][1].view(np.uint32))
    toks, lg = run()                       # default kernels again: same tokens, logits within tolerance
    assert toks == want
    assert_close(lg, runs[0][1], what="default step against the deterministic one")


def test_forward_trace_reports_timing_and_non_finite_layers(dev):
    """The trace switches of the reference's forward (KALOSM_TRACE_FORWARD_TIMING / FUSOR_TRACE_GPU_KERNELS /
    KALOSM_TRACE_LAYER_NAN, models/kalosm-llama/src/raw/mod.rs:943-1043) as device options: per-stage and layer-loop
    timing lines, no NaN line for a healthy model, and - with one NaN planted in layer 1's attention norm weight -
    NaN lines from layer 1 on, with the counts and first indices that weight implies."""
    cfg = SMALL
    D, L = cfg["d_model"], cfg["n_layers"]
    prompt = np.random.default_rng(5).integers(0, cfg["vocab"], 9)

    def build(poison):
        m = Model(dev, cfg, use_graph=False)
        for name, ty, n, k in synth.llama_tensor_specs(cfg):
            data = synth.llama_random_tensor(name, ty, n, k, 0, 2e-4)
            if poison and name == "blk.1.attn_norm.weight":
                data = data.copy()
                data.view(np.float32)[3] = np.nan
            m.load_tensor(name, ty, n, k, data)
        m.finalize()
        return m

    try:
        m = build(False)
        m.forward(prompt)
        assert m.trace_text() == ""  # everything off: nothing recorded
        dev.set_option("trace_nan", 1)
        dev.set_option("trace_timing", 2)
        lg = m.forward([1, 2, 3])
        lines = m.trace_text().splitlines()
        assert not [l for l in lines if l.startswith("trace_nan")]
        stage = [l for l in lines if l.startswith("[timing] layer ")]
        assert len(stage) == 5 * L and stage[0].startswith("[timing] layer 0 attn_norm+qkv: ")
        assert sum(l.startswith("[timing] out_norm+lm_head: ") for l in lines) == 1
        total = [l for l in lines if l.startswith("[timing] text layer loop: ")]
        assert len(total) == 1 and total[0].endswith("seq_len=3")
        loop_ms = float(total[0].split(": ")[1].split(" ms")[0])
        stage_us = sum(float(l.rsplit(": ", 1)[1].split(" us")[0]) for l in stage)
        assert loop_ms > 0 and abs(stage_us / 1e3 - loop_ms) < 1e-3 * max(1.0, loop_ms) + 0.01  # stages tile the loop
        # tracing does not change the result
        dev.set_option("trace_nan", 0)
        dev.set_option("trace_timing", 0)
        m.reset()
        m.forward(prompt)
        assert np.array_equal(m.forward([1, 2, 3]), lg)
        # layer-loop total only
        dev.set_option("trace_timing", 1)
        m.forward([4])
        assert [l.split(":")[0] for l in m.trace_text().splitlines()] == ["[timing] text layer loop"]
        dev.set_option("trace_timing", 0)

        bad = build(True)
        dev.set_option("trace_nan", 1)
        out = bad.forward(prompt)
        assert np.isnan(out).all()
        lines = [l for l in bad.trace_text().splitlines() if l.startswith("trace_nan")]
        assert lines and all(" layer=1 " in l for l in lines)  # the embedding and layer 0 are clean
        s = prompt.size
        first = lines[0]
        assert first.startswith(f"trace_nan layer=1 label=post_attn_norm index_pos=0 shape=[1, {s}, {D}] nan={s} ")
        assert f"first_nan_indices=[3, {3 + D}, {3 + 2 * D}, {3 + 3 * D}]" in first and "+inf=0 -inf=0" in first
        labels = [l.split("label=")[1].split(" ")[0] for l in lines]
        assert labels == ["post_attn_norm", "attn_out", "ffn_unfused"]
        assert f"nan={s * D} " in lines[1] and f"nan={s * D} " in lines[2]  # a NaN input poisons every output
        # single-token steps take the fused residual form
        bad.forward([7])
        assert [l.split("label=")[1].split(" ")[0] for l in bad.trace_text().splitlines()][-1] == "ffn_fused"
    finally:
        for key in ("trace_nan", "trace_timing", "trace_stderr"):
            dev.set_option(key, 0)


def test_trace_switches_from_the_environment():
    """The reference's variables, present in the environment when the device is created, switch the trace on and send
    its lines to stderr (raw/mod.rs:943-955; fusor-ml/core/src/compute_graph/resolve/run.rs:141)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import numpy as np\n"
        "from kalosm_amd.fusor import Device\n"
        "from kalosm_amd.llama import Model\n"
        f"cfg = {SMALL!r}\n"
        "m = Model.random_init(Device.gpu(0), cfg, seed=0, sigma=2e-4, use_graph=False)\n"
        "m.forward([1, 2, 3, 4])\n"
        "print('TEXT', len(m.trace_text().splitlines()))\n")
    env = dict(os.environ, PYTHONPATH=root, FUSOR_TRACE_GPU_KERNELS="1", KALOSM_TRACE_LAYER_NAN="1")
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stderr[-2000:]
    err = [l for l in r.stderr.splitlines() if l.startswith("[timing]") or l.startswith("trace_nan")]
    assert len(err) == 5 * SMALL["n_layers"] + 2 and err[-1].startswith("[timing] text layer loop: ")
    assert f"TEXT {len(err)}" in r.stdout
    env = {k: v for k, v in env.items() if k not in ("FUSOR_TRACE_GPU_KERNELS", "KALOSM_TRACE_LAYER_NAN")}
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=100)
    assert r.returncode == 0 and "TEXT 0" in r.stdout and "[timing]" not in r.stderr
