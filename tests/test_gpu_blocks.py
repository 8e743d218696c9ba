"""GPU parity: block decode (bit-exact) and decode-side quantized matmul against the CPU checker."""
import numpy as np
import pytest

import refgen
from refgen import Q4_0, Q4_K, Q6_K, Q8_0, assert_close
from kalosm_amd import synth
from kalosm_amd.fusor import FusorHipError, QMatrix, Tensor

pytestmark = pytest.mark.gpu
ALL = [Q4_0, Q8_0, Q4_K, Q6_K]
NAMES = synth.TYPE_NAMES


def h16(v):
    return np.frombuffer(np.float32(v).astype(np.float16).tobytes(), np.uint8)


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("n,k", [(1, 256), (16, 512), (37, 1024), (130, 768)])
def test_dequantize_bit_exact(dev, oracle, ty, n, k):
    """QMatrix::dequantize == GgufBlock::dequantize bit for bit, including row counts that are not a multiple
    of the 16-row tile and block counts that are not a multiple of the record size."""
    raw = synth.random_weight(ty, n, k, seed=100 + n + k + ty)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    got = q.dequantize().as_slice()
    want = oracle.dequantize(ty, raw).reshape(n, k)
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
def test_dequantize_edge_blocks(dev, oracle, ty):
    """negative and subnormal f16 scales, sub-scales 0 and 63, all-zero and all-0xFF blocks (NaN scale)."""
    rng = np.random.default_rng(7)
    nb = 64
    raw = synth.random_blocks(ty, nb, rng).reshape(nb, -1).copy()
    raw[0, :] = 0
    raw[1, :] = 0xFF
    if ty == Q4_K:
        raw[2, 0:2] = h16(3e-6); raw[2, 2:4] = h16(-2e-6)
        raw[3, 4:16] = synth.pack_k4_scales(np.full(8, 63, np.uint8), np.zeros(8, np.uint8))
        raw[4, 4:16] = synth.pack_k4_scales(np.zeros(8, np.uint8), np.full(8, 63, np.uint8))
    elif ty == Q6_K:
        raw[2, 208:210] = h16(-4e-6); raw[3, 192:208] = 0x80
    else:
        raw[2, 0:2] = h16(-5e-7)
    e = synth.BLOCK_ELEMS[ty]
    n, k = 4, nb // 4 * e
    q = QMatrix.from_raw_bytes(dev, (n, k), raw.reshape(-1), ty)
    got = q.dequantize().as_slice()
    want = oracle.dequantize(ty, raw.reshape(-1)).reshape(n, k)
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
def test_dequantize_reference_fixture_bytes(dev, oracle, ty):
    """The reference's deterministic fixture generators (conformance common/quantized.rs:175-272)."""
    e = synth.BLOCK_ELEMS[ty]
    n, k = 24, 2 * e * 3
    raw = refgen.REF_GENERATORS[ty](n * (k // e))
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    assert np.array_equal(bits(q.dequantize().as_slice()), bits(oracle.dequantize(ty, raw).reshape(n, k)))


def test_known_answers(dev):
    """core/src/quantized/matmul/tests.rs:1337-1397 (+-528) and the Q4_K analogue of :1399-1423 (32896)."""
    x = Tensor.from_slice(dev, np.arange(1, 33, dtype=np.float32)[None, :])
    raw = np.concatenate([h16(1.0), np.full(16, 0x99, np.uint8), h16(1.0), np.full(16, 0x77, np.uint8)])
    y = x.q_mat_mul(QMatrix.from_raw_bytes(dev, (2, 32), raw, Q4_0)).as_slice()
    assert y.shape == (1, 2) and abs(y[0, 0] - 528) < 1e-3 and abs(y[0, 1] + 528) < 1e-3
    raw = np.concatenate([h16(1.0), np.full(32, 1, np.uint8), h16(1.0), np.full(32, 0xFF, np.uint8)])
    y = x.q_mat_mul(QMatrix.from_raw_bytes(dev, (2, 32), raw, Q8_0)).as_slice()
    assert abs(y[0, 0] - 528) < 1e-3 and abs(y[0, 1] + 528) < 1e-3
    raw = np.concatenate([h16(1.0), h16(0.0), np.uint8([1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1]), np.full(128, 0x11, np.uint8)])
    x = Tensor.from_slice(dev, np.arange(1, 257, dtype=np.float32)[None, :])
    y = x.q_mat_mul(QMatrix.from_raw_bytes(dev, (1, 256), raw, Q4_K)).as_slice()
    assert abs(y[0, 0] - 32896) < 1e-2


def test_config0_q4_0_matvec(dev, oracle):
    """Benchmark configuration 0: Q4_0 4096x4096, f16 scales ~ N(0, 0.02), uniform nibbles, x ~ N(0,1) f32, batch 1."""
    n = k = 4096
    raw = synth.random_weight(Q4_0, n, k, seed=1)
    x = synth.random_activation(1, k, seed=2)
    got = Tensor.from_slice(dev, x).q_mat_mul(QMatrix.from_raw_bytes(dev, (n, k), raw, Q4_0)).as_slice()
    want = oracle.q_mat_mul(Q4_0, x, raw, n)
    assert_close(got, want, what="Q4_0 4096x4096 m=1")


@pytest.mark.parametrize("kernel", [1, 0], ids=["generic", "auto"])
@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m", [1, 2, 4, 16])
def test_qmatmul_small_m_vs_checker(dev, oracle, ty, m, kernel):
    """Tolerance of the north star: 1e-3 relative or 1e-2 absolute per element, f32 accumulation."""
    n, k = 272, 2048
    raw = synth.random_weight(ty, n, k, seed=20 + ty)
    x = synth.random_activation(m, k, seed=30 + m)
    dev.set_option("matvec_kernel", kernel)
    try:
        q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
        out = Tensor.filled_bytes(dev, (m, n), 0xFF)  # poisoned output: unwritten elements show as NaN
        got = Tensor.from_slice(dev, x).q_mat_mul(q, out=out).as_slice()
    finally:
        dev.set_option("matvec_kernel", 0)
    want = oracle.q_mat_mul(ty, x, raw, n)
    assert_close(got, want, what=f"{NAMES[ty]} {n}x{k} m={m}")


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m", [2, 3, 4])
@pytest.mark.parametrize("n,k", [(100, 14336), (272, 5120), (48, 8704)])
def test_qmatmul_few_rows_long_k(dev, oracle, ty, m, n, k):
    """2 .. 4 rows with k longer than one workgroup of the row kernel takes: 56 blocks in four parts of 14, 20 blocks in two
    parts of 10 (their planes are added by a second launch), 34 blocks (no even split into parts of at most 16: another
    kernel); ragged last tile; plain and two-residual epilogue; one and two row tiles per wavefront."""
    raw = synth.random_weight(ty, n, k, seed=180 + ty)
    x = synth.random_activation(m, k, seed=190 + m)
    a, b = synth.random_activation(m, n, seed=191), synth.random_activation(m, n, seed=192)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    want = oracle.q_mat_mul(ty, x, raw, n)
    xt = Tensor.from_slice(dev, x)
    try:
        for tiles in (0, 1, 2):
            dev.set_option("matvec_tiles", tiles)
            got = xt.q_mat_mul(q, out=Tensor.filled_bytes(dev, (m, n), 0xFF)).as_slice()
            assert_close(got, want, what=f"{NAMES[ty]} {n}x{k} m={m} tiles={tiles}")
            got = xt.q_mat_mul_add2(q, Tensor.from_slice(dev, a), Tensor.from_slice(dev, b),
                                    out=Tensor.filled_bytes(dev, (m, n), 0xFF)).as_slice()
            assert_close(got, oracle.add3(want, a, b), what=f"add2 {NAMES[ty]} {n}x{k} m={m} tiles={tiles}")
    finally:
        dev.set_option("matvec_tiles", 0)


@pytest.mark.parametrize("n,k", [(1024, 4096), (1000, 4096), (40, 256), (264, 2048), (512, 14336), (2048, 8192)])
def test_q4k_single_row_rows_of_a_tile_split_over_workgroups(dev, oracle, n, k):
    """The single-row Q4_K kernel with the 16 rows of a tile shared out over 2 or 4 workgroups (2 or 4 blocks per
    wavefront and MFMA): few row tiles for the device (the default for up to 128 tiles on 256 compute units), a ragged
    last tile, 1 .. 56 blocks of k, one and two block groups per wavefront; plain and two-residual epilogue."""
    raw = synth.random_weight(Q4_K, n, k, seed=210)
    x = synth.random_activation(1, k, seed=211)
    a, b = synth.random_activation(1, n, seed=212), synth.random_activation(1, n, seed=213)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, Q4_K)
    want = oracle.q_mat_mul(Q4_K, x, raw, n)
    xt = Tensor.from_slice(dev, x)
    try:
        for rs, per in ((0, 0), (1, 0), (2, 0), (2, 2), (4, 0)):
            dev.set_option("matvec_rowsplit", rs)
            dev.set_option("matvec_per", per)
            got = xt.q_mat_mul(q, out=Tensor.filled_bytes(dev, (1, n), 0xFF)).as_slice()
            assert_close(got, want, what=f"Q4_K {n}x{k} row split {rs} per {per}")
            got = xt.q_mat_mul_add2(q, Tensor.from_slice(dev, a), Tensor.from_slice(dev, b),
                                    out=Tensor.filled_bytes(dev, (1, n), 0xFF)).as_slice()
            assert_close(got, oracle.add3(want, a, b), what=f"add2 Q4_K {n}x{k} row split {rs} per {per}")
    finally:
        dev.set_option("matvec_rowsplit", 0)
        dev.set_option("matvec_per", 0)


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
def test_qmatmul_invariants(dev, oracle, ty):
    """one-hot (tests.rs:951-995), zero input / zero weight -> exact zero (:450-476, :997-1020), batched == unbatched."""
    n, k = 96, 1024
    raw = synth.random_weight(ty, n, k, seed=40 + ty)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    w = oracle.dequantize(ty, raw).reshape(n, k)
    x = np.zeros((1, k), np.float32)
    x[0, 777] = 0.125
    y = Tensor.from_slice(dev, x).q_mat_mul(q).as_slice()
    assert_close(y[0], np.float32(0.125) * w[:, 777], abs_tol=1e-6, rel_tol=1e-6, what="one-hot")
    y = Tensor.from_slice(dev, np.zeros((3, k), np.float32)).q_mat_mul(q).as_slice()
    assert not y.any()
    qz = QMatrix.from_raw_bytes(dev, (n, k), np.zeros_like(raw), ty)
    y = Tensor.from_slice(dev, np.ones((1, k), np.float32)).q_mat_mul(qz).as_slice()
    assert not y.any()
    xs = synth.random_activation(4, k, seed=41)
    yb = Tensor.from_slice(dev, xs).q_mat_mul(q).as_slice()
    for r in range(4):
        yr = Tensor.from_slice(dev, xs[r:r + 1]).q_mat_mul(q).as_slice()
        assert_close(yr, yb[r:r + 1], abs_tol=1e-3, rel_tol=1e-4, what="batched vs unbatched")


def test_q4k_extreme_activations(dev, oracle):
    """Activation magnitudes far outside the f16 range: the MFMA kernel normalises per 256-block."""
    n, k = 64, 1024
    raw = synth.random_weight(Q4_K, n, k, seed=50)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, Q4_K)
    for scale in (1e-20, 1e-6, 1e6, 1e20):
        x = synth.random_activation(1, k, seed=51) * np.float32(scale)
        x[0, 256:512] *= np.float32(1e-4)  # blocks of very different magnitude
        got = Tensor.from_slice(dev, x).q_mat_mul(q).as_slice()
        want = oracle.q_mat_mul(Q4_K, x, raw, n)
        assert_close(got / np.float32(scale), want / np.float32(scale), what=f"activation scale {scale}")


def test_epilogues(dev, oracle):
    """The decode epilogues the reference folds into the matmul dispatch (raw/attention_layer.rs:147-196)."""
    n, k = 256, 1024
    raw_g = synth.random_weight(Q4_K, n, k, seed=60, sigma=2e-3)
    raw_u = synth.random_weight(Q4_K, n, k, seed=61, sigma=2e-3)
    x = synth.random_activation(1, k, seed=62)
    g, u = QMatrix.from_raw_bytes(dev, (n, k), raw_g, Q4_K), QMatrix.from_raw_bytes(dev, (n, k), raw_u, Q4_K)
    gu = QMatrix.concat_rows([g, u])
    assert gu is not None and gu.shape() == (2 * n, k)
    xt = Tensor.from_slice(dev, x)
    want = oracle.swiglu(oracle.q_mat_mul(Q4_K, x, raw_g, n), oracle.q_mat_mul(Q4_K, x, raw_u, n))
    for kern in (1, 0):
        dev.set_option("matvec_kernel", kern)
        got = xt.q_mat_mul_swiglu(gu).as_slice()
        dev.set_option("matvec_kernel", 0)
        assert_close(got, want, what=f"swiglu epilogue kernel={kern}")
    a = synth.random_activation(1, n, seed=63)
    b = synth.random_activation(1, n, seed=64)
    want = oracle.add3(oracle.q_mat_mul(Q4_K, x, raw_g, n), a, b)
    for kern in (1, 0):
        dev.set_option("matvec_kernel", kern)
        got = xt.q_mat_mul_add2(g, Tensor.from_slice(dev, a), Tensor.from_slice(dev, b)).as_slice()
        dev.set_option("matvec_kernel", 0)
        assert_close(got, want, what=f"add2 epilogue kernel={kern}")
    # concat == stacking the raw streams
    got = gu.dequantize().as_slice()
    want = oracle.dequantize(Q4_K, np.concatenate([raw_g, raw_u])).reshape(2 * n, k)
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m", [1, 2, 4])
@pytest.mark.parametrize("n", [48, 272])
def test_epilogues_all_formats_auto_dispatch(dev, oracle, ty, m, n):
    """SwiGLU and add2 through whichever kernel the dispatch picks for 1 .. 4 rows (raw/attention_layer.rs:147-196);
    the stacked gate|up matrix needs halves of whole 16-row tiles; 3 and 17 tiles per half are both odd counts."""
    k = 1280
    raw_g = synth.random_weight(ty, n, k, seed=70 + ty, sigma=2e-3)
    raw_u = synth.random_weight(ty, n, k, seed=71 + ty, sigma=2e-3)
    x = synth.random_activation(m, k, seed=72 + m)
    g, u = QMatrix.from_raw_bytes(dev, (n, k), raw_g, ty), QMatrix.from_raw_bytes(dev, (n, k), raw_u, ty)
    gu = QMatrix.concat_rows([g, u])
    xt = Tensor.from_slice(dev, x)
    a, b = synth.random_activation(m, n, seed=73), synth.random_activation(m, n, seed=74)
    yg, yu = oracle.q_mat_mul(ty, x, raw_g, n), oracle.q_mat_mul(ty, x, raw_u, n)
    out = Tensor.filled_bytes(dev, (m, n), 0xFF)
    got = xt.q_mat_mul_swiglu(gu, out=out).as_slice()
    assert_close(got, oracle.swiglu(yg, yu), what=f"{NAMES[ty]} swiglu m={m} n={n}")
    out = Tensor.filled_bytes(dev, (m, n), 0xFF)
    got = xt.q_mat_mul_add2(g, Tensor.from_slice(dev, a), Tensor.from_slice(dev, b), out=out).as_slice()
    assert_close(got, oracle.add3(yg, a, b), what=f"{NAMES[ty]} add2 m={m} n={n}")


def test_errors_are_status_codes(dev):
    """Programmer errors the reference panics on are FH_ERR_INVALID here (cpu/src/quantized.rs:54-59, :270-274)."""
    raw = synth.random_weight(Q4_K, 16, 256, seed=70)
    with pytest.raises(FusorHipError) as e:
        QMatrix.from_raw_bytes(dev, (16, 250), raw, Q4_K)
    assert e.value.status == -1
    with pytest.raises(FusorHipError) as e:
        QMatrix.from_raw_bytes(dev, (16, 256), raw[:-1], Q4_K)
    assert e.value.status == -1
    with pytest.raises(FusorHipError) as e:
        QMatrix.from_raw_bytes(dev, (16, 256), raw, 10)  # Q2K: GgufReadError::UnsupportedDType
    assert e.value.status == -3
    q = QMatrix.from_raw_bytes(dev, (16, 256), raw, Q4_K)
    with pytest.raises(FusorHipError, match="dimension mismatch"):
        Tensor.from_slice(dev, np.zeros((1, 512), np.float32)).q_mat_mul(q)
    with pytest.raises(FusorHipError):
        q.embed([16])


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
def test_embedding_rows(dev, oracle, ty):
    n, k = 300, 512
    raw = synth.random_weight(ty, n, k, seed=80 + ty)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    ids = [0, 299, 17, 17, 128]
    got = q.embed(ids).as_slice()
    want = oracle.embed_rows(ty, raw, n, k, ids)
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("ty", [Q8_0, Q4_0], ids=lambda t: NAMES[t])
def test_q8_activation_path(dev, oracle, ty):
    """Per-32 activation quantisation + integer vec_dot: block codes and i32 sums bit-exact, f32 result to tolerance."""
    n, k, m = 80, 1024, 3
    raw = synth.random_weight(ty, n, k, seed=90 + ty)
    x = synth.random_activation(m, k, seed=91)
    xt = Tensor.from_slice(dev, x)
    aq = xt.quantize_q8_0().as_slice().reshape(-1)
    assert np.array_equal(aq, oracle.q8_0_quantize(x))
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    y, isums = xt.q_mat_mul_q8(q, want_isums=True)
    if ty == Q8_0:
        want, wsums = oracle.q8_0_matmul_q8(x, raw, n, want_isums=True)
        assert np.array_equal(isums.as_slice(), wsums)
        assert_close(y.as_slice(), want, abs_tol=1e-3, rel_tol=1e-5, what="Q8_0 x Q8")
    else:
        aqb = oracle.q8_0_quantize(x).reshape(m, k // 32, 34)
        wb = raw.reshape(n, k // 32, 18)
        want = np.zeros((m, n), np.float32)
        for r in range(m):
            for c in range(n):
                acc = np.float32(0)
                for b in range(k // 32):
                    acc = np.float32(acc + np.float32(oracle.vec_dot_q4_0_q8_0(wb[c, b], aqb[r, b])))
                want[r, c] = acc
        assert_close(y.as_slice(), want, abs_tol=1e-3, rel_tol=1e-5, what="Q4_0 x Q8")


# ------------------------------------------------------------------ Q5_0, Q5_K, dense f16 / f32 weights
PLAIN = [synth.Q5_0, synth.Q5_K, synth.W_F16, synth.W_F32]


@pytest.mark.parametrize("ty", PLAIN, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("n,k", [(1, 256), (37, 1024), (130, 768)])
def test_plain_types_dequantize_bit_exact(dev, oracle, ty, n, k):
    """GgufBlock::dequantize of BlockQ5_0 / BlockQ5K (gguf/src/lib.rs:1046-1073, :1819-1861) and dense weights."""
    raw = synth.random_weight(ty, n, k, seed=300 + ty)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    assert q.shape() == (n, k) and q.ggml_type == ty
    got = q.dequantize().as_slice()
    want = oracle.dequantize(ty, raw).reshape(n, k)
    assert np.array_equal(bits(got), bits(want))


def test_plain_types_known_answers(dev):
    """core/src/quantized/matmul/tests.rs:1305-1335 (Q5_0: +528 / -528) and :1399-1423 (Q5K: 32896)."""
    blk = lambda hb, lo: np.concatenate([h16(1.0), np.uint8(hb), np.full(16, lo, np.uint8)])
    raw = np.concatenate([blk([0xFF] * 4, 0x11), blk([0] * 4, 0xFF)])
    x = Tensor.from_slice(dev, np.arange(1, 33, dtype=np.float32)[None, :])
    y = x.q_mat_mul(QMatrix.from_raw_bytes(dev, (2, 32), raw, synth.Q5_0)).as_slice()
    assert y.shape == (1, 2) and y[0, 0] == 528.0 and y[0, 1] == -528.0
    raw = np.concatenate([h16(1.0), h16(0.0), np.uint8([1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1]), np.zeros(32, np.uint8),
                          np.full(128, 0x11, np.uint8)])
    x = Tensor.from_slice(dev, np.arange(1, 257, dtype=np.float32)[None, :])
    y = x.q_mat_mul(QMatrix.from_raw_bytes(dev, (1, 256), raw, synth.Q5_K)).as_slice()
    assert y[0, 0] == 32896.0


@pytest.mark.parametrize("ty", [synth.Q5_K, synth.Q5_0], ids=lambda t: NAMES[t])
@pytest.mark.parametrize("n,k", [(72, 1024), (1000, 4096), (96, 14336), (4096, 256), (40, 8192)])
def test_five_bit_formats_single_row_matrix_core_kernel(dev, oracle, ty, n, k):
    """Q5_K and Q5_0 with one activation row go through the single-row matrix-core kernel, which reads the file's own
    block order and adds the fifth bit to the 4-bit code of its Q4_K / Q4_0 form: ragged last tile, 1 .. 56 chunks of
    k, one / two / four row tiles and one / two / four chunks per wavefront, plain, two-residual and SwiGLU epilogues,
    against the checker and against the per-element kernel."""
    raw = synth.random_weight(ty, n, k, seed=330 + ty, sigma=2e-3)
    x = synth.random_activation(1, k, seed=331)
    a, b = synth.random_activation(1, n, seed=332), synth.random_activation(1, n, seed=333)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    want = oracle.q_mat_mul(ty, x, raw, n)
    xt = Tensor.from_slice(dev, x)
    dev.set_option("matvec_kernel", 1)
    slow = xt.q_mat_mul(q).as_slice()
    dev.set_option("matvec_kernel", 0)
    assert_close(slow, want, what="per-element kernel")
    try:
        for tiles, per in ((0, 0), (1, 1), (2, 1), (1, 2), (4, 1), (1, 4), (2, 2)):
            dev.set_option("matvec_tiles", tiles)
            dev.set_option("matvec_per", per)
            got = xt.q_mat_mul(q, out=Tensor.filled_bytes(dev, (1, n), 0xFF)).as_slice()
            assert_close(got, want, what=f"{NAMES[ty]} {n}x{k} tiles={tiles} per={per}")
            assert_close(got, slow, abs_tol=2e-3, rel_tol=1e-4, what=f"{NAMES[ty]} {n}x{k} against the per-element kernel")
            got = xt.q_mat_mul_add2(q, Tensor.from_slice(dev, a), Tensor.from_slice(dev, b),
                                    out=Tensor.filled_bytes(dev, (1, n), 0xFF)).as_slice()
            assert_close(got, oracle.add3(want, a, b), what=f"add2 {NAMES[ty]} {n}x{k} tiles={tiles} per={per}")
            if n % 32 == 0:
                got = xt.q_mat_mul_swiglu(q, out=Tensor.filled_bytes(dev, (1, n // 2), 0xFF)).as_slice()
                assert_close(got, oracle.swiglu(want[:, :n // 2], want[:, n // 2:]),
                             what=f"swiglu {NAMES[ty]} {n}x{k} tiles={tiles} per={per}")
    finally:
        dev.set_option("matvec_tiles", 0)
        dev.set_option("matvec_per", 0)


@pytest.mark.parametrize("ty", PLAIN, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m", [1, 4, 33])
def test_plain_types_matmul_and_glue(dev, oracle, ty, m):
    """q_mat_mul, the SwiGLU / add2 epilogues, concat_rows (any row counts for dense rows, whole 16-row tiles for the
    5-bit formats, which are tiled like the 4-bit ones) and the embedding gather."""
    n, k = (72, 1024) if ty in (synth.W_F32, synth.W_F16) else (80, 1024)
    raw_g = synth.random_weight(ty, n, k, seed=310 + ty, sigma=2e-3)
    raw_u = synth.random_weight(ty, n, k, seed=311 + ty, sigma=2e-3)
    x = synth.random_activation(m, k, seed=312 + m)
    g, u = QMatrix.from_raw_bytes(dev, (n, k), raw_g, ty), QMatrix.from_raw_bytes(dev, (n, k), raw_u, ty)
    xt = Tensor.from_slice(dev, x)
    yg, yu = oracle.q_mat_mul(ty, x, raw_g, n), oracle.q_mat_mul(ty, x, raw_u, n)
    out = Tensor.filled_bytes(dev, (m, n), 0xFF)
    assert_close(xt.q_mat_mul(g, out=out).as_slice(), yg, what=f"{NAMES[ty]} m={m}")
    gu = QMatrix.concat_rows([g, u])
    assert gu.shape() == (2 * n, k)
    assert np.array_equal(bits(gu.dequantize().as_slice()),
                          bits(oracle.dequantize(ty, np.concatenate([raw_g, raw_u])).reshape(2 * n, k)))
    if (2 * n) % 32 == 0:
        assert_close(xt.q_mat_mul_swiglu(gu).as_slice(), oracle.swiglu(yg, yu), what="swiglu")
    a, b = synth.random_activation(m, n, seed=313), synth.random_activation(m, n, seed=314)
    got = xt.q_mat_mul_add2(g, Tensor.from_slice(dev, a), Tensor.from_slice(dev, b)).as_slice()
    assert_close(got, oracle.add3(yg, a, b), what="add2")
    ids = np.array([0, n - 1, 5, 5], np.uint32)
    assert np.array_equal(bits(g.embed(ids).as_slice()), bits(oracle.embed_rows(ty, raw_g, n, k, ids)))
    assert QMatrix.concat_rows([g, QMatrix.from_raw_bytes(dev, (n, k), synth.random_weight(synth.Q4_K, n, k, seed=1),
                                                         synth.Q4_K)]) is None
