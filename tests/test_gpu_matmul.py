"""GPU parity: the prefill-side quantized matmul (matrix-core tile kernel) against the CPU checker.

Tolerance of the north star for floating point: 1e-3 relative or 1e-2 absolute per element, f32 accumulation.
"""
import numpy as np
import pytest

from refgen import Q4_0, Q4_K, Q6_K, Q8_0, assert_close
from kalosm_amd import synth
from kalosm_amd.fusor import QMatrix, Tensor

pytestmark = pytest.mark.gpu
ALL = [Q4_0, Q8_0, Q4_K, Q6_K]
NAMES = synth.TYPE_NAMES


def bf16_round(x):
    """f32 -> bf16 bits (round to nearest even) and the f32 value those bits stand for."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r, (r.astype(np.uint32) << 16).view(np.float32)


def tile_matmul(dev, x, q, force=2):
    """force = 2: the tile kernels for every m (128 x 128 or 128 x 256 by size); 4: always the pipelined 128 x 256 one."""
    out = Tensor.filled_bytes(dev, (x.shape[0], q.n), 0xFF)  # poisoned: unwritten elements show as NaN
    dev.set_option("matmul_kernel", force)
    try:
        return Tensor.from_slice(dev, x).q_mat_mul(q, out=out).as_slice()
    finally:
        dev.set_option("matmul_kernel", 0)


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m,n,k", [(17, 272, 2048), (33, 130, 1024), (64, 128, 512), (65, 100, 768), (130, 300, 1024),
                                   (256, 256, 256), (3, 37, 512)])
def test_tile_matmul_f32_vs_checker(dev, oracle, ty, m, n, k):
    """Ragged m (tile edges 32 / 64 / 128 / 256), ragged n (not a multiple of 4, 16 or 128), k of 1..8 super-blocks;
    both tile kernels."""
    raw = synth.random_weight(ty, n, k, seed=50 + ty)
    x = synth.random_activation(m, k, seed=60 + m)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    want = oracle.q_mat_mul(ty, x, raw, n, fast=True)
    for force in (2, 4):
        got = tile_matmul(dev, x, q, force)
        assert_close(got, want, what=f"{NAMES[ty]} {n}x{k} m={m} kernel option {force}")


@pytest.mark.parametrize("ty", [synth.Q5_0, synth.Q5_K], ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m,n,k", [(17, 272, 2048), (33, 130, 1024), (65, 100, 768), (130, 300, 1024), (300, 1024, 4096),
                                   (3, 37, 512)])
def test_tile_matmul_five_bit_formats(dev, oracle, ty, m, n, k):
    """Q5_0 and Q5_K through the matrix-core tile kernels (decoded with the exact f32 block arithmetic, then split
    into f16 pairs like the other formats): ragged m and n, the 128 x 128 and the pipelined 128 x 256 kernel, the
    default dispatch (per-element kernel up to 16 rows, tiles above), f32 and bf16 activations."""
    raw = synth.random_weight(ty, n, k, seed=250 + ty, sigma=2e-3)
    x = synth.random_activation(m, k, seed=260 + m)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    want = oracle.q_mat_mul(ty, x, raw, n, fast=True)
    for force in (0, 2, 4):
        got = tile_matmul(dev, x, q, force)
        assert_close(got, want, what=f"{NAMES[ty]} {n}x{k} m={m} kernel option {force}")
    if m > 16:
        bits, xb = bf16_round(x)
        got = Tensor.from_slice(dev, bits, dtype="bf16").q_mat_mul(q, out=Tensor.filled_bytes(dev, (m, n), 0xFF)).as_slice()
        assert_close(got, oracle.q_mat_mul(ty, xb, raw, n, fast=True), what=f"{NAMES[ty]} {n}x{k} m={m} bf16")


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m,n,k", [(200, 384, 4096), (70, 132, 8192), (512, 4096, 2048), (512, 4096, 4096)])
def test_tile_matmul_split_k(dev, oracle, ty, m, n, k):
    """Few output tiles for the device and a long k: the default dispatch splits k over workgroups and sums the
    partial planes in a second launch (on 256 compute units: 64-row tiles four- and eight-fold, 128-row tiles
    two-fold, 256-row tiles four-fold); f32 and bf16 activations.  The sum is in plane order, so two runs agree bit
    for bit.  The large cases are checked on the activation rows around the tile edges."""
    raw = synth.random_weight(ty, n, k, seed=150 + ty)
    x = synth.random_activation(m, k, seed=160 + m)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    rows = np.arange(m) if m * n * k < 2 ** 30 else np.array([0, 63, 64, 127, 128, 255, 256, m - 1])
    got = tile_matmul(dev, x, q, 0)
    assert_close(got[rows], oracle.q_mat_mul(ty, x[rows], raw, n, fast=True), what=f"{NAMES[ty]} {n}x{k} m={m} split k")
    assert np.array_equal(got.view(np.uint32), tile_matmul(dev, x, q, 0).view(np.uint32))
    bits, xb = bf16_round(x)
    out = Tensor.filled_bytes(dev, (m, n), 0xFF)
    gb = Tensor.from_slice(dev, bits, dtype="bf16").q_mat_mul(q, out=out).as_slice()
    assert_close(gb[rows], oracle.q_mat_mul(ty, xb[rows], raw, n, fast=True),
                 what=f"{NAMES[ty]} {n}x{k} m={m} split k, bf16")
    assert not np.isnan(gb).any() and not np.isnan(got).any()


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
def test_tile_matmul_matches_decode_kernels(dev, oracle, ty):
    """The same product through the decode matvec (row by row) and through the tile kernel."""
    n, k, m = 272, 2048, 40
    raw = synth.random_weight(ty, n, k, seed=70 + ty)
    x = synth.random_activation(m, k, seed=71)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    yt = tile_matmul(dev, x, q)
    for r in (0, 17, 39):
        yr = Tensor.from_slice(dev, x[r:r + 1]).q_mat_mul(q).as_slice()
        assert_close(yt[r:r + 1], yr, abs_tol=1e-2, rel_tol=1e-3, what=f"row {r}")


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
def test_tile_matmul_invariants(dev, oracle, ty):
    """One-hot rows pick single weights exactly (tests.rs:951-995); zero rows give exact zeros (:450-476);
    rows of very different magnitude do not disturb each other (each row carries its own scale); linearity."""
    n, k, m = 96, 1024, 48
    raw = synth.random_weight(ty, n, k, seed=80 + ty)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    w = oracle.dequantize(ty, raw).reshape(n, k)
    x = np.zeros((m, k), np.float32)
    cols = (np.arange(m) * 37 + 5) % k
    x[np.arange(m), cols] = 0.125
    x[7] = 0.0
    y = tile_matmul(dev, x, q)
    for r in range(m):
        want = np.zeros(n, np.float32) if r == 7 else np.float32(0.125) * w[:, cols[r]]
        assert_close(y[r], want, abs_tol=1e-6, rel_tol=1e-6, what=f"one-hot row {r}")
    assert not y[7].any()
    xs = synth.random_activation(m, k, seed=81)
    xs[3] *= np.float32(1e20)
    xs[4] *= np.float32(1e-20)
    xs[5, 100] = 3.0e4  # one outlier in a row of N(0,1)
    got = tile_matmul(dev, xs, q)
    want = oracle.q_mat_mul(ty, xs, raw, n, fast=True)
    scale = np.ones((m, 1), np.float32)
    scale[3], scale[4] = 1e-20, 1e20
    assert_close(got * scale, want * scale, what="rows of mixed magnitude")
    y2 = tile_matmul(dev, xs * np.float32(2.0), q)
    assert np.array_equal(y2, got * np.float32(2.0)), "scaling the input by 2 must scale the output exactly"


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m", [1, 20, 130])
def test_tile_matmul_bf16_activations(dev, oracle, ty, m):
    """bf16 activations (the prefill configuration): the checker gets the f32 values of the same bf16 bits."""
    n, k = 272, 1024
    raw = synth.random_weight(ty, n, k, seed=90 + ty)
    xb, xf = bf16_round(synth.random_activation(m, k, seed=91 + m))
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    want = oracle.q_mat_mul(ty, xf, raw, n, fast=True)
    for force in (0, 4):
        dev.set_option("matmul_kernel", force)
        try:
            out = Tensor.filled_bytes(dev, (m, n), 0xFF)
            got = Tensor.from_slice(dev, xb, dtype="bf16").q_mat_mul(q, out=out).as_slice()
        finally:
            dev.set_option("matmul_kernel", 0)
        assert_close(got, want, what=f"bf16 {NAMES[ty]} m={m} kernel option {force}")


@pytest.mark.parametrize("act", ["f32", "bf16"])
@pytest.mark.parametrize("ty", [Q8_0, Q4_0], ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m,n,k", [(256, 128, 256), (300, 200, 96), (300, 200, 192), (129, 1000, 1024), (513, 130, 4096)])
@pytest.mark.parametrize("force", [8, 9])
def test_integer_code_tile_kernel(dev, oracle, ty, act, m, n, k, force):
    """Q8_0 / Q4_0 through the tile kernels that multiply the integer codes and apply the block scale to the
    accumulated block (matmul_kernel = 8 selects them whatever the size; the dispatch takes them for large products):
    64 of k per step for one activation plane (bf16) and k a multiple of 64, 32 of k per step otherwise (f32, k = 96,
    or matmul_kernel = 9); ragged tiles in both directions, odd numbers of steps; against the checker, and one-hot
    activations pick single dequantised weights exactly."""
    raw = synth.random_weight(ty, n, k, seed=m + n + k)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    xa = synth.random_activation(m, k, seed=7)
    if act == "bf16":
        bits = synth.to_bf16_bits(xa)
        xa = (bits.astype(np.uint32) << 16).view(np.float32)
        x = Tensor.from_slice(dev, bits, dtype="bf16")
    else:
        x = Tensor.from_slice(dev, xa)
    want = oracle.q_mat_mul(ty, xa, raw, n)
    dev.set_option("matmul_kernel", force)
    try:
        got = x.q_mat_mul(q).as_slice()
        onehot = np.zeros((m, k), dtype=np.float32)
        cols = (np.arange(m) * 37 + 5) % k
        onehot[np.arange(m), cols] = 0.5
        if act == "bf16":  # 0.5 is a bf16 value: the same kernel as above picks the weights
            picked = Tensor.from_slice(dev, synth.to_bf16_bits(onehot), dtype="bf16").q_mat_mul(q).as_slice()
        else:
            picked = Tensor.from_slice(dev, onehot).q_mat_mul(q).as_slice()
    finally:
        dev.set_option("matmul_kernel", 0)
    assert_close(got, want, abs_tol=1e-2, rel_tol=1e-3, what=f"integer-code tile {NAMES[ty]} {act} {m}x{n}x{k}")
    deq = oracle.dequantize(ty, raw).reshape(n, k)
    assert np.array_equal(picked, 0.5 * deq[:, cols].T), "one-hot activations pick dequantised weights exactly"


@pytest.mark.parametrize("act", ["f32", "bf16"])
@pytest.mark.parametrize("ty,k", [(Q8_0, 4096), (Q8_0, 96), (Q6_K, 14336), (Q4_K, 2304)], ids=lambda t: NAMES.get(t, t))
def test_activation_planes_one_pass_kernel(dev, oracle, ty, k, act):
    """The activation planes of the tile kernels come from a kernel that reads a contiguous row once (k a multiple of 32,
    at most 16384) or from the general two-pass one (matmul_kernel = 12 forces it): the same
    planes, so the same product bit for bit - except Q4_K, whose sub-block sums are added in another order."""
    m, n = 150, 136
    raw = synth.random_weight(ty, n, k, seed=k)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    xa = synth.random_activation(m, k, seed=3)
    xa[7] = 0.0  # a row of zeros: the scale clamps
    xa[9] *= 1e-30
    x = Tensor.from_slice(dev, synth.to_bf16_bits(xa), dtype="bf16") if act == "bf16" else Tensor.from_slice(dev, xa)
    dev.set_option("matmul_kernel", 2)
    try:
        one = x.q_mat_mul(q).as_slice()
        dev.set_option("matmul_kernel", 12)
        two = x.q_mat_mul(q).as_slice()
    finally:
        dev.set_option("matmul_kernel", 0)
    if ty == Q4_K:
        assert np.abs(one - two).max() <= 1e-5 * np.abs(two).max()
    else:
        assert np.array_equal(one, two)


@pytest.mark.parametrize("m,n,k,force", [(256, 128, 256, 8), (300, 200, 512, 8), (129, 1000, 1024, 8), (513, 130, 4096, 8),
                                          (300, 200, 512, 10), (257, 132, 3584, 10), (40, 128, 768, 10)])
def test_q6k_integer_code_tile_kernel(dev, oracle, m, n, k, force):
    """Q6_K with bf16 activations through the tile kernel whose weight operand is two exact integer terms,
    (sc & ~15) (q - 32) and (sc & 15) (q - 32), with the 256-block's d applied to the accumulated block (matmul_kernel =
    8 selects it whatever the size, 10 with k split over two workgroups): ragged tiles, one and several 256-blocks,
    even and odd steps; against the checker, and one-hot activations pick single dequantised weights (d * sc * (q - 32)
    in one rounding where the reference rounds d * sc first)."""
    raw = synth.random_weight(Q6_K, n, k, seed=m + n + k)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, Q6_K)
    bits, xa = bf16_round(synth.random_activation(m, k, seed=7))
    onehot = np.zeros((m, k), dtype=np.float32)
    cols = (np.arange(m) * 37 + 5) % k
    onehot[np.arange(m), cols] = 0.5
    want = oracle.q_mat_mul(Q6_K, xa, raw, n)
    dev.set_option("matmul_kernel", force)
    try:
        got = Tensor.from_slice(dev, bits, dtype="bf16").q_mat_mul(q).as_slice()
        picked = Tensor.from_slice(dev, synth.to_bf16_bits(onehot), dtype="bf16").q_mat_mul(q).as_slice()
    finally:
        dev.set_option("matmul_kernel", 0)
    assert_close(got, want, abs_tol=1e-2, rel_tol=1e-3, what=f"Q6_K integer-code tile {m}x{n}x{k}")
    deq = oracle.dequantize(Q6_K, raw).reshape(n, k)
    assert np.abs(picked - 0.5 * deq[:, cols].T).max() <= 2e-7 * np.abs(deq).max()


@pytest.mark.parametrize("n", [2556, 2555])
@pytest.mark.parametrize("ty,act", [(Q8_0, "bf16"), (Q4_0, "bf16"), (Q8_0, "f32"), (Q6_K, "bf16"), (Q6_K, "f32"), (Q4_K, "bf16"),
                                    (Q4_K, "f32")], ids=lambda t: NAMES.get(t, t) if not isinstance(t, str) else t)
def test_tile_kernels_split_last_round(dev, oracle, ty, act, n):
    """More output tiles than compute units, the remainder at most half of them: the tiles of the last round are two
    workgroups each, one per half of k, summed by a second launch (280 tiles of 256 x 128 on 256 compute units: 24 tiles
    are split; ragged in both directions, n a multiple of four or odd) - in every kernel with 256 x 128 tiles: integer
    codes with 64 and 32 of k per step (Q8_0 / Q4_0), Q6_K on two integer terms (bf16) and on the split form (f32), Q4_K
    on integer codes with one and two activation planes.  Against the checker on sampled columns, and against the same
    product with the split switched off (matmul_kernel = 11), which must agree to the rounding of one addition."""
    m, k = 3333, 512
    raw = synth.random_weight(ty, n, k, seed=77)
    xb, xf = bf16_round(synth.random_activation(m, k, seed=78))
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    x = Tensor.from_slice(dev, xb, dtype="bf16") if act == "bf16" else Tensor.from_slice(dev, xf)
    got = x.q_mat_mul(q).as_slice()
    dev.set_option("matmul_kernel", 11)
    try:
        whole = x.q_mat_mul(q).as_slice()
    finally:
        dev.set_option("matmul_kernel", 0)
    assert np.abs(got - whole).max() <= 1e-5 * np.abs(whole).max()
    rows = (np.arange(96) * 53 + 7) % n
    bpr = len(raw) // n
    sub = np.concatenate([raw[r * bpr:(r + 1) * bpr] for r in rows])
    want = oracle.q_mat_mul(ty, xf, sub, 96, fast=True)
    assert_close(got[:, rows], want, what="sampled columns")
    last = np.arange(n - 40, n)  # the split tiles are the last ones: the last columns of the last rows
    sub = np.concatenate([raw[r * bpr:(r + 1) * bpr] for r in last])
    assert_close(got[-300:, last], oracle.q_mat_mul(ty, xf[-300:], sub, 40, fast=True), what="last tiles")


@pytest.mark.parametrize("act", ["f32", "bf16"])
@pytest.mark.parametrize("m,n,k,force", [(256, 128, 256, 8), (300, 200, 512, 8), (129, 1000, 1024, 8), (513, 130, 4096, 8),
                                          (300, 200, 512, 10), (257, 132, 3584, 10), (40, 128, 768, 10)])
def test_q4k_integer_code_tile_kernel(dev, oracle, act, m, n, k, force):
    """Q4_K through the tile kernel that multiplies the integer codes sc * q, applies the 256-block's d to the
    accumulated block and takes the offsets from one more matrix-core product of the block minimums with the sums of
    the activations per sub-block (matmul_kernel = 8 selects it whatever the size, 10 with k split over two workgroups and
    the planes summed; the dispatch takes it for large products): ragged tiles in both directions, one and several
    256-blocks, odd block counts per k part; against the checker, and one-hot activations pick single dequantised
    weights to the last bits (the scale is applied to sc * q in one rounding instead of two)."""
    raw = synth.random_weight(Q4_K, n, k, seed=m + n + k)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, Q4_K)
    xa = synth.random_activation(m, k, seed=7)
    onehot = np.zeros((m, k), dtype=np.float32)
    cols = (np.arange(m) * 37 + 5) % k
    onehot[np.arange(m), cols] = 0.5
    if act == "bf16":
        bits = synth.to_bf16_bits(xa)
        xa = (bits.astype(np.uint32) << 16).view(np.float32)
        x = Tensor.from_slice(dev, bits, dtype="bf16")
        oh = Tensor.from_slice(dev, synth.to_bf16_bits(onehot), dtype="bf16")
    else:
        x = Tensor.from_slice(dev, xa)
        oh = Tensor.from_slice(dev, onehot)
    want = oracle.q_mat_mul(Q4_K, xa, raw, n)
    dev.set_option("matmul_kernel", force)
    try:
        got = x.q_mat_mul(q).as_slice()
        picked = oh.q_mat_mul(q).as_slice()
    finally:
        dev.set_option("matmul_kernel", 0)
    assert_close(got, want, abs_tol=1e-2, rel_tol=1e-3, what=f"Q4_K integer-code tile {act} {m}x{n}x{k}")
    deq = oracle.dequantize(Q4_K, raw).reshape(n, k)
    assert np.abs(picked - 0.5 * deq[:, cols].T).max() <= 2e-6 * np.abs(deq).max()


@pytest.mark.parametrize("m", [512, 2048])
@pytest.mark.parametrize("ty", [Q6_K, Q8_0, Q4_K], ids=lambda t: NAMES[t])
def test_prefill_shape_spot_check(dev, oracle, ty, m):
    """Full prefill shapes (m = 512 and 2048, k = 4096, n = 14336, bf16 activations): 64 output columns spread over the
    matrix against the checker, and the sum over all outputs of a row against x . (sum of weight rows) -- a checksum
    that every output element enters."""
    k, n = 4096, 14336
    raw = synth.random_weight(ty, n, k, seed=100 + ty)
    xb, xf = bf16_round(synth.random_activation(m, k, seed=101))
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    got = Tensor.from_slice(dev, xb, dtype="bf16").q_mat_mul(q).as_slice()
    assert np.isfinite(got).all()
    rows = (np.arange(64) * 223 + 11) % n
    bpr = len(raw) // n
    sub = np.concatenate([raw[r * bpr:(r + 1) * bpr] for r in rows])
    want = oracle.q_mat_mul(ty, xf, sub, 64, fast=True)
    assert_close(got[:, rows], want, what="sampled columns")
    w = oracle.dequantize(ty, raw).reshape(n, k).astype(np.float64)
    colsum = w.sum(axis=0)
    want_sum = xf.astype(np.float64) @ colsum
    got_sum = got.astype(np.float64).sum(axis=1)
    norm = np.sqrt((xf.astype(np.float64) ** 2).sum(axis=1) * (w ** 2).sum())
    assert np.all(np.abs(got_sum - want_sum) <= 1e-5 * norm)


# ---------------------------------------------------------------------------------------------- batch kernel (m <= 16)
@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m", [1, 3, 4, 7, 16])
@pytest.mark.parametrize("n,k", [(272, 2048), (37, 256), (300, 3328), (64, 14336)])
def test_batch_matvec_vs_checker(dev, oracle, ty, m, n, k):
    """The 16-row matrix-core matvec: k of 1, 8, 13 and 56 chunks (fewer chunks than slices, a last round with idle
    slices, more rounds than chunks in flight); n with a partial last tile and a partial last tile group."""
    raw = synth.random_weight(ty, n, k, seed=120 + ty)
    x = synth.random_activation(m, k, seed=130 + m)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    want = oracle.q_mat_mul(ty, x, raw, n)
    dev.set_option("matvec_kernel", 4)
    try:
        for pre in (1, 2):  # activations converted inside the kernel / once by a launch of its own
            dev.set_option("matvec_per", pre)
            out = Tensor.filled_bytes(dev, (m, n), 0xFF)
            got = Tensor.from_slice(dev, x).q_mat_mul(q, out=out).as_slice()
            assert_close(got, want, what=f"{NAMES[ty]} {n}x{k} m={m} pre={pre}")
    finally:
        dev.set_option("matvec_kernel", 0)
        dev.set_option("matvec_per", 0)


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m", [3, 5, 16])
@pytest.mark.parametrize("n,k", [(272, 2048), (37, 256), (300, 3328), (64, 14336)])
def test_unstaged_batch_matvec_tiles_per_wavefront(dev, oracle, ty, m, n, k):
    """The kernel that reads prepared activation images straight from memory, with one, two and four row tiles per
    wavefront forced (four: Q4_K and Q4_0; the other formats then take one): tile groups that end inside the matrix
    (17, 3, 19 and 4 tiles), k in one part and in four, the two-residual epilogue on the four-tile form."""
    raw = synth.random_weight(ty, n, k, seed=160 + ty)
    x = synth.random_activation(m, k, seed=170 + m)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    want = oracle.q_mat_mul(ty, x, raw, n)
    a, b = synth.random_activation(m, n, seed=171), synth.random_activation(m, n, seed=172)
    xt = Tensor.from_slice(dev, x)
    dev.set_option("matvec_kernel", 4)
    dev.set_option("matvec_direct", 2)  # also for fewer than five rows
    try:
        for tiles in (1, 2, 4):
            dev.set_option("matvec_tiles", tiles)
            got = xt.q_mat_mul(q, out=Tensor.filled_bytes(dev, (m, n), 0xFF)).as_slice()
            assert_close(got, want, what=f"{NAMES[ty]} {n}x{k} m={m} tiles={tiles}")
        got = xt.q_mat_mul_add2(q, Tensor.from_slice(dev, a), Tensor.from_slice(dev, b)).as_slice()
        assert_close(got, oracle.add3(want, a, b), what=f"add2 {NAMES[ty]} {n}x{k} m={m} tiles=4")
    finally:
        for key in ("matvec_kernel", "matvec_direct", "matvec_tiles"):
            dev.set_option(key, 0)


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
def test_batch_matvec_invariants(dev, oracle, ty):
    """One-hot rows pick single weights (tests.rs:951-995), zero rows give exact zeros (:450-476), chunks of very
    different magnitude in one row keep their own scale, ragged n (37 rows: three tiles, the last with 5 rows)."""
    n, k, m = 37, 1024, 6
    raw = synth.random_weight(ty, n, k, seed=140 + ty)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, ty)
    w = oracle.dequantize(ty, raw).reshape(n, k)
    x = np.zeros((m, k), np.float32)
    cols = np.array([0, 255, 256, 700, 1023, 31])
    x[np.arange(m), cols] = 0.125
    x[3] = 0.0
    dev.set_option("matvec_kernel", 4)
    try:
        y = Tensor.from_slice(dev, x).q_mat_mul(q, out=Tensor.filled_bytes(dev, (m, n), 0xFF)).as_slice()
        for r in range(m):
            want = np.zeros(n, np.float32) if r == 3 else np.float32(0.125) * w[:, cols[r]]
            assert_close(y[r], want, abs_tol=1e-6, rel_tol=1e-6, what=f"one-hot row {r}")
        assert not y[3].any()
        xs = synth.random_activation(m, k, seed=141)
        xs[1, :256] *= np.float32(1e12)
        xs[2, 512:768] *= np.float32(1e-12)
        got = Tensor.from_slice(dev, xs).q_mat_mul(q).as_slice()
        want = oracle.q_mat_mul(ty, xs, raw, n)
        scale = np.ones((m, 1), np.float32)
        scale[1] = 1e-12
        assert_close(got * scale, want * scale, what="chunks of mixed magnitude")
    finally:
        dev.set_option("matvec_kernel", 0)


@pytest.mark.parametrize("ty", ALL, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m", [1, 5, 16])
def test_batch_matvec_epilogues(dev, oracle, ty, m):
    """SwiGLU over stacked gate|up rows and the two-residual add (raw/attention_layer.rs:147-196), several rows."""
    n, k = 96, 1024
    raw_g = synth.random_weight(ty, n, k, seed=150 + ty, sigma=2e-3)
    raw_u = synth.random_weight(ty, n, k, seed=151 + ty, sigma=2e-3)
    x = synth.random_activation(m, k, seed=152)
    g, u = QMatrix.from_raw_bytes(dev, (n, k), raw_g, ty), QMatrix.from_raw_bytes(dev, (n, k), raw_u, ty)
    gu = QMatrix.concat_rows([g, u])
    xt = Tensor.from_slice(dev, x)
    a, b = synth.random_activation(m, n, seed=153), synth.random_activation(m, n, seed=154)
    yg, yu = oracle.q_mat_mul(ty, x, raw_g, n), oracle.q_mat_mul(ty, x, raw_u, n)
    dev.set_option("matvec_kernel", 4)
    try:
        got = xt.q_mat_mul_swiglu(gu).as_slice()
        assert_close(got, oracle.swiglu(yg, yu), what=f"swiglu m={m}")
        got = xt.q_mat_mul_add2(g, Tensor.from_slice(dev, a), Tensor.from_slice(dev, b)).as_slice()
        assert_close(got, oracle.add3(yg, a, b), what=f"add2 m={m}")
    finally:
        dev.set_option("matvec_kernel", 0)


# ---------------------------------------------------------------------------------------------- Q8_0 x Q8 on int8 MFMA
@pytest.mark.parametrize("m,n,k", [(3, 80, 1024), (130, 300, 96), (64, 128, 2048), (257, 100, 320)])
def test_q8_activation_matmul_mfma(dev, oracle, m, n, k):
    """Q8_0 weights x per-32 quantised activations on the integer matrix cores: the block sums are exact integers; the
    f32 block terms are added in k order as fma(f32(isum) * d_a, d_w, acc), which differs from the checker's
    acc + f32(isum) * (d_w * d_a) by roundings only (a few f32 ulps of the largest partial sum).  The per-output kernel
    keeps the checker's operation order and its bits.  Shapes with ragged tiles and an odd number of blocks (the device
    record holds two)."""
    raw = synth.random_weight(Q8_0, n, k, seed=200 + m)
    x = synth.random_activation(m, k, seed=201)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, Q8_0)
    got = Tensor.from_slice(dev, x).q_mat_mul_q8(q)
    want = oracle.q8_0_matmul_q8(x, raw, n)
    assert np.abs(got.as_slice() - want).max() <= 4e-6 * np.abs(want).max(), \
        f"max abs diff {np.abs(got.as_slice() - want).max()} against outputs up to {np.abs(want).max()}"
    assert_close(got.as_slice(), want, what="Q8_0 x Q8 on the integer matrix cores")
    dev.set_option("matmul_kernel", 1)  # the per-output kernel gives the checker's bits
    try:
        old = Tensor.from_slice(dev, x).q_mat_mul_q8(q)
    finally:
        dev.set_option("matmul_kernel", 0)
    assert np.array_equal(old.as_slice().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("m", [512, 2048])
def test_q8_activation_matmul_prefill_shape(dev, oracle, m):
    """configs[2], integer variant, full shapes (m = 512 and 2048, k = 4096, n = 14336): 48 sampled weight rows against
    the checker within a few f32 ulps of the largest output (the order of the roundings differs, the integer block sums
    do not), every output finite."""
    k, n = 4096, 14336
    raw = synth.random_weight(Q8_0, n, k, seed=210)
    x = synth.random_activation(m, k, seed=211)
    q = QMatrix.from_raw_bytes(dev, (n, k), raw, Q8_0)
    got = Tensor.from_slice(dev, x).q_mat_mul_q8(q).as_slice()
    assert np.isfinite(got).all()
    rows = (np.arange(48) * 299 + 7) % n
    bpr = len(raw) // n
    sub = np.concatenate([raw[r * bpr:(r + 1) * bpr] for r in rows])
    want = oracle.q8_0_matmul_q8(x, sub, 48)
    assert np.abs(got[:, rows] - want).max() <= 4e-6 * np.abs(want).max()
    assert_close(got[:, rows], want, what="Q8_0 x Q8 at the prefill shape")
