"""The matrix-core decode attention (one query position against a long f16 cache, all query heads of a KV head as the
columns of one product): forced for short and ragged caches with the attn_kernel option and checked against the
oracle's flash attention (fusor-ml/fusor/src/composite/flash_attention.rs:58-236) within the attention tolerance."""
import numpy as np
import pytest

from refgen import assert_close
from kalosm_amd.fusor import Tensor

pytestmark = pytest.mark.gpu
SIGNAL_TOL = 5e-3  # largest error over the rms of the outputs (f16 output rounding alone is 5e-4 of a value)


@pytest.fixture
def forced(dev):
    dev.set_option("attn_kernel", 5)
    yield dev
    dev.set_option("attn_kernel", 0)
    dev.set_option("attn_splits", 0)


@pytest.mark.parametrize("hq,hkv,L", [
    (32, 8, 4096),     # the decode shape of the 8B architecture
    (32, 8, 4097),            # one key into a new chunk
    (8, 8, 33),        # one query head per KV head, two chunks, the second with a single key
    (6, 2, 1000),      # three heads per KV head
    (16, 1, 777),      # sixteen heads per KV head: every column of the product in use
    (4, 4, 1),         # a single key: most wavefronts have nothing to do
    (4, 2, 31),        # less than one chunk
])
def test_matrix_core_decode_attention_matches_oracle(forced, oracle, hq, hkv, L):
    rng = np.random.default_rng(hq * 100003 + L)
    q = rng.standard_normal((1, hq, 1, 128)).astype(np.float16)
    k = rng.standard_normal((1, hkv, L, 128)).astype(np.float16)
    v = rng.standard_normal((1, hkv, L, 128)).astype(np.float16)
    scale = 1 / np.sqrt(128)
    ref = oracle.flash_attention(*(a.astype(np.float32) for a in (q, k, v)), scale)
    qt, kt, vt = (Tensor.from_slice(forced, a, "f16") for a in (q, k, v))
    for splits in (0, 1, 3, 128):
        forced.set_option("attn_splits", splits)
        got = qt.flash_attention(kt, vt, scale).as_slice().astype(np.float32)
        assert_close(got, ref, abs_tol=1e-2, rel_tol=1e-3, what=f"decode attention hq={hq} hkv={hkv} L={L} parts={splits}")
        # the tolerance above is loose against outputs that average L values of N(0, 1): hold the error to the signal
        assert np.abs(got - ref).max() <= SIGNAL_TOL * np.sqrt((ref ** 2).mean()), \
            f"hq={hq} hkv={hkv} L={L} parts={splits}: {np.abs(got - ref).max()} against rms {np.sqrt((ref ** 2).mean())}"
    # an f32 query against the f16 cache: the kernel rounds q and the weights P to f16
    forced.set_option("attn_splits", 0)
    got = Tensor.from_slice(forced, q.astype(np.float32)).flash_attention(kt, vt, scale).as_slice().astype(np.float32)
    assert np.abs(got - ref).max() <= SIGNAL_TOL * np.sqrt((ref ** 2).mean())


def test_matrix_core_decode_attention_peaked_scores(forced, oracle):
    """Scores far apart (one key dominates, and it sits in the last chunk): the running maximum has to move late."""
    rng = np.random.default_rng(7)
    hq, hkv, L = 8, 2, 2048 + 5
    q = rng.standard_normal((1, hq, 1, 128)).astype(np.float16)
    k = (0.1 * rng.standard_normal((1, hkv, L, 128))).astype(np.float16)
    k[0, :, L - 2] = (4 * q[0, ::4, 0]).astype(np.float16)
    v = rng.standard_normal((1, hkv, L, 128)).astype(np.float16)
    scale = 1 / np.sqrt(128)
    ref = oracle.flash_attention(*(a.astype(np.float32) for a in (q, k, v)), scale)
    qt, kt, vt = (Tensor.from_slice(forced, a, "f16") for a in (q, k, v))
    got = qt.flash_attention(kt, vt, scale).as_slice().astype(np.float32)
    assert_close(got, ref, abs_tol=1e-2, rel_tol=1e-3, what="peaked decode attention")
