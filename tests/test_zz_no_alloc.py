"""The entry point that allocates nothing (fh_flash_attention_decode_static): its partial results live in the library's
file-scope device array instead of a buffer grown with hipMalloc.  Checked through the C ABI against
fh_flash_attention on the same inputs on two calls in a row, the second with a smaller input, so stale contents of
the shared array would show: bit for bit where both run the same kernels with the same cut of the key range (f32
caches, short f16 caches), within the attention tolerance where fh_flash_attention takes its matrix-core kernel
(f16 caches from 4096 keys)."""
import numpy as np
import pytest

from refgen import assert_close
from kalosm_amd.fusor import FusorHipError, Tensor

pytestmark = pytest.mark.gpu


def _case(dev, oracle, hq, hkv, L, dtype, seed):
    rng = np.random.default_rng(seed)
    npdt = np.float16 if dtype == "f16" else np.float32
    q = rng.standard_normal((1, hq, 1, 128)).astype(npdt)
    k = rng.standard_normal((1, hkv, L, 128)).astype(npdt)
    v = rng.standard_normal((1, hkv, L, 128)).astype(npdt)
    qt, kt, vt = (Tensor.from_slice(dev, a, dtype) for a in (q, k, v))
    scale = 1 / np.sqrt(128)
    want = qt.flash_attention(kt, vt, scale).as_slice()
    out = Tensor.filled_bytes(dev, (1, hq, 1, 128), 0xFF, dtype)
    got = qt.flash_attention_decode_static(kt, vt, scale, out=out).as_slice()
    if dtype == "f16" and L >= 4096:
        assert_close(got.astype(np.float32), want.astype(np.float32), abs_tol=1e-2, rel_tol=1e-3,
                     what=f"static vs allocating decode attention hq={hq} L={L} {dtype}")
    else:
        assert np.array_equal(got.view(np.uint16 if dtype == "f16" else np.uint32),
                              want.view(np.uint16 if dtype == "f16" else np.uint32)), f"hq={hq} L={L} {dtype}"
    ref = oracle.flash_attention(*(a.astype(np.float32) for a in (q, k, v)), scale)
    assert_close(got.astype(np.float32), ref, abs_tol=1e-2, rel_tol=1e-3, what=f"static decode attention hq={hq} L={L} {dtype}")


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_static_scratch_attention_matches_the_allocating_entry_point(dev, oracle, dtype):
    _case(dev, oracle, 32, 8, 4096, dtype, 1)      # 16 key parts, two query heads per workgroup
    _case(dev, oracle, 8, 2, 300, dtype, 2)        # smaller: fewer heads, 8 parts, most slots of the array untouched
    _case(dev, oracle, 64, 8, 2049, dtype, 3)      # the most the array holds: 64 heads x 16 parts
    _case(dev, oracle, 4, 4, 1, dtype, 4)          # a single key: parts without keys


def test_static_scratch_limits(dev):
    q = Tensor.zeros(dev, (1, 128, 1, 128))
    kv = Tensor.zeros(dev, (1, 8, 4096, 128))
    with pytest.raises(FusorHipError, match="static scratch"):
        q.flash_attention_decode_static(kv, kv, 0.1)          # 128 heads x 16 parts do not fit
    q = Tensor.zeros(dev, (1, 8, 1, 64))
    kv = Tensor.zeros(dev, (1, 8, 32, 64))
    with pytest.raises(FusorHipError, match="head_dim 128"):
        q.flash_attention_decode_static(kv, kv, 0.1)
