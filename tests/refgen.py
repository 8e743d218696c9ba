"""Test support: (1) an independent numpy restatement of the four block decodes, written from the
published ggml layouts (vectorised, shares no code with the C checker), (2) the deterministic byte
generators the reference's own tests use (inputs only; the reference computes expectations at test
time), (3) the tolerance predicate of the reference's conformance suite."""
from __future__ import annotations

import numpy as np

Q4_0, Q8_0, Q4_K, Q6_K = 2, 8, 12, 14
BLOCK_ELEMS = {Q4_0: 32, Q8_0: 32, Q4_K: 256, Q6_K: 256}
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34, Q4_K: 144, Q6_K: 210}


def _f16(b: np.ndarray) -> np.ndarray:
    """[..., 2] little-endian bytes -> f32"""
    return np.ascontiguousarray(b).view(np.float16)[..., 0].astype(np.float32)


def np_dequantize(ty: int, raw: np.ndarray) -> np.ndarray:
    """float32 arithmetic, one rounding per written operation (numpy never fuses)."""
    raw = np.ascontiguousarray(raw, np.uint8).reshape(-1, BLOCK_BYTES[ty])
    nb = raw.shape[0]
    f32 = np.float32
    if ty == Q4_0:
        d = _f16(raw[:, 0:2])[:, None]
        qs = raw[:, 2:18].astype(np.int32)
        lo = (qs & 15) - 8
        hi = (qs >> 4) - 8
        return (np.concatenate([lo, hi], 1).astype(f32) * d).reshape(-1)
    if ty == Q8_0:
        d = _f16(raw[:, 0:2])[:, None]
        return (raw[:, 2:34].view(np.int8).astype(f32) * d).reshape(-1)
    if ty == Q4_K:
        d = _f16(raw[:, 0:2])[:, None]
        dmin = _f16(raw[:, 2:4])[:, None]
        p = raw[:, 4:16].astype(np.int32)
        sc = np.empty((nb, 8), np.int32)
        mn = np.empty((nb, 8), np.int32)
        sc[:, :4] = p[:, 0:4] & 63
        mn[:, :4] = p[:, 4:8] & 63
        sc[:, 4:] = (p[:, 8:12] & 15) | ((p[:, 0:4] >> 6) << 4)
        mn[:, 4:] = (p[:, 8:12] >> 4) | ((p[:, 4:8] >> 6) << 4)
        qs = raw[:, 16:144].astype(np.int32).reshape(nb, 4, 32)
        q = np.stack([qs & 15, qs >> 4], 2).reshape(nb, 8, 32).astype(f32)      # sub-block order 2c, 2c+1
        scale = (sc.astype(f32) * d)[:, :, None]
        off = (mn.astype(f32) * dmin)[:, :, None]
        return (scale * q - off).reshape(-1)
    if ty == Q6_K:
        ql = raw[:, 0:128].astype(np.int32).reshape(nb, 2, 2, 32)   # [half n][first/second 32][l]
        qh = raw[:, 128:192].astype(np.int32).reshape(nb, 2, 32)
        sc = raw[:, 192:208].view(np.int8).astype(f32).reshape(nb, 2, 4, 2)  # [n][jj][l/16]
        d = _f16(raw[:, 208:210])
        out = np.empty((nb, 2, 4, 32), f32)
        for jj in range(4):
            nib = (ql[:, :, jj & 1, :] >> (4 if jj >= 2 else 0)) & 15
            hb = (qh >> (2 * jj)) & 3
            q = ((hb << 4) | nib) - 32
            s = np.repeat(sc[:, :, jj, :], 16, axis=2)              # [nb, 2, 32]
            out[:, :, jj, :] = (d[:, None, None] * s) * q.astype(f32)
        return out.reshape(-1)
    raise ValueError(ty)


def np_matmul_f64(ty: int, x: np.ndarray, raw: np.ndarray, n: int) -> np.ndarray:
    """X . dequantize(W)^T in float64: the reference's own host check (conformance common/quantized.rs:147-157)."""
    k = x.shape[-1]
    w = np_dequantize(ty, raw).reshape(n, k).astype(np.float64)
    return x.astype(np.float64) @ w.T


def approx_or_relative_eq(a: np.ndarray, b: np.ndarray, abs_tol: float = 1e-2, rel_tol: float = 1e-3):
    """conformance/src/comparison.rs:98-110: pass iff |a-b| <= abs_tol OR |a-b| <= rel_tol*max(|a|,|b|).
    Returns (ok, max_abs, max_rel_over_elements_that_fail_abs)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    both_nan = np.isnan(a) & np.isnan(b)
    diff = np.where(both_nan, 0.0, np.abs(a - b))
    scale = np.maximum(np.abs(a), np.abs(b))
    ok = (diff <= abs_tol) | (diff <= rel_tol * scale)
    ok &= ~(np.isnan(diff))
    rel = np.where(scale > 0, diff / np.where(scale > 0, scale, 1), 0.0)
    return bool(ok.all()), float(np.nanmax(diff)) if diff.size else 0.0, float(np.nanmax(rel)) if rel.size else 0.0


def assert_close(got, want, abs_tol=1e-2, rel_tol=1e-3, what=""):
    ok, ma, mr = approx_or_relative_eq(got, want, abs_tol, rel_tol)
    assert ok, f"{what}: max abs err {ma:.3e}, max rel err {mr:.3e} (abs tol {abs_tol}, rel tol {rel_tol})"
    return ma, mr


def assert_greedy_follows(ref, first_token, got, margin=2e-2, what="greedy decode"):
    """The device's greedy tokens against the checker's decoder fed with the SAME tokens: token i must be the checker's
    pick after [first_token, got[0], .., got[i-1]] or have a checker logit within `margin` of its best one.  A greedy
    pick is only defined up to the logit tolerance, and the k-split sums of a decode step are accumulated with float
    atomics whose order varies from run to run, so a near tie may fall either way; feeding the device's own tokens
    keeps every later step checked all the same.  Leaves the checker's cache where the device's is and returns the
    number of steps whose pick was the checker's own."""
    t, same = int(first_token), 0
    for i, g in enumerate(np.asarray(got).tolist()):
        wl = ref.forward([t])
        best = float(np.max(wl))
        assert float(wl[g]) >= best - margin, (f"{what}: step {i} picked {g} (checker logit {float(wl[g]):.5f}) but the "
                                               f"checker's best is {int(np.argmax(wl))} ({best:.5f})")
        same += int(float(wl[g]) == best)
        t = int(g)
    return same


# ----------------------------------------------------------------------------------------------
# The reference's deterministic byte generators (conformance/src/common/quantized.rs:175-272 and
# core/src/quantized/matmul/tests.rs:306-345, :478-489).  Scales are computed in f32, rounded with
# half::f16::from_f32 (RNE) and stored little-endian.
def _h(v) -> bytes:
    return np.float32(v).astype(np.float16).tobytes()


def _nib(lo: int, hi: int) -> int:
    return (lo & 0xF) | ((hi & 0xF) << 4)


def q4_0_raw_bytes(nblocks: int) -> np.ndarray:
    out = bytearray()
    for b in range(nblocks):
        out += _h(np.float32(0.025) + np.float32(b) * np.float32(0.003))
        out += bytes(_nib(10 + ((b + 2 * i) % 6), 9 + ((3 * b + 5 * i) % 7)) for i in range(16))
    return np.frombuffer(bytes(out), np.uint8).copy()


def q8_0_raw_bytes(nblocks: int) -> np.ndarray:
    out = bytearray()
    for b in range(nblocks):
        out += _h(np.float32(0.01) + np.float32(b) * np.float32(0.0015))
        out += bytes((4 + ((7 * b + 5 * i) % 17)) & 0xFF for i in range(32))
    return np.frombuffer(bytes(out), np.uint8).copy()


def q4k_raw_bytes(nblocks: int, patterned: bool = False) -> np.ndarray:
    out = bytearray()
    for b in range(nblocks):
        if patterned:
            out += _h(0.004) + _h(0.0005)
        else:
            out += _h(np.float32(0.004) + np.float32(b) * np.float32(0.0005))
            out += _h(np.float32(0.0005) + np.float32(b) * np.float32(0.0001))
        out += bytes(((5 * b + 3 * i) % 24) + 1 for i in range(12))
        out += bytes(_nib(10 + ((b + 2 * i) % 6), 11 + ((3 * b + i) % 5)) for i in range(128))
    return np.frombuffer(bytes(out), np.uint8).copy()


def q6k_raw_bytes(nblocks: int, patterned: bool = False) -> np.ndarray:
    out = bytearray()
    for b in range(nblocks):
        out += bytes(_nib(5 * b + 3 * i + 1, 7 * b + 11 * i + 2) for i in range(128))
        out += bytes((17 * b + 9 * i + 0x12) & 0xFF for i in range(64))
        out += bytes(((5 * b + 2 * i) % 7 + 1) & 0xFF for i in range(16))
        out += _h(0.0035) if patterned else _h(np.float32(0.0035) + np.float32(b) * np.float32(0.00035))
    return np.frombuffer(bytes(out), np.uint8).copy()


def patterned_q8_0_bytes(nblocks: int) -> np.ndarray:
    out = bytearray()
    for b in range(nblocks):
        out += _h(0.01)
        out += bytes((((5 * b + 3 * i) % 64) - 32) & 0xFF for i in range(32))
    return np.frombuffer(bytes(out), np.uint8).copy()


REF_GENERATORS = {Q4_0: q4_0_raw_bytes, Q8_0: q8_0_raw_bytes, Q4_K: q4k_raw_bytes, Q6_K: q6k_raw_bytes}


def deterministic_input(count: int, seed: int) -> np.ndarray:
    """conformance common/quantized.rs:165-173"""
    i = np.arange(count)
    return ((((i + seed) % 23) - 11) * 0.04).astype(np.float32)


def activation_pattern(count: int, a: int, b: int, mod: int, centre: int, scale: float) -> np.ndarray:
    """core/src/quantized/matmul/tests.rs:558-563 and friends: ((a*i + b) % mod - centre) * scale"""
    i = np.arange(count)
    return (((a * i + b) % mod - centre) * scale).astype(np.float32)


# fixture table of conformance common/quantized.rs:309-335: (type, n, k, rows m)
REF_FIXTURES = [
    (Q4_0, 2, 64, 3), (Q8_0, 96, 64, 1), (Q4_K, 8192, 512, 1), (Q4_K, 4096, 512, 1), (Q4_K, 128, 4608, 1),
    (Q4_K, 128, 4096, 48), (Q4_K, 64, 512, 64), (Q6_K, 8192, 512, 1), (Q6_K, 128, 4608, 1), (Q6_K, 64, 512, 64),
]


# attention inputs of the reference's tests
def attn_pattern(count: int, off: float) -> np.ndarray:
    """conformance flash_attention_ops.rs:20-24: ((i % 17) - 8) * 0.12 + off"""
    i = np.arange(count)
    return (((i % 17) - 8) * 0.12 + off).astype(np.float32)


def attn_sin(count: int, s: float) -> np.ndarray:
    """core/tests/attention.rs:98-100: sin(i * s)"""
    return np.sin(np.arange(count, dtype=np.float32) * np.float32(s)).astype(np.float32)


def np_attention(q, k, v, scale, causal=False, mask=None):
    """Textbook GQA softmax attention in float64 (core/tests/attention.rs:25-81 restated)."""
    q, k, v = (np.asarray(t, np.float64) for t in (q, k, v))
    b, h, sq, d = q.shape
    hkv, skv = k.shape[1], k.shape[2]
    g = h // hkv
    out = np.empty((b, h, sq, d))
    for bi in range(b):
        for hi in range(h):
            s = q[bi, hi] @ k[bi, hi // g].T * scale
            if causal:
                i = np.arange(sq)[:, None]
                j = np.arange(skv)[None, :]
                s = np.where(j > i + (skv - sq), -np.inf, s)
            if mask is not None:
                s = s + mask
            s = s - s.max(axis=1, keepdims=True)
            p = np.exp(s)
            p /= p.sum(axis=1, keepdims=True)
            out[bi, hi] = p @ v[bi, hi // g]
    return out
