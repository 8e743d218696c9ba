"""Seeded synthetic inputs in GGUF block layout (numpy only; no device work).

The generators follow the input recipes of the benchmark configurations: one f16 super-scale per
block drawn from N(0, sigma), uniformly random quant codes, 6-bit sub-scales / mins packed into the
12-byte K-quant field (the inverse of `unpack_k4_scales_offsets`, fusor-ml/gguf/src/lib.rs:2138-2208).
numpy's `default_rng(seed)` (PCG64) gives identical streams on every host.
"""
from __future__ import annotations

import numpy as np

Q4_0, Q8_0, Q4_K, Q6_K = 2, 8, 12, 14
W_F32, W_F16, Q5_0, Q5_K = 0, 1, 6, 13  # kept in the file's layout by the library (per-element kernels)
BLOCK_ELEMS = {Q4_0: 32, Q8_0: 32, Q4_K: 256, Q6_K: 256, W_F32: 1, W_F16: 1, Q5_0: 32, Q5_K: 256}
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34, Q4_K: 144, Q6_K: 210, W_F32: 4, W_F16: 2, Q5_0: 22, Q5_K: 176}
TYPE_NAMES = {Q4_0: "Q4_0", Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K", W_F32: "F32", W_F16: "F16", Q5_0: "Q5_0",
              Q5_K: "Q5_K"}


def f16_bytes(x: np.ndarray) -> np.ndarray:
    """f32 -> IEEE binary16 (round to nearest even) as little-endian byte pairs [..., 2]."""
    return np.asarray(x, np.float32).astype(np.float16).view(np.uint8).reshape(*np.shape(x), 2)


def pack_k4_scales(sc: np.ndarray, mn: np.ndarray) -> np.ndarray:
    """[..., 8] 6-bit scales and mins -> [..., 12] packed bytes."""
    sc = np.asarray(sc, np.uint8)
    mn = np.asarray(mn, np.uint8)
    out = np.zeros((*sc.shape[:-1], 12), np.uint8)
    out[..., 0:4] = (sc[..., 0:4] & 63) | ((sc[..., 4:8] >> 4) << 6)
    out[..., 4:8] = (mn[..., 0:4] & 63) | ((mn[..., 4:8] >> 4) << 6)
    out[..., 8:12] = (sc[..., 4:8] & 0x0F) | ((mn[..., 4:8] & 0x0F) << 4)
    return out


def random_blocks(ggml_type: int, nblocks: int, rng: np.random.Generator, sigma: float = 0.02) -> np.ndarray:
    """`nblocks` random blocks of the given type as a flat uint8 array."""
    bb = BLOCK_BYTES[ggml_type]
    out = np.empty((nblocks, bb), np.uint8)
    if ggml_type == Q4_0:
        out[:, 0:2] = f16_bytes(rng.normal(0.0, sigma, nblocks))
        out[:, 2:18] = rng.integers(0, 256, (nblocks, 16), dtype=np.uint8)
    elif ggml_type == Q8_0:
        out[:, 0:2] = f16_bytes(rng.normal(0.0, sigma, nblocks))
        out[:, 2:34] = rng.integers(-127, 128, (nblocks, 32), dtype=np.int8).view(np.uint8)
    elif ggml_type == Q4_K:
        out[:, 0:2] = f16_bytes(rng.normal(0.0, sigma, nblocks))
        out[:, 2:4] = f16_bytes(rng.normal(0.0, sigma, nblocks))
        sc = rng.integers(0, 64, (nblocks, 8), dtype=np.uint8)
        mn = rng.integers(0, 64, (nblocks, 8), dtype=np.uint8)
        out[:, 4:16] = pack_k4_scales(sc, mn)
        out[:, 16:144] = rng.integers(0, 256, (nblocks, 128), dtype=np.uint8)
    elif ggml_type == Q6_K:
        out[:, 0:192] = rng.integers(0, 256, (nblocks, 192), dtype=np.uint8)
        out[:, 192:208] = rng.integers(-128, 128, (nblocks, 16), dtype=np.int8).view(np.uint8)
        out[:, 208:210] = f16_bytes(rng.normal(0.0, sigma, nblocks))
    elif ggml_type == Q5_0:
        out[:, 0:2] = f16_bytes(rng.normal(0.0, sigma, nblocks))
        out[:, 2:22] = rng.integers(0, 256, (nblocks, 20), dtype=np.uint8)
    elif ggml_type == Q5_K:
        out[:, 0:2] = f16_bytes(rng.normal(0.0, sigma, nblocks))
        out[:, 2:4] = f16_bytes(rng.normal(0.0, sigma, nblocks))
        sc = rng.integers(0, 64, (nblocks, 8), dtype=np.uint8)
        mn = rng.integers(0, 64, (nblocks, 8), dtype=np.uint8)
        out[:, 4:16] = pack_k4_scales(sc, mn)
        out[:, 16:176] = rng.integers(0, 256, (nblocks, 160), dtype=np.uint8)
    elif ggml_type == W_F16:
        out[:, 0:2] = f16_bytes(rng.normal(0.0, sigma * 100.0, nblocks))
    elif ggml_type == W_F32:
        out[:] = rng.normal(0.0, sigma * 100.0, nblocks).astype(np.float32).view(np.uint8).reshape(nblocks, 4)
    else:
        raise ValueError(f"unsupported type {ggml_type}")
    return out.reshape(-1)


def random_weight(ggml_type: int, n: int, k: int, seed: int, sigma: float = 0.02) -> np.ndarray:
    """Raw GGUF byte stream of a random [n, k] weight (blocks contiguous along k)."""
    assert k % BLOCK_ELEMS[ggml_type] == 0
    rng = np.random.default_rng(seed)
    return random_blocks(ggml_type, n * (k // BLOCK_ELEMS[ggml_type]), rng, sigma)


def random_activation(m: int, k: int, seed: int, dtype=np.float32) -> np.ndarray:
    return np.random.default_rng(seed).standard_normal((m, k)).astype(dtype)


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """f32 -> bf16 bit patterns (round to nearest even)."""
    u = np.asarray(x, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def matvec_bytes(ggml_type: int, n: int, k: int, m: int) -> int:
    """Algorithmic bytes of one y[m,n] = x[m,k].W[n,k]^T call: weight stream + f32 activations in and out."""
    return n * (k // BLOCK_ELEMS[ggml_type]) * BLOCK_BYTES[ggml_type] + 4 * m * k + 4 * m * n


# ---------------------------------------------------------------------------------------------
# Llama-3-8B-architecture decoder with random-init Q4_K_M weights (Q4_K everywhere, Q6_K for
# ffn_down and output; models/kalosm-llama/src/raw/mod.rs:473-604 names the tensors).
LLAMA3_8B = dict(n_layers=32, d_model=4096, n_heads=32, n_kv_heads=8, head_dim=128, ffn=14336, vocab=128256,
                 ctx=8192, eps=1e-5, theta=500000.0)


def llama_tensor_specs(cfg: dict):
    """[(name, ggml_type or 0 for f32, n, k)] in load order."""
    D, QD, KD, F, V = cfg["d_model"], cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"], cfg["ffn"], \
        cfg["vocab"]
    ta, tg, td = cfg.get("type_attn", Q4_K), cfg.get("type_ffn_gate_up", Q4_K), cfg.get("type_ffn_down", Q6_K)
    specs = [("token_embd.weight", cfg.get("type_embd", Q4_K), V, D), ("output_norm.weight", 0, D, 0),
             ("output.weight", cfg.get("type_output", Q6_K), V, D)]
    for l in range(cfg["n_layers"]):
        p = f"blk.{l}."
        specs += [(p + "attn_norm.weight", 0, D, 0), (p + "attn_q.weight", ta, QD, D), (p + "attn_k.weight", ta, KD, D),
                  (p + "attn_v.weight", ta, KD, D), (p + "attn_output.weight", ta, D, QD),
                  (p + "ffn_norm.weight", 0, D, 0), (p + "ffn_gate.weight", tg, F, D), (p + "ffn_up.weight", tg, F, D),
                  (p + "ffn_down.weight", td, D, F)]
    return specs


def llama_random_tensor(name: str, ty: int, n: int, k: int, seed: int, sigma: float) -> np.ndarray:
    """Deterministic per-tensor content: the seed is mixed with a hash of the tensor name."""
    h = np.uint64(1469598103934665603)
    for ch in name.encode():
        h = np.uint64((int(h) ^ ch) * 1099511628211 % (1 << 64))
    s = (int(h) ^ (seed * 0x9E3779B97F4A7C15)) % (1 << 63)
    if ty == 0:
        return (1.0 + 0.1 * np.random.default_rng(s).standard_normal(n)).astype(np.float32)
    return random_weight(ty, n, k, s, sigma)
