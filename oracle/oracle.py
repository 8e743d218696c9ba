"""ctypes loader for the CPU checker (``fusor_cpu_oracle.c``).

TEST INFRASTRUCTURE.  Only tests, the smoke check and the benchmark's CPU-baseline
leg import this module; the product package ``kalosm_amd`` never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libfusor_cpu_oracle.so")

Q4_0, Q8_0, Q4_K, Q6_K = 2, 8, 12, 14
BLOCK_ELEMS = {Q4_0: 32, Q8_0: 32, Q4_K: 256, Q6_K: 256, 0: 1, 1: 1, 6: 32, 13: 256}   # 0 f32, 1 f16, 6 Q5_0, 13 Q5_K
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34, Q4_K: 144, Q6_K: 210, 0: 4, 1: 2, 6: 22, 13: 176}


def build(force: bool = False) -> str:
    """Compile the checker with the Makefile beside it."""
    src = os.path.join(_HERE, "fusor_cpu_oracle.c")
    stale = not os.path.exists(_SO) or os.path.getmtime(src) > os.path.getmtime(_SO)
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        fp, u8p, u16p, u32p, i32p = (C.POINTER(C.c_float), C.POINTER(C.c_uint8), C.POINTER(C.c_uint16),
                                     C.POINTER(C.c_uint32), C.POINTER(C.c_int32))
        L.fo_f16_to_f32.restype = C.c_float
        L.fo_f16_to_f32.argtypes = [C.c_uint16]
        L.fo_f32_to_f16.restype = C.c_uint16
        L.fo_f32_to_f16.argtypes = [C.c_float]
        L.fo_f16_to_f32_array.argtypes = [u16p, fp, C.c_size_t]
        L.fo_f32_to_f16_array.argtypes = [fp, u16p, C.c_size_t]
        L.fo_unpack_k4_scales.argtypes = [u8p, u8p, u8p]
        L.fo_dequantize.argtypes = [C.c_int, u8p, C.c_size_t, fp]
        for name in ("fo_q_mat_mul", "fo_q_mat_mul_fast"):
            getattr(L, name).argtypes = [C.c_int, fp, C.c_int, C.c_int, u8p, C.c_int, fp, C.c_int, C.c_int]
        L.fo_q8_0_quantize.argtypes = [fp, C.c_size_t, u8p, C.c_int]
        L.fo_vec_dot_q8_0_q8_0.restype = C.c_float
        L.fo_vec_dot_q8_0_q8_0.argtypes = [u8p, u8p]
        L.fo_vec_dot_q4_0_q8_0.restype = C.c_float
        L.fo_vec_dot_q4_0_q8_0.argtypes = [u8p, u8p]
        L.fo_q8_0_matmul_q8.argtypes = [fp, C.c_int, C.c_int, u8p, C.c_int, fp, i32p, C.c_int]
        L.fo_flash_attention.argtypes = [fp, fp, fp] + [C.c_int] * 6 + [C.c_float, C.c_int, fp, fp, C.c_int]
        L.fo_causal_mask.argtypes = [C.c_int, C.c_int, fp]
        L.fo_rms_norm.argtypes = [fp, fp, fp, fp, C.c_float, C.c_int, C.c_int, fp]
        L.fo_rope_inverse_frequency.argtypes = [C.c_int, C.c_float, fp]
        L.fo_rope_tables.argtypes = [C.c_int, C.c_int, C.c_float, fp, fp]
        L.fo_rope.argtypes = [fp, C.c_int, C.c_int, C.c_int, C.c_int, fp, fp, C.c_int, C.c_int, fp]
        L.fo_silu.argtypes = [fp, fp, C.c_size_t]
        L.fo_swiglu.argtypes = [fp, fp, fp, C.c_size_t]
        L.fo_add3.argtypes = [fp, fp, fp, fp, C.c_size_t]
        L.fo_argmax.restype = C.c_int64
        L.fo_argmax.argtypes = [fp, C.c_size_t]
        L.fo_embed_rows.argtypes = [C.c_int, u8p, C.c_int, C.c_int, u32p, C.c_int, fp]
        L.fo_llama_create.restype = C.c_void_p
        L.fo_llama_create.argtypes = [C.c_void_p, C.c_int]
        L.fo_llama_set_layer.argtypes = [C.c_void_p, C.c_int] + [u8p] * 7 + [fp, fp]
        L.fo_llama_set_globals.argtypes = [C.c_void_p, u8p, fp, u8p]
        L.fo_llama_set_layer_types.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_int)]
        L.fo_llama_set_rope_freq_weight.argtypes = [C.c_void_p, fp]
        L.fo_rope_tables_weighted.argtypes = [C.c_int, C.c_int, C.c_float, fp, fp, fp]
        L.fo_rope_tables_scaled.argtypes = [C.c_int, C.c_int, C.c_float, fp, fp, fp, fp]
        L.fo_llama_reset.argtypes = [C.c_void_p]
        L.fo_llama_destroy.argtypes = [C.c_void_p]
        L.fo_llama_forward.argtypes = [C.c_void_p, u32p, C.c_int, fp, fp]
        _lib = L
    return _lib


def _p(a: np.ndarray, ty):
    return a.ctypes.data_as(C.POINTER(ty))


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    return a.view(np.uint8).reshape(-1)


def default_threads() -> int:
    return max(1, min(os.cpu_count() or 1, 64))


def f16_to_f32(h: np.ndarray) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().fo_f16_to_f32_array(_p(h, C.c_uint16), _p(out, C.c_float), h.size)
    return out


def f32_to_f16(f: np.ndarray) -> np.ndarray:
    f = _f32(f)
    out = np.empty(f.shape, np.uint16)
    lib().fo_f32_to_f16_array(_p(f, C.c_float), _p(out, C.c_uint16), f.size)
    return out


def unpack_k4_scales(p12: np.ndarray):
    p12 = _u8(p12)
    assert p12.size == 12
    sc, mn = np.zeros(8, np.uint8), np.zeros(8, np.uint8)
    lib().fo_unpack_k4_scales(_p(p12, C.c_uint8), _p(sc, C.c_uint8), _p(mn, C.c_uint8))
    return sc, mn


def dequantize(ggml_type: int, raw: np.ndarray) -> np.ndarray:
    raw = _u8(raw)
    bb, e = BLOCK_BYTES[ggml_type], BLOCK_ELEMS[ggml_type]
    assert raw.size % bb == 0
    nb = raw.size // bb
    out = np.empty(nb * e, np.float32)
    rc = lib().fo_dequantize(ggml_type, _p(raw, C.c_uint8), nb, _p(out, C.c_float))
    assert rc == 0
    return out


def q_mat_mul(ggml_type: int, x: np.ndarray, raw: np.ndarray, n: int, lanes: int = 8,
              threads: int | None = None, fast: bool = False) -> np.ndarray:
    """y[m, n] = x[m, k] . dequantize(W[n, k])^T with the reference's lane-wise FMA order."""
    x = _f32(x)
    if x.ndim == 1:
        x = x[None, :]
    m, k = x.shape
    raw = _u8(raw)
    assert raw.size == n * (k // BLOCK_ELEMS[ggml_type]) * BLOCK_BYTES[ggml_type]
    y = np.empty((m, n), np.float32)
    fn = lib().fo_q_mat_mul_fast if fast else lib().fo_q_mat_mul
    rc = fn(ggml_type, _p(x, C.c_float), m, k, _p(raw, C.c_uint8), n, _p(y, C.c_float), lanes,
            threads or default_threads())
    if rc:
        raise ValueError(f"fo_q_mat_mul rc={rc}")
    return y


def q8_0_quantize(x: np.ndarray, round_half_away: bool = False) -> np.ndarray:
    x = _f32(x).reshape(-1)
    assert x.size % 32 == 0
    out = np.empty(x.size // 32 * 34, np.uint8)
    lib().fo_q8_0_quantize(_p(x, C.c_float), x.size // 32, _p(out, C.c_uint8), int(round_half_away))
    return out


def vec_dot_q8_0_q8_0(w34: np.ndarray, a34: np.ndarray) -> float:
    w34, a34 = _u8(w34), _u8(a34)
    return float(lib().fo_vec_dot_q8_0_q8_0(_p(w34, C.c_uint8), _p(a34, C.c_uint8)))


def vec_dot_q4_0_q8_0(w18: np.ndarray, a34: np.ndarray) -> float:
    w18, a34 = _u8(w18), _u8(a34)
    return float(lib().fo_vec_dot_q4_0_q8_0(_p(w18, C.c_uint8), _p(a34, C.c_uint8)))


def q8_0_matmul_q8(x: np.ndarray, raw: np.ndarray, n: int, want_isums: bool = False,
                   round_half_away: bool = False):
    x = _f32(x)
    m, k = x.shape
    raw = _u8(raw)
    y = np.empty((m, n), np.float32)
    isums = np.empty((m, n, k // 32), np.int32) if want_isums else None
    rc = lib().fo_q8_0_matmul_q8(_p(x, C.c_float), m, k, _p(raw, C.c_uint8), n, _p(y, C.c_float),
                                 _p(isums, C.c_int32) if want_isums else None, int(round_half_away))
    assert rc == 0
    return (y, isums) if want_isums else y


MASK_NONE, MASK_CAUSAL, MASK_ADDITIVE = 0, 1, 2


def flash_attention(q, k, v, scale: float, mask_kind: int = MASK_NONE, mask=None,
                    threads: int | None = None) -> np.ndarray:
    q, k, v = _f32(q), _f32(k), _f32(v)
    b, h, sq, d = q.shape
    _, hkv, skv, _ = k.shape
    out = np.empty_like(q)
    mp = None
    if mask is not None:
        mask = _f32(mask)
        assert mask.shape == ((b, skv) if mask_kind == 3 else (sq, skv))
        mp = _p(mask, C.c_float)
    rc = lib().fo_flash_attention(_p(q, C.c_float), _p(k, C.c_float), _p(v, C.c_float), b, h, hkv, sq, skv, d,
                                  scale, mask_kind, mp, _p(out, C.c_float), threads or default_threads())
    if rc:
        raise ValueError(f"fo_flash_attention rc={rc}")
    return out


def flash_attention_f16(q, k, v, scale: float, causal: bool = False) -> np.ndarray:
    """The reference's f16 instantiation of the attention composite: f16 in, f16 out, a rounding to f16 after every
    tensor op (see fo_flash_attention_f16).  Small cases only (one thread)."""
    q, k, v = (np.ascontiguousarray(t, np.float16) for t in (q, k, v))
    b, h, sq, d = q.shape
    _, hkv, skv, _ = k.shape
    out = np.empty_like(q)
    L = lib()
    L.fo_flash_attention_f16.argtypes = [C.c_void_p] * 3 + [C.c_int] * 6 + [C.c_float, C.c_int, C.c_void_p]
    rc = L.fo_flash_attention_f16(q.ctypes.data, k.ctypes.data, v.ctypes.data, b, h, hkv, sq, skv, d, scale,
                                  1 if causal else 0, out.ctypes.data)
    if rc:
        raise ValueError(f"fo_flash_attention_f16 rc={rc}")
    return out


def causal_mask(s: int, p: int = 0) -> np.ndarray:
    m = np.empty((s, p + s), np.float32)
    lib().fo_causal_mask(s, p, _p(m, C.c_float))
    return m


def rms_norm(x, w, eps: float, residual=None, bias=None) -> np.ndarray:
    x = _f32(x)
    cols = x.shape[-1]
    rows = x.size // cols
    w = _f32(w)
    y = np.empty_like(x)
    r = _f32(residual) if residual is not None else None
    bb = _f32(bias) if bias is not None else None
    lib().fo_rms_norm(_p(x, C.c_float), _p(r, C.c_float) if r is not None else None, _p(w, C.c_float),
                      _p(bb, C.c_float) if bb is not None else None, eps, rows, cols, _p(y, C.c_float))
    return y


def rope_inverse_frequency(dim: int, theta: float) -> np.ndarray:
    inv = np.empty(dim // 2, np.float32)
    lib().fo_rope_inverse_frequency(dim, theta, _p(inv, C.c_float))
    return inv


def rope_tables_scaled(dim: int, ctx: int, theta: float, scaling, freq_weight=None):
    """scaling = (factor, high_freq_factor, low_freq_factor, original_max_position_embeddings) or None."""
    cos = np.empty((ctx, dim // 2), np.float32)
    sin = np.empty((ctx, dim // 2), np.float32)
    sc = None if scaling is None else _f32(np.asarray(scaling, np.float32))
    w = None if freq_weight is None else _f32(freq_weight)
    lib().fo_rope_tables_scaled(dim, ctx, theta, None if sc is None else _p(sc, C.c_float),
                                None if w is None else _p(w, C.c_float), _p(cos, C.c_float), _p(sin, C.c_float))
    return cos, sin


def rope_tables_weighted(dim: int, ctx: int, theta: float, freq_weight):
    cos = np.empty((ctx, dim // 2), np.float32)
    sin = np.empty((ctx, dim // 2), np.float32)
    w = _f32(freq_weight)
    lib().fo_rope_tables_weighted(dim, ctx, theta, _p(w, C.c_float), _p(cos, C.c_float), _p(sin, C.c_float))
    return cos, sin


def rope_tables(dim: int, ctx: int, theta: float):
    cos = np.empty((ctx, dim // 2), np.float32)
    sin = np.empty((ctx, dim // 2), np.float32)
    lib().fo_rope_tables(dim, ctx, theta, _p(cos, C.c_float), _p(sin, C.c_float))
    return cos, sin


def rope(x, cos, sin, start_pos: int = 0, interleaved: bool = True) -> np.ndarray:
    x, cos, sin = _f32(x), _f32(cos), _f32(sin)
    b, h, s, d = x.shape
    assert cos.shape[1] == d // 2 and cos.shape[0] >= start_pos + s
    y = np.empty_like(x)
    lib().fo_rope(_p(x, C.c_float), b, h, s, d, _p(cos, C.c_float), _p(sin, C.c_float), start_pos,
                  int(interleaved), _p(y, C.c_float))
    return y


def silu(x) -> np.ndarray:
    x = _f32(x)
    y = np.empty_like(x)
    lib().fo_silu(_p(x, C.c_float), _p(y, C.c_float), x.size)
    return y


def swiglu(gate, up) -> np.ndarray:
    gate, up = _f32(gate), _f32(up)
    y = np.empty_like(gate)
    lib().fo_swiglu(_p(gate, C.c_float), _p(up, C.c_float), _p(y, C.c_float), gate.size)
    return y


def add3(a, b, c) -> np.ndarray:
    a, b, c = _f32(a), _f32(b), _f32(c)
    y = np.empty_like(a)
    lib().fo_add3(_p(a, C.c_float), _p(b, C.c_float), _p(c, C.c_float), _p(y, C.c_float), a.size)
    return y


def top_k(x, k: int):
    """[(id, value)] as Tensor::top_k_pairs(k) returns them."""
    x = _f32(x).reshape(-1)
    ids, vals = np.empty(max(k, 1), np.uint32), np.empty(max(k, 1), np.float32)
    L = lib()
    L.fo_top_k.argtypes = [C.POINTER(C.c_float), C.c_size_t, C.c_int, C.POINTER(C.c_uint32), C.POINTER(C.c_float)]
    n = L.fo_top_k(_p(x, C.c_float), x.size, k, _p(ids, C.c_uint32), _p(vals, C.c_float))
    return list(zip(ids[:n].tolist(), vals[:n].tolist()))


class SamplerParams(C.Structure):
    _fields_ = [("kind", C.c_uint32), ("top_k", C.c_uint32), ("temperature", C.c_float), ("repetition_penalty", C.c_float),
                ("top_p", C.c_float), ("min_p", C.c_float), ("tau", C.c_float), ("eta", C.c_float), ("random", C.c_float)]


def sample_token(logits, kind: int, top_k: int, temperature=1.0, repetition_penalty=1.0, top_p=1.0, min_p=0.0, tau=5.0,
                 eta=0.1, random=0.0, previous=(), mu=None):
    """Device sampler of fusor-ml/core/src/sampling restated: returns a dict with `token` (None when no logit is
    finite), `ids` / `values` (processed top-k, sorted), `mu` (after the update) and `margin` (smallest relative
    gap of a deciding comparison)."""
    x = _f32(logits).reshape(-1)
    prev = np.ascontiguousarray(previous, np.uint32)
    p = SamplerParams(kind, top_k, temperature, repetition_penalty, top_p, min_p, tau, eta, random)
    ids, vals = np.empty(top_k, np.uint32), np.empty(top_k, np.float32)
    res = np.zeros(2, np.uint32)
    mu_c, margin = C.c_float(0.0 if mu is None else mu), C.c_float(1.0)
    L = lib()
    L.fo_sample_token.argtypes = [C.POINTER(C.c_float), C.c_size_t, C.POINTER(SamplerParams), C.POINTER(C.c_uint32),
                                  C.c_uint32, C.POINTER(C.c_float), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32),
                                  C.POINTER(C.c_float), C.POINTER(C.c_float)]
    rc = L.fo_sample_token(_p(x, C.c_float), x.size, C.byref(p), _p(prev, C.c_uint32), prev.size, C.byref(mu_c),
                           _p(res, C.c_uint32), _p(ids, C.c_uint32), _p(vals, C.c_float), C.byref(margin))
    if rc:
        raise ValueError(f"fo_sample_token: {rc}")
    return {"token": int(res[1]) if res[0] == 1 else None, "status": int(res[0]), "ids": ids, "values": vals,
            "mu": mu_c.value, "margin": margin.value}


def argmax(x) -> int:
    x = _f32(x).reshape(-1)
    return int(lib().fo_argmax(_p(x, C.c_float), x.size))


def embed_rows(ggml_type: int, raw: np.ndarray, n: int, k: int, ids) -> np.ndarray:
    raw = _u8(raw)
    ids = np.ascontiguousarray(ids, dtype=np.uint32).reshape(-1)
    out = np.empty((ids.size, k), np.float32)
    rc = lib().fo_embed_rows(ggml_type, _p(raw, C.c_uint8), n, k, _p(ids, C.c_uint32), ids.size, _p(out, C.c_float))
    if rc:
        raise ValueError(f"fo_embed_rows rc={rc}")
    return out


class LlamaConfig(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("n_layers", "d_model", "n_heads", "n_kv_heads", "head_dim", "ffn", "vocab",
                                       "ctx")] + [("eps", C.c_float), ("theta", C.c_float)] + \
               [(n, C.c_int) for n in ("type_attn", "type_ffn_gate_up", "type_ffn_down", "type_embd", "type_output")]


class Llama:
    """The checker's decoder (models/kalosm-llama raw Model restated).  `weights` maps GGUF tensor
    names to numpy arrays (uint8 raw block streams or float32 norm vectors); arrays are kept alive here."""

    def __init__(self, cfg: dict, weights: dict, threads: int | None = None):
        self.cfg = cfg
        c = LlamaConfig(cfg["n_layers"], cfg["d_model"], cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"],
                        cfg["ffn"], cfg["vocab"], cfg["ctx"], cfg["eps"], cfg["theta"], cfg["type_attn"],
                        cfg["type_ffn_gate_up"], cfg["type_ffn_down"], cfg["type_embd"], cfg["type_output"])
        self._keep = []
        self._h = lib().fo_llama_create(C.byref(c), threads or default_threads())

        def u8(name):
            a = _u8(weights[name]); self._keep.append(a); return _p(a, C.c_uint8)

        def f32(name):
            a = _f32(weights[name]); self._keep.append(a); return _p(a, C.c_float)

        for l in range(cfg["n_layers"]):
            p = f"blk.{l}."
            lib().fo_llama_set_layer(self._h, l, u8(p + "attn_q.weight"), u8(p + "attn_k.weight"),
                                     u8(p + "attn_v.weight"), u8(p + "attn_output.weight"),
                                     u8(p + "ffn_gate.weight"), u8(p + "ffn_up.weight"), u8(p + "ffn_down.weight"),
                                     f32(p + "attn_norm.weight"), f32(p + "ffn_norm.weight"))
        lib().fo_llama_set_globals(self._h, u8("token_embd.weight"), f32("output_norm.weight"), u8("output.weight"))
        # per-tensor block types (model files mix them from layer to layer): cfg["tensor_types"] = {name: type}
        types = cfg.get("tensor_types")
        if types:
            names = ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")
            for l in range(cfg["n_layers"]):
                arr = (C.c_int * 7)(*[types[f"blk.{l}.{n}.weight"] for n in names])
                lib().fo_llama_set_layer_types(self._h, l, arr)
        if "rope_freqs.weight" in weights:
            lib().fo_llama_set_rope_freq_weight(self._h, f32("rope_freqs.weight"))
        if cfg.get("rope_scaling") is not None:     # (factor, high_freq_factor, low_freq_factor, original_max_position)
            sc = np.asarray(cfg["rope_scaling"], np.float32)
            self._keep.append(sc)
            L = lib()
            L.fo_llama_set_rope.argtypes = [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float)]
            L.fo_llama_set_rope(self._h, _p(sc, C.c_float),
                                f32("rope_freqs.weight") if "rope_freqs.weight" in weights else None)

    def reset(self):
        lib().fo_llama_reset(self._h)

    def forward(self, tokens, want_hidden: bool = False):
        t = np.ascontiguousarray(tokens, dtype=np.uint32).reshape(-1)
        logits = np.empty(self.cfg["vocab"], np.float32)
        hidden = np.empty(self.cfg["d_model"], np.float32)
        rc = lib().fo_llama_forward(self._h, _p(t, C.c_uint32), t.size, _p(logits, C.c_float), _p(hidden, C.c_float))
        if rc:
            raise ValueError(f"fo_llama_forward rc={rc}")
        return (logits, hidden) if want_hidden else logits

    def __del__(self):
        try:
            lib().fo_llama_destroy(self._h)
        except Exception:
            pass
