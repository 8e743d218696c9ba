"""Host-side mirror of the `fusor` crate's operator surface for the quantized-inference path,
bound to libfusor_hip.so.  Names and argument meaning follow the reference facade
(fusor-ml/fusor/src: device.rs, quantized.rs, lib.rs, composite/*.rs, cache/*.rs, layers/*.rs) so
tests read like the reference's own.  Every operator runs on the HIP library; nothing here computes
on the host except shape bookkeeping and host<->device copies.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

import numpy as np

from . import _lib
from ._lib import (F16, F32, MASK_ADDITIVE, MASK_CAUSAL, MASK_NONE, Q4_0, Q4_K, Q6_K, Q8_0, FusorHipError, check)

__all__ = ["Device", "Tensor", "QMatrix", "RopeCache", "KvCache", "MaskKind", "GgmlType", "FusorHipError",
           "GpuStandardSamplerParams", "GpuMirostat2SamplerParams", "GpuMirostat2Sampler"]


class GpuStandardSamplerParams:
    """fusor-ml/core/src/sampling/mod.rs:106-114"""

    def __init__(self, top_k: int, temperature: float, repetition_penalty: float, top_p: float, min_p: float,
                 random: float):
        self.top_k, self.temperature, self.repetition_penalty = top_k, temperature, repetition_penalty
        self.top_p, self.min_p, self.random = top_p, min_p, random

    def to_c(self) -> "_lib.SamplerParams":
        return _lib.SamplerParams(0, self.top_k, self.temperature, self.repetition_penalty, self.top_p, self.min_p, 0.0,
                                  0.0, self.random)


class GpuMirostat2SamplerParams:
    """fusor-ml/core/src/sampling/mod.rs:96-104"""

    def __init__(self, top_k: int, temperature: float, repetition_penalty: float, tau: float, eta: float,
                 random: float):
        self.top_k, self.temperature, self.repetition_penalty = top_k, temperature, repetition_penalty
        self.tau, self.eta, self.random = tau, eta, random

    def to_c(self) -> "_lib.SamplerParams":
        return _lib.SamplerParams(1, self.top_k, self.temperature, self.repetition_penalty, 1.0, 0.0, self.tau,
                                  self.eta, self.random)


class GpuMirostat2Sampler:
    """GpuMirostat2Sampler::new(device, mu) (sampling/mod.rs:116-125): the state mu in device memory."""

    def __init__(self, device: "Device", mu: float):
        self.state = Tensor.from_slice(device, np.array([mu], np.float32))

    @property
    def mu(self) -> float:
        return float(self.state.as_slice()[0])


class GgmlType:
    """fusor-ml/gguf/src/lib.rs:35-50"""
    Q4_0, Q8_0, Q4K, Q6K = Q4_0, Q8_0, Q4_K, Q6_K
    BLOCK_ELEMS = {Q4_0: 32, Q8_0: 32, Q4_K: 256, Q6_K: 256}
    BLOCK_BYTES = {Q4_0: 18, Q8_0: 34, Q4_K: 144, Q6_K: 210}


class MaskKind:
    """fusor-ml/fusor/src/composite/flash_attention.rs:12-24"""
    QKMask, Causal, BatchKeyMask = MASK_ADDITIVE, MASK_CAUSAL, 3


_NP = {"f32": np.float32, "f16": np.float16, "bf16": np.uint16, "u32": np.uint32, "i32": np.int32, "u8": np.uint8}


class Device:
    """fusor::Device::Gpu (fusor-ml/fusor/src/device.rs:7-78) on HIP."""

    def __init__(self, ordinal: int = 0):
        self._lib = _lib.load()
        h = C.c_void_p()
        check(self._lib.fh_device_create(ordinal, C.byref(h)))
        self._h = h

    @staticmethod
    def gpu(ordinal: int = 0) -> "Device":
        return Device(ordinal)

    @staticmethod
    def count() -> int:
        n = C.c_int32()
        check(_lib.load().fh_device_count(C.byref(n)))
        return n.value

    def info(self) -> dict:
        name = C.create_string_buffer(256)
        cu, mem = C.c_int32(), C.c_uint64()
        check(self._lib.fh_device_info(self._h, name, 256, C.byref(cu), C.byref(mem)))
        return {"name": name.value.decode(), "compute_units": cu.value, "total_mem": mem.value}

    def sync(self) -> None:
        check(self._lib.fh_device_sync(self._h))

    def set_option(self, key: str, value: int) -> None:
        check(self._lib.fh_set_option(self._h, key.encode(), value))

    def timer_start(self) -> None:
        check(self._lib.fh_timer_start(self._h))

    def timer_stop(self) -> float:
        ms = C.c_float()
        check(self._lib.fh_timer_stop(self._h, C.byref(ms)))
        return ms.value

    # -- record / replay (the reference's lazy graph + single submit)
    def graph_begin(self) -> None:
        check(self._lib.fh_graph_begin(self._h))

    def graph_end(self) -> "Graph":
        h = C.c_void_p()
        check(self._lib.fh_graph_end(self._h, C.byref(h)))
        return Graph(self, h)

    # -- memory
    def alloc(self, nbytes: int) -> int:
        p = C.c_void_p()
        check(self._lib.fh_malloc(self._h, nbytes, C.byref(p)))
        return p.value

    def free(self, ptr: int) -> None:
        check(self._lib.fh_free(self._h, C.c_void_p(ptr)))

    def close(self) -> None:
        if self._h is not None:
            self._lib.fh_device_destroy(self._h)
            self._h = None


class Graph:
    def __init__(self, device: Device, handle):
        self.device, self._h = device, handle

    def launch(self) -> None:
        check(self.device._lib.fh_graph_launch(self._h))

    def __del__(self):
        try:
            if self._h and self.device._h is not None:
                self.device._lib.fh_graph_free(self._h)
        except Exception:
            pass


class Tensor:
    """A contiguous row-major device tensor (fusor::Tensor::Gpu).  dtype in f32/f16/bf16/u32/i32/u8."""

    def __init__(self, device: Device, shape: Sequence[int], dtype: str = "f32", ptr: Optional[int] = None):
        self.device, self.shape, self.dtype = device, tuple(int(s) for s in shape), dtype
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * np.dtype(_NP[dtype]).itemsize
        self._own = ptr is None
        self.ptr = device.alloc(max(self.nbytes, 16)) if ptr is None else ptr

    # Tensor::from_slice / Tensor::new (fusor-ml/fusor/src/lib.rs:356-368)
    @staticmethod
    def from_slice(device: Device, data, dtype: str = "f32") -> "Tensor":
        a = np.ascontiguousarray(data, dtype=_NP[dtype])
        t = Tensor(device, a.shape, dtype)
        if a.nbytes:
            check(device._lib.fh_upload(device._h, C.c_void_p(t.ptr), a.ctypes.data_as(C.c_void_p), a.nbytes))
        return t

    @staticmethod
    def zeros(device: Device, shape, dtype: str = "f32") -> "Tensor":
        t = Tensor(device, shape, dtype)
        check(device._lib.fh_memset(device._h, C.c_void_p(t.ptr), 0, max(t.nbytes, 1)))
        return t

    @staticmethod
    def filled_bytes(device: Device, shape, byte: int, dtype: str = "f32") -> "Tensor":
        """A buffer pre-filled with a byte pattern ("poisoned" outputs, as the reference's dirty buffer pool)."""
        t = Tensor(device, shape, dtype)
        check(device._lib.fh_memset(device._h, C.c_void_p(t.ptr), byte, max(t.nbytes, 1)))
        return t

    def as_slice(self) -> np.ndarray:
        """Blocking read-back (Tensor::as_slice)."""
        out = np.empty(self.shape, _NP[self.dtype])
        if out.nbytes:
            check(self.device._lib.fh_download(self.device._h, out.ctypes.data_as(C.c_void_p), C.c_void_p(self.ptr),
                                               out.nbytes))
        return out

    def reshape(self, shape) -> "Tensor":
        shape = tuple(shape)
        assert int(np.prod(shape)) == int(np.prod(self.shape)), "reshape changes the element count"
        t = Tensor(self.device, shape, self.dtype, ptr=self.ptr)
        t._keep = self
        return t

    def cast(self, dtype: str) -> "Tensor":
        if dtype == self.dtype:
            return self
        out = Tensor(self.device, self.shape, dtype)
        n = int(np.prod(self.shape))
        L, d = self.device._lib, self.device._h
        if (self.dtype, dtype) == ("f32", "f16"):
            check(L.fh_cast_f32_f16(d, C.c_void_p(self.ptr), C.c_void_p(out.ptr), n))
        elif (self.dtype, dtype) == ("f16", "f32"):
            check(L.fh_cast_f16_f32(d, C.c_void_p(self.ptr), C.c_void_p(out.ptr), n))
        elif (self.dtype, dtype) == ("f32", "bf16"):
            check(L.fh_cast_f32_bf16(d, C.c_void_p(self.ptr), C.c_void_p(out.ptr), n))
        else:
            raise FusorHipError(_lib.FH_ERR_UNSUPPORTED, f"cast {self.dtype}->{dtype}")
        return out

    # ---- operators -------------------------------------------------------------------------
    def q_mat_mul(self, w: "QMatrix", out: Optional["Tensor"] = None) -> "Tensor":
        """Tensor::q_mat_mul (fusor-ml/fusor/src/lib.rs:1132-1223); rank 1, 2 or 3 (rank 1 is viewed as [1, k])."""
        k = self.shape[-1]
        if k != w.k:
            raise FusorHipError(_lib.FH_ERR_INVALID,
                                f"Matrix dimension mismatch: lhs columns ({k}) != weight in_features ({w.k})")
        m = int(np.prod(self.shape[:-1])) if len(self.shape) > 1 else 1
        oshape = (*self.shape[:-1], w.n) if len(self.shape) > 1 else (w.n,)
        out = out or Tensor(self.device, oshape, "f32")
        L = self.device._lib
        if self.dtype == "bf16":
            check(L.fh_qmatmul_bf16(w._h, C.c_void_p(self.ptr), m, C.c_void_p(out.ptr)))
        else:
            assert self.dtype == "f32"
            check(L.fh_qmatmul(w._h, C.c_void_p(self.ptr), m, C.c_void_p(out.ptr)))
        return out

    def matmul(self, rhs: "Tensor", rhs_transposed: bool = False, out: Optional["Tensor"] = None) -> "Tensor":
        """Tensor::matmul (fusor-ml/fusor/src/lib.rs:1094-1103): [.., M, K] @ [.., K, N] -> [.., M, N], f32 or f16, batched
        over the leading dimensions (which must match).  With rhs_transposed the right operand is the lazy transpose
        of a contiguous [.., N, K] tensor (the strided view the reference's `transpose` hands to matmul)."""
        if len(self.shape) < 2 or len(rhs.shape) != len(self.shape):
            raise FusorHipError(_lib.FH_ERR_INVALID, "Matrix multiplication requires at least 2 dimensions and equal ranks")
        if self.dtype != rhs.dtype or self.dtype not in ("f32", "f16"):
            raise FusorHipError(_lib.FH_ERR_INVALID, "matmul operands must both be f32 or both f16")
        m, k = self.shape[-2:]
        if rhs_transposed:
            n, k2 = rhs.shape[-2:]
            b_sr, b_sc = 1, k2
        else:
            k2, n = rhs.shape[-2:]
            b_sr, b_sc = n, 1
        if k != k2 or tuple(self.shape[:-2]) != tuple(rhs.shape[:-2]):
            raise FusorHipError(_lib.FH_ERR_INVALID, f"matmul shapes {self.shape} and {rhs.shape} do not agree")
        batch = int(np.prod(self.shape[:-2])) if len(self.shape) > 2 else 1
        if out is None:
            out = Tensor(self.device, (*self.shape[:-2], m, n), self.dtype)
        check(self.device._lib.fh_matmul(self.device._h, F16 if self.dtype == "f16" else F32, C.c_void_p(self.ptr), m * k, k, 1,
                                         C.c_void_p(rhs.ptr), k * n, b_sr, b_sc, batch, m, k, n, C.c_void_p(out.ptr)))
        return out

    def q_mat_mul_add2(self, w: "QMatrix", first: "Tensor", second: "Tensor",
                       out: Optional["Tensor"] = None) -> "Tensor":
        """(x.W^T + first) + second, the decode epilogue of raw/attention_layer.rs:147-174."""
        m = int(np.prod(self.shape[:-1]))
        out = out or Tensor(self.device, (*self.shape[:-1], w.n), "f32")
        check(self.device._lib.fh_qmatmul_add2(w._h, C.c_void_p(self.ptr), m, C.c_void_p(first.ptr),
                                               C.c_void_p(second.ptr), C.c_void_p(out.ptr)))
        return out

    def q_mat_mul_swiglu(self, gate_up: "QMatrix", out: Optional["Tensor"] = None) -> "Tensor":
        """silu(x.Wg^T) * (x.Wu^T) with gate_up = concat_rows(gate, up), raw/attention_layer.rs:186-196."""
        m = int(np.prod(self.shape[:-1]))
        out = out or Tensor(self.device, (*self.shape[:-1], gate_up.n // 2), "f32")
        check(self.device._lib.fh_qmatmul_swiglu(gate_up._h, C.c_void_p(self.ptr), m, C.c_void_p(out.ptr)))
        return out

    def q_mat_mul_q8(self, w: "QMatrix", want_isums: bool = False, out: Optional["Tensor"] = None):
        """The Q8_0 x Q8 integer variant (per-32 activation quantisation + vec_dot)."""
        m = int(np.prod(self.shape[:-1]))
        if out is None:
            out = Tensor(self.device, (*self.shape[:-1], w.n), "f32")
        isums = Tensor(self.device, (m, w.n, w.k // 32), "i32") if want_isums else None
        check(self.device._lib.fh_qmatmul_q8(w._h, C.c_void_p(self.ptr), m, C.c_void_p(out.ptr),
                                             C.c_void_p(isums.ptr) if isums else None))
        return (out, isums) if want_isums else out

    def quantize_q8_0(self) -> "Tensor":
        n = int(np.prod(self.shape))
        out = Tensor(self.device, (n // 32, 34), "u8")
        check(self.device._lib.fh_q8_0_quantize(self.device._h, C.c_void_p(self.ptr), n, C.c_void_p(out.ptr)))
        return out

    def rms_norm_fused(self, weight: "Tensor", bias: Optional["Tensor"], eps: float) -> "Tensor":
        """fusor-ml/fusor/src/composite/normalization.rs:287-326"""
        return self._rms(None, weight, bias, eps)

    def rms_norm_residual_fused(self, residual: "Tensor", weight: "Tensor", bias: Optional["Tensor"],
                                eps: float) -> "Tensor":
        """normalization.rs:356-401"""
        return self._rms(residual, weight, bias, eps)

    def _rms(self, residual, weight, bias, eps):
        cols = self.shape[-1]
        rows = int(np.prod(self.shape[:-1])) if len(self.shape) > 1 else 1
        assert weight.shape == (cols,)
        out = Tensor(self.device, self.shape, "f32")
        check(self.device._lib.fh_rms_norm(self.device._h, C.c_void_p(self.ptr),
                                           C.c_void_p(residual.ptr) if residual else None, C.c_void_p(weight.ptr),
                                           C.c_void_p(bias.ptr) if bias else None, eps, rows, cols,
                                           C.c_void_p(out.ptr)))
        return out

    def flash_attention(self, k: "Tensor", v: "Tensor", scale: float, mask=None,
                        q_strides: Optional[Sequence[int]] = None, out: Optional["Tensor"] = None) -> "Tensor":
        """Tensor<4>::flash_attention(&k, &v, scale, Option<(&mask, MaskKind)>)
        (fusor-ml/fusor/src/composite/flash_attention.rs:58-109).  `mask` is None, MaskKind.Causal, or a
        ([sq, skv] f32 Tensor, MaskKind.QKMask) pair.  q_strides = (batch, head, position) element strides of a
        transposed query view whose logical shape is self.shape (the [b,s,h,d] -> [b,h,s,d] case)."""
        b, hq, sq, d = self.shape
        b2, hkv, skv, d2 = k.shape
        if hq % hkv:
            raise FusorHipError(_lib.FH_ERR_INVALID,
                                f"Number of Q heads ({hq}) must be divisible by number of K/V heads ({hkv})")
        assert (b2, d2) == (b, d) and v.shape == k.shape
        kind, mptr = MASK_NONE, None
        if mask is not None:
            if mask == MaskKind.Causal:
                kind = MASK_CAUSAL
            else:
                mt, kind = mask
                if kind == MASK_ADDITIVE:
                    assert mt.shape == (sq, skv), f"QKMask shape {mt.shape} does not match expected [{sq}, {skv}]"
                    mptr = C.c_void_p(mt.ptr)
                elif kind == MaskKind.BatchKeyMask:
                    assert mt.shape == (b, skv), f"BatchKeyMask shape {mt.shape} does not match expected [{b}, {skv}]"
                    mptr = C.c_void_p(mt.ptr)
        qs = q_strides or (hq * sq * d, sq * d, d)
        qdt = F16 if self.dtype == "f16" else F32
        kdt = F16 if k.dtype == "f16" else F32
        if out is None:
            out = Tensor(self.device, (b, hq, sq, d), self.dtype)
        check(self.device._lib.fh_flash_attention_ex(self.device._h, qdt, kdt, C.c_void_p(self.ptr), qs[0], qs[1], qs[2],
                                                     C.c_void_p(k.ptr), C.c_void_p(v.ptr), hkv * skv * d, skv * d, d, b,
                                                     hq, hkv, sq, skv, d, scale, kind, mptr, C.c_void_p(out.ptr)))
        return out

    def flash_attention_decode_static(self, k: "Tensor", v: "Tensor", scale: float, out: Optional["Tensor"] = None) -> "Tensor":
        """fh_flash_attention_decode_static: one query position per head ([1, hq, 1, 128]) against the cached keys, with
        the partial results in the library's static device array (no allocation at call time; `out` must be given
        for the call to allocate nothing on the Python side either)."""
        b, hq, sq, d = self.shape
        _, hkv, skv, _ = k.shape
        assert b == 1 and sq == 1 and v.shape == k.shape
        if out is None:
            out = Tensor(self.device, (1, hq, 1, d), self.dtype)
        check(self.device._lib.fh_flash_attention_decode_static(
            self.device._h, F16 if self.dtype == "f16" else F32, F16 if k.dtype == "f16" else F32, C.c_void_p(self.ptr),
            C.c_void_p(k.ptr), C.c_void_p(v.ptr), skv * d, d, hq, hkv, d, scale, skv, C.c_void_p(out.ptr)))
        return out

    def silu_mul(self, up: "Tensor") -> "Tensor":
        """silu(self) * up (activations.rs:47-65, raw/attention_layer.rs:195)"""
        out = Tensor(self.device, self.shape, "f32")
        check(self.device._lib.fh_swiglu(self.device._h, C.c_void_p(self.ptr), C.c_void_p(up.ptr), C.c_void_p(out.ptr),
                                         int(np.prod(self.shape))))
        return out

    def add(self, b: "Tensor", c: Optional["Tensor"] = None) -> "Tensor":
        """(self + b) [+ c]"""
        out = Tensor(self.device, self.shape, "f32")
        check(self.device._lib.fh_add3(self.device._h, C.c_void_p(self.ptr), C.c_void_p(b.ptr),
                                       C.c_void_p(c.ptr) if c else None, C.c_void_p(out.ptr), int(np.prod(self.shape))))
        return out

    def transpose_shd(self) -> "Tensor":
        """[s, h, d] -> [h, s, d] materialised (reshape + transpose(1, 2) + to_concrete)."""
        s, h, d = self.shape
        out = Tensor(self.device, (h, s, d), "f32")
        check(self.device._lib.fh_transpose_shd(self.device._h, C.c_void_p(self.ptr), s, h, d, C.c_void_p(out.ptr)))
        return out

    def top_k_pairs(self, k: int):
        """Tensor::top_k_pairs(k) (fusor-ml/fusor/src/lib.rs:416-447): [(token id, logit)] in descending order."""
        if k == 0:
            return []
        ids, vals, found = Tensor(self.device, (k,), "u32"), Tensor(self.device, (k,), "f32"), Tensor(self.device, (1,), "u32")
        check(self.device._lib.fh_top_k(self.device._h, C.c_void_p(self.ptr), int(np.prod(self.shape)), k,
                                        C.c_void_p(ids.ptr), C.c_void_p(vals.ptr), C.c_void_p(found.ptr)))
        n = int(found.as_slice()[0])
        return list(zip(ids.as_slice()[:n].tolist(), vals.as_slice()[:n].tolist()))

    def _sample(self, params, previous_tokens, mu_ptr, previous_gpu_token=None, want_candidates=False):
        prev = np.ascontiguousarray(previous_tokens, np.uint32)
        res = Tensor(self.device, (2,), "u32")
        k = params.top_k
        ids = Tensor(self.device, (k,), "u32") if want_candidates else None
        vals = Tensor(self.device, (k,), "f32") if want_candidates else None
        cp = params.to_c()
        check(self.device._lib.fh_sample_token(
            self.device._h, C.c_void_p(self.ptr), int(np.prod(self.shape)), C.byref(cp),
            prev.ctypes.data_as(C.c_void_p) if prev.size else None, int(prev.size),
            C.c_void_p(previous_gpu_token.ptr) if previous_gpu_token is not None else None,
            C.c_void_p(mu_ptr) if mu_ptr else None, C.c_void_p(res.ptr),
            C.c_void_p(ids.ptr) if ids is not None else None, C.c_void_p(vals.ptr) if vals is not None else None))
        status, token = (int(v) for v in res.as_slice())
        token = token if status == 1 else None
        if want_candidates:
            return token, ids.as_slice(), vals.as_slice()
        return token

    def sample_standard_token(self, previous_tokens, params: "GpuStandardSamplerParams", previous_gpu_token=None,
                              want_candidates=False):
        """Tensor::sample_standard_token (fusor-ml/core/src/sampling/pipeline.rs): the sampled id, or None when no
        logit is finite.  `want_candidates` also returns the processed top-k ids and values in sorted order."""
        return self._sample(params, previous_tokens, None, previous_gpu_token, want_candidates)

    def sample_mirostat2_token(self, sampler: "GpuMirostat2Sampler", previous_tokens,
                               params: "GpuMirostat2SamplerParams", previous_gpu_token=None, want_candidates=False):
        """Tensor::sample_mirostat2_token (fusor-ml/core/src/sampling/pipeline.rs); updates `sampler`'s mu."""
        return self._sample(params, previous_tokens, sampler.state.ptr, previous_gpu_token, want_candidates)

    def check_finite(self) -> dict:
        """debug_check_nan_f32 (models/kalosm-llama/src/raw/mod.rs:9-58): counts of NaN / +inf / -inf, the largest
        finite magnitude and the flat indices of the first (up to four) NaNs of an f32 tensor."""
        assert self.dtype == "f32"
        st = _lib.FiniteStats()
        check(self.device._lib.fh_check_finite(self.device._h, C.c_void_p(self.ptr), int(np.prod(self.shape)),
                                               C.byref(st)))
        return dict(nan=st.nan, pos_inf=st.pos_inf, neg_inf=st.neg_inf, max_abs=st.max_abs,
                    first_nan_indices=list(st.first_nan[:st.first_nan_count]))

    def top_k_pairs_1(self) -> int:
        """Tensor::top_k_pairs(1) (fusor-ml/fusor/src/lib.rs:416-447): the greedy token id, or -1."""
        out = Tensor(self.device, (1,), "u32")
        check(self.device._lib.fh_argmax(self.device._h, C.c_void_p(self.ptr), int(np.prod(self.shape)),
                                         C.c_void_p(out.ptr)))
        v = int(out.as_slice()[0])
        return -1 if v == 0xFFFFFFFF else v

    def __del__(self):
        try:
            if self._own and self.ptr and self.device._h is not None:
                self.device.free(self.ptr)
        except Exception:
            pass


class QMatrix:
    """fusor::QMatrix::Gpu (fusor-ml/fusor/src/quantized.rs:80-279)."""

    def __init__(self, device: Device, handle):
        self.device, self._h = device, handle
        t, n, k, b = C.c_uint32(), C.c_int64(), C.c_int64(), C.c_uint64()
        check(device._lib.fh_qmatrix_info(handle, C.byref(t), C.byref(n), C.byref(k), C.byref(b)))
        self.ggml_type, self.n, self.k, self.device_bytes = t.value, n.value, k.value, b.value

    @staticmethod
    def from_raw_bytes(device: Device, shape: Sequence[int], raw, ty: int) -> "QMatrix":
        n, k = int(shape[0]), int(shape[1])
        a = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        h = C.c_void_p()
        check(device._lib.fh_qmatrix_from_gguf_bytes(device._h, ty, n, k, a.ctypes.data_as(C.c_void_p), a.nbytes,
                                                     C.byref(h)))
        return QMatrix(device, h)

    @staticmethod
    def concat_rows(matrices: Sequence["QMatrix"]) -> Optional["QMatrix"]:
        dev = matrices[0].device
        arr = (C.c_void_p * len(matrices))(*[m._h for m in matrices])
        h = C.c_void_p()
        st = dev._lib.fh_qmatrix_concat_rows(dev._h, arr, len(matrices), C.byref(h))
        if st == _lib.FH_ERR_UNSUPPORTED:
            return None  # the reference returns Option::None when it cannot concatenate
        check(st)
        return QMatrix(dev, h)

    def shape(self):
        return (self.n, self.k)

    def dequantize(self) -> Tensor:
        out = Tensor(self.device, (self.n, self.k), "f32")
        check(self.device._lib.fh_qmatrix_dequantize(self._h, C.c_void_p(out.ptr)))
        return out

    def embed(self, ids) -> Tensor:
        """Embedding::forward (fusor-ml/fusor/src/layers/embedding.rs:43-89)"""
        idh = np.ascontiguousarray(ids, dtype=np.uint32).reshape(-1)
        idt = Tensor.from_slice(self.device, idh, "u32")
        out = Tensor(self.device, (idh.size, self.k), "f32")
        check(self.device._lib.fh_embed_rows(self._h, C.c_void_p(idt.ptr), idh.ctypes.data_as(C.c_void_p), idh.size,
                                             C.c_void_p(out.ptr)))
        return out

    def __del__(self):
        try:
            if self._h and self.device._h is not None:
                self.device._lib.fh_qmatrix_free(self._h)
        except Exception:
            pass


class RopeCache:
    """fusor::RopeCache (fusor-ml/fusor/src/composite/rope.rs:248-329)."""

    def __init__(self, device: Device, cos: Tensor, sin: Tensor):
        self.device, self.cos, self.sin = device, cos, sin

    @staticmethod
    def new(head_dim: int, context_length: int, rope_theta: float, device: Device) -> "RopeCache":
        cos = Tensor(device, (context_length, head_dim // 2), "f32")
        sin = Tensor(device, (context_length, head_dim // 2), "f32")
        check(device._lib.fh_rope_tables(device._h, head_dim, context_length, rope_theta, C.c_void_p(cos.ptr),
                                         C.c_void_p(sin.ptr)))
        return RopeCache(device, cos, sin)

    @staticmethod
    def scaled(head_dim: int, context_length: int, rope_theta: float, device: Device, scaling=None,
               freq_weight=None) -> "RopeCache":
        """RopeImplementation::new (models/kalosm-llama/src/raw/rope.rs:63-85) with create_inverse_frequency's
        options (:9-50): `scaling` = (factor, high_freq_factor, low_freq_factor, original_max_position_embeddings),
        `freq_weight` = the file's rope_freqs.weight values."""
        cos = Tensor(device, (context_length, head_dim // 2), "f32")
        sin = Tensor(device, (context_length, head_dim // 2), "f32")
        sc = None if scaling is None else _lib.RopeScaling(float(scaling[0]), float(scaling[1]), float(scaling[2]),
                                                           int(scaling[3]))
        w = None if freq_weight is None else np.ascontiguousarray(freq_weight, np.float32)
        check(device._lib.fh_rope_tables_scaled(device._h, head_dim, context_length, rope_theta,
                                                None if sc is None else C.byref(sc),
                                                None if w is None else w.ctypes.data_as(C.c_void_p),
                                                C.c_void_p(cos.ptr), C.c_void_p(sin.ptr)))
        return RopeCache(device, cos, sin)

    @staticmethod
    def from_parts(cos: Tensor, sin: Tensor) -> "RopeCache":
        return RopeCache(cos.device, cos, sin)

    def _fwd(self, q: Tensor, k: Tensor, start_pos: int, interleaved: bool, q_strides=None, k_strides=None):
        b, hq, s, d = q.shape
        _, hk, _, _ = k.shape
        qs = q_strides or (hq * s * d, s * d, d)
        ks = k_strides or (hk * s * d, s * d, d)
        qo, ko = Tensor(self.device, q.shape, "f32"), Tensor(self.device, k.shape, "f32")
        check(self.device._lib.fh_rope_pair(self.device._h, C.c_void_p(q.ptr), qs[0], qs[1], qs[2], C.c_void_p(k.ptr),
                                            ks[0], ks[1], ks[2], b, hq, hk, s, d, C.c_void_p(self.cos.ptr),
                                            C.c_void_p(self.sin.ptr), self.cos.shape[0], start_pos, int(interleaved),
                                            C.c_void_p(qo.ptr), C.c_void_p(ko.ptr)))
        return qo, ko

    def forward(self, q, k, start_pos, **kw):
        return self._fwd(q, k, start_pos, False, **kw)

    def forward_interleaved(self, q, k, start_pos, **kw):
        return self._fwd(q, k, start_pos, True, **kw)


class KvCache:
    """fusor::KvCache (fusor-ml/fusor/src/cache/kv_cache.rs:24-63) for `layers` layers at once."""

    def __init__(self, device: Device, layers: int, kv_heads: int, head_dim: int, max_len: int, dtype: str = "f32",
                 sliding_window: bool = False):
        self.device, self.layers, self.kv_heads, self.head_dim, self.dtype = device, layers, kv_heads, head_dim, dtype
        h = C.c_void_p()
        check(device._lib.fh_kvcache_create(device._h, layers, kv_heads, head_dim, max_len, F16 if dtype == "f16" else F32,
                                            C.byref(h)))
        self._h = h
        if sliding_window:  # keep the last max_len positions (tensor_cache.rs:175-202) instead of failing when full
            check(device._lib.fh_kvcache_set_sliding(h, 1))

    def append(self, layer: int, k: Tensor, v: Tensor) -> None:
        """k, v: [kv_heads, s, head_dim] f32 contiguous."""
        hk, s, d = k.shape
        check(self.device._lib.fh_kvcache_append(self._h, layer, C.c_void_p(k.ptr), C.c_void_p(v.ptr), s * d, d, s))

    def view(self, layer: int):
        ln, cap, kp, vp = C.c_int32(), C.c_int32(), C.c_void_p(), C.c_void_p()
        check(self.device._lib.fh_kvcache_view(self._h, layer, C.byref(ln), C.byref(cap), C.byref(kp), C.byref(vp)))
        shape = (self.kv_heads, cap.value, self.head_dim)
        kt = Tensor(self.device, shape, self.dtype, ptr=kp.value) if kp.value else None
        vt = Tensor(self.device, shape, self.dtype, ptr=vp.value) if vp.value else None
        return ln.value, cap.value, kt, vt

    def reset(self) -> None:
        check(self.device._lib.fh_kvcache_reset(self._h))

    def __del__(self):
        try:
            if self._h and self.device._h is not None:
                self.device._lib.fh_kvcache_destroy(self._h)
        except Exception:
            pass
