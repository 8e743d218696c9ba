"""Host-side handle of the Llama-architecture decoder (models/kalosm-llama/src/raw/mod.rs `Model`),
bound to the fh_llama_* entry points of libfusor_hip.so."""
from __future__ import annotations

import ctypes as C
from typing import Callable, Iterable, Optional, Tuple

import numpy as np

from . import _lib, synth
from ._lib import F16, F32, LlamaConfig, check
from .fusor import Device


class Model:
    def __init__(self, device: Device, cfg: dict, kv_dtype: str = "f32", fuse_qkv: bool = True,
                 fuse_gate_up: bool = True, use_graph: bool = True):
        self.device, self.cfg = device, dict(cfg)
        c = LlamaConfig(cfg["n_layers"], cfg["d_model"], cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["ffn"],
                        cfg["vocab"], cfg["ctx"], cfg["eps"], cfg["theta"], F16 if kv_dtype == "f16" else F32,
                        int(fuse_qkv), int(fuse_gate_up), int(use_graph))
        h = C.c_void_p()
        check(device._lib.fh_llama_create(device._h, C.byref(c), C.byref(h)))
        self._h = h
        self._final = False

    def load_tensor(self, name: str, ggml_type: int, n: int, k: int, data: np.ndarray) -> None:
        a = np.ascontiguousarray(data)
        a = a.view(np.uint8).reshape(-1)
        check(self.device._lib.fh_llama_load_tensor(self._h, name.encode(), ggml_type, n, k,
                                                    a.ctypes.data_as(C.c_void_p), a.nbytes))

    def load_all(self, tensors: Iterable[Tuple[str, int, int, int, np.ndarray]]) -> None:
        for name, ty, n, k, data in tensors:
            self.load_tensor(name, ty, n, k, data)
        self.finalize()

    @staticmethod
    def random_init(device: Device, cfg: dict, seed: int = 0, sigma: float = 1e-4,
                    keep: Optional[Callable[[str, np.ndarray], None]] = None, **kw) -> "Model":
        """Random-init weights in GGUF block layout, generated tensor by tensor (so an 8B model never
        sits on the host in full).  `keep(name, array)` receives each tensor for a checker to hold."""
        m = Model(device, cfg, **kw)
        for name, ty, n, k in synth.llama_tensor_specs(cfg):
            data = synth.llama_random_tensor(name, ty, n, k, seed, sigma)
            m.load_tensor(name, ty, n, k, data)
            if keep is not None:
                keep(name, data)
        m.finalize()
        return m

    @staticmethod
    def from_gguf(device: Device, source, ctx: Optional[int] = None, kv_dtype: str = "f32", fuse_qkv: bool = True,
                  fuse_gate_up: bool = True, use_graph: bool = True, rope_scaling=None) -> "Model":
        """Model::from_gguf for the Llama architecture (raw/mod.rs:284-648): parameters from the metadata, every
        decoder tensor from the file.  `source` is a path or an open `GgufMetadata`; `ctx` caps the context
        length (and with it the KV cache) below the file's `context_length`; `rope_scaling` is the reference's
        argument of that name: (factor, high_freq_factor, low_freq_factor, original_max_position_embeddings)."""
        from .gguf import GgufMetadata
        g = source if isinstance(source, GgufMetadata) else GgufMetadata.read(source)
        c = LlamaConfig()
        check(device._lib.fh_llama_config_from_gguf(g._h, C.byref(c)))
        cfg = {n: getattr(c, n) for n in ("n_layers", "d_model", "n_heads", "n_kv_heads", "head_dim", "ffn", "vocab",
                                          "ctx", "eps", "theta")}
        if ctx is not None:
            cfg["ctx"] = min(cfg["ctx"], int(ctx))
        m = Model(device, cfg, kv_dtype=kv_dtype, fuse_qkv=fuse_qkv, fuse_gate_up=fuse_gate_up, use_graph=use_graph)
        check(device._lib.fh_llama_load_gguf(m._h, g._h))
        if rope_scaling is not None:
            m.set_rope_scaling(*rope_scaling)
        m.finalize()
        return m

    def set_rope_scaling(self, factor: float, high_freq_factor: float, low_freq_factor: float,
                         original_max_position_embeddings: int) -> None:
        """RopeScalingConfig (raw/mod.rs:163-169); before `finalize`."""
        sc = _lib.RopeScaling(factor, high_freq_factor, low_freq_factor, original_max_position_embeddings)
        check(self.device._lib.fh_llama_set_rope_scaling(self._h, C.byref(sc)))

    def finalize(self) -> None:
        check(self.device._lib.fh_llama_finalize(self._h))
        self._final = True

    def reset(self) -> None:
        check(self.device._lib.fh_llama_reset(self._h))

    def forward(self, tokens, want_hidden: bool = False):
        """Model::forward: logits of the last of `tokens` (raw/mod.rs:851-865)."""
        t = np.ascontiguousarray(tokens, dtype=np.uint32).reshape(-1)
        logits = np.empty(self.cfg["vocab"], np.float32)
        hidden = np.empty(self.cfg["d_model"], np.float32)
        check(self.device._lib.fh_llama_forward(self._h, t.ctypes.data_as(C.c_void_p), t.size,
                                                logits.ctypes.data_as(C.c_void_p), hidden.ctypes.data_as(C.c_void_p)))
        return (logits, hidden) if want_hidden else logits

    def decode_greedy(self, first_token: int, steps: int):
        """Greedy decode of `steps` tokens on the device; returns (token ids, device milliseconds)."""
        out = np.empty(steps, np.uint32)
        ms = C.c_float()
        check(self.device._lib.fh_llama_decode_greedy(self._h, int(first_token), steps, out.ctypes.data_as(C.c_void_p),
                                                      C.byref(ms)))
        return out, ms.value

    def decode_sampled(self, first_token: int, steps: int, params, randoms, previous_tokens=(), repetition_range: int = 64,
                       mu: Optional[float] = None):
        """Sampled decode of `steps` tokens with the token resident on the device (models/kalosm-llama/src/model/
        inference.rs:38-173).  `params`: GpuStandardSamplerParams or GpuMirostat2SamplerParams (its `random` is
        replaced by `randoms[step]`).  Returns (token ids, device milliseconds, mu after the last step)."""
        out = np.empty(steps, np.uint32)
        rnd = np.ascontiguousarray(randoms, np.float32)
        assert rnd.size >= steps
        prev = np.ascontiguousarray(previous_tokens, np.uint32)
        ms, mu_c = C.c_float(), C.c_float(0.0 if mu is None else mu)
        cp = params.to_c()
        check(self.device._lib.fh_llama_decode_sampled(
            self._h, int(first_token), steps, C.byref(cp), rnd.ctypes.data_as(C.c_void_p),
            prev.ctypes.data_as(C.c_void_p) if prev.size else None, int(prev.size), int(repetition_range),
            C.byref(mu_c), out.ctypes.data_as(C.c_void_p), C.byref(ms)))
        return out, ms.value, mu_c.value

    def trace_text(self) -> str:
        """Lines traced by the last `forward` (device options trace_nan / trace_timing, or the reference's
        KALOSM_TRACE_LAYER_NAN / KALOSM_TRACE_FORWARD_TIMING / FUSOR_TRACE_GPU_KERNELS in the environment)."""
        n = C.c_size_t()
        check(self.device._lib.fh_llama_trace_text(self._h, None, 0, C.byref(n)))
        buf = C.create_string_buffer(n.value + 1)
        check(self.device._lib.fh_llama_trace_text(self._h, buf, n.value + 1, None))
        return buf.value.decode()

    def weight_bytes(self) -> int:
        b = C.c_uint64()
        check(self.device._lib.fh_llama_weight_bytes(self._h, C.byref(b)))
        return b.value

    def __del__(self):
        try:
            if self._h and self.device._h is not None:
                self.device._lib.fh_llama_destroy(self._h)
        except Exception:
            pass
