"""ctypes binding of libfusor_hip.so (declared in include/fusor_hip.h).

The library is the product: there is no CPU or PyTorch fallback.  Loading fails loudly when the
shared object has not been built (`python -m kalosm_amd.build`)."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libfusor_hip.so")

FH_OK, FH_ERR_INVALID, FH_ERR_HIP, FH_ERR_UNSUPPORTED, FH_ERR_OOM, FH_ERR_NO_DEVICE = 0, -1, -2, -3, -4, -5
FH_ERR_IO, FH_ERR_NOT_FOUND = -6, -7
Q4_0, Q8_0, Q4_K, Q6_K = 2, 8, 12, 14
MASK_NONE, MASK_CAUSAL, MASK_ADDITIVE = 0, 1, 2
F32, F16 = 0, 1


class FusorHipError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"fusor-hip error {status}: {message}")
        self.status = status


class LlamaConfig(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "d_model", "n_heads", "n_kv_heads", "head_dim", "ffn", "vocab",
                                         "ctx")] + [("eps", C.c_float), ("theta", C.c_float)] + \
               [(n, C.c_int32) for n in ("kv_dtype", "fuse_qkv", "fuse_gate_up", "use_graph")]


class FiniteStats(C.Structure):
    _fields_ = [("nan", C.c_uint64), ("pos_inf", C.c_uint64), ("neg_inf", C.c_uint64), ("max_abs", C.c_float),
                ("first_nan_count", C.c_uint32), ("first_nan", C.c_uint64 * 4)]


class RopeScaling(C.Structure):
    _fields_ = [("factor", C.c_float), ("high_freq_factor", C.c_float), ("low_freq_factor", C.c_float),
                ("original_max_position_embeddings", C.c_int32)]


class SamplerParams(C.Structure):
    _fields_ = [("kind", C.c_uint32), ("top_k", C.c_uint32), ("temperature", C.c_float), ("repetition_penalty", C.c_float),
                ("top_p", C.c_float), ("min_p", C.c_float), ("tau", C.c_float), ("eta", C.c_float), ("random", C.c_float)]


class GgufTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("ggml_type", C.c_uint32), ("rank", C.c_int32), ("shape", C.c_int64 * 8),
                ("offset", C.c_uint64)]


_p = C.c_void_p
_i32, _i64, _u32, _u64, _f32, _sz = C.c_int32, C.c_int64, C.c_uint32, C.c_uint64, C.c_float, C.c_size_t
_pp = C.POINTER(C.c_void_p)

# name -> argtypes; every function returns fh_status except the two string getters.
SIGNATURES = {
    "fh_device_count": [C.POINTER(_i32)],
    "fh_device_create": [_i32, _pp],
    "fh_device_destroy": [_p],
    "fh_device_sync": [_p],
    "fh_device_info": [_p, C.c_char_p, _sz, C.POINTER(_i32), C.POINTER(_u64)],
    "fh_malloc": [_p, _sz, _pp],
    "fh_free": [_p, _p],
    "fh_memset": [_p, _p, _i32, _sz],
    "fh_upload": [_p, _p, _p, _sz],
    "fh_download": [_p, _p, _p, _sz],
    "fh_copy": [_p, _p, _p, _sz],
    "fh_timer_start": [_p],
    "fh_timer_stop": [_p, C.POINTER(_f32)],
    "fh_probe_empty": [_p, _i32, _i32],
    "fh_probe_read": [_p, _p, C.c_size_t],
    "fh_probe_device": [_p, _i32, _i32, _i32, _p, _sz, C.POINTER(C.c_double)],
    "fh_check_finite": [_p, _p, _i64, C.POINTER(FiniteStats)],
    "fh_graph_begin": [_p],
    "fh_graph_end": [_p, _pp],
    "fh_graph_launch": [_p],
    "fh_graph_free": [_p],
    "fh_qmatrix_from_gguf_bytes": [_p, _u32, _i64, _i64, _p, _sz, _pp],
    "fh_qmatrix_concat_rows": [_p, _pp, _i32, _pp],
    "fh_qmatrix_free": [_p],
    "fh_qmatrix_info": [_p, C.POINTER(_u32), C.POINTER(_i64), C.POINTER(_i64), C.POINTER(_u64)],
    "fh_qmatrix_dequantize": [_p, _p],
    "fh_embed_rows": [_p, _p, _p, _i32, _p],
    "fh_qmatmul": [_p, _p, _i32, _p],
    "fh_qmatmul_add2": [_p, _p, _i32, _p, _p, _p],
    "fh_qmatmul_swiglu": [_p, _p, _i32, _p],
    "fh_qmatmul_bf16": [_p, _p, _i32, _p],
    "fh_qmatmul_q8": [_p, _p, _i32, _p, _p],
    "fh_q8_0_quantize": [_p, _p, _i64, _p],
    "fh_set_option": [_p, C.c_char_p, _i64],
    "fh_rms_norm": [_p, _p, _p, _p, _p, _f32, _i32, _i32, _p],
    "fh_rope_tables": [_p, _i32, _i32, _f32, _p, _p],
    "fh_rope_pair": [_p, _p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _i32, _p, _p, _i32, _i32,
                     _i32, _p, _p],
    "fh_kvcache_create": [_p, _i32, _i32, _i32, _i32, _i32, _pp],
    "fh_kvcache_destroy": [_p],
    "fh_kvcache_reset": [_p],
    "fh_kvcache_append": [_p, _i32, _p, _p, _i64, _i64, _i32],
    "fh_kvcache_view": [_p, _i32, C.POINTER(_i32), C.POINTER(_i32), _pp, _pp],
    "fh_matmul": [_p, _i32, _p, _i64, _i64, _i64, _p, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _p],
    "fh_flash_attention": [_p, _i32, _p, _i64, _i64, _i64, _p, _p, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _i32, _i32,
                           _f32, _i32, _p, _p],
    "fh_flash_attention_ex": [_p, _i32, _i32, _p, _i64, _i64, _i64, _p, _p, _i64, _i64, _i64, _i32, _i32, _i32, _i32,
                              _i32, _i32, _f32, _i32, _p, _p],
    "fh_flash_attention_decode_static": [_p, _i32, _i32, _p, _p, _p, _i64, _i64, _i32, _i32, _i32, _f32, _i32, _p],
    "fh_swiglu": [_p, _p, _p, _p, _i64],
    "fh_add3": [_p, _p, _p, _p, _p, _i64],
    "fh_transpose_shd": [_p, _p, _i32, _i32, _i32, _p],
    "fh_cast_f32_f16": [_p, _p, _p, _i64],
    "fh_cast_f16_f32": [_p, _p, _p, _i64],
    "fh_cast_f32_bf16": [_p, _p, _p, _i64],
    "fh_argmax": [_p, _p, _i64, _p],
    "fh_kvcache_set_sliding": [_p, _i32],
    "fh_top_k": [_p, _p, _i64, _i32, _p, _p, _p],
    "fh_sample_token": [_p, _p, _i64, C.POINTER(SamplerParams), _p, _u32, _p, _p, _p, _p, _p],
    "fh_llama_decode_sampled": [_p, _u32, _i32, C.POINTER(SamplerParams), _p, _p, _u32, _u32, C.POINTER(_f32), _p,
                                C.POINTER(_f32)],
    "fh_llama_create": [_p, C.POINTER(LlamaConfig), _pp],
    "fh_llama_destroy": [_p],
    "fh_llama_load_tensor": [_p, C.c_char_p, _u32, _i64, _i64, _p, _sz],
    "fh_llama_set_rope_scaling": [_p, C.POINTER(RopeScaling)],
    "fh_llama_finalize": [_p],
    "fh_llama_reset": [_p],
    "fh_llama_forward": [_p, _p, _i32, _p, _p],
    "fh_llama_decode_greedy": [_p, _u32, _i32, _p, C.POINTER(_f32)],
    "fh_llama_weight_bytes": [_p, C.POINTER(_u64)],
    "fh_llama_trace_text": [_p, C.c_char_p, _sz, C.POINTER(C.c_size_t)],
    "fh_llama_config_from_gguf": [_p, C.POINTER(LlamaConfig)],
    "fh_llama_load_gguf": [_p, _p],
    "fh_rope_tables_weighted": [_p, _i32, _i32, _f32, _p, _p, _p],
    "fh_rope_tables_scaled": [_p, _i32, _i32, _f32, C.POINTER(RopeScaling), _p, _p, _p],
    "fh_gguf_open": [C.c_char_p, _pp],
    "fh_gguf_open_memory": [_p, _sz, _pp],
    "fh_gguf_close": [_p],
    "fh_gguf_info": [_p, C.POINTER(_u32), C.POINTER(_u64), C.POINTER(_u64), C.POINTER(_u64), C.POINTER(_u64)],
    "fh_gguf_meta_key": [_p, _u64, C.POINTER(C.c_char_p), C.POINTER(_u32)],
    "fh_gguf_meta_find": [_p, C.c_char_p, C.POINTER(C.c_char_p), C.POINTER(_u32)],
    "fh_gguf_meta_int": [_p, C.c_char_p, C.POINTER(_i64)],
    "fh_gguf_meta_float": [_p, C.c_char_p, C.POINTER(C.c_double)],
    "fh_gguf_meta_bool": [_p, C.c_char_p, C.POINTER(_i32)],
    "fh_gguf_meta_string": [_p, C.c_char_p, _pp, C.POINTER(_u64)],
    "fh_gguf_meta_array": [_p, C.c_char_p, C.POINTER(_u32), C.POINTER(_u64), _pp],
    "fh_gguf_meta_array_int": [_p, C.c_char_p, _u64, C.POINTER(_i64)],
    "fh_gguf_meta_array_float": [_p, C.c_char_p, _u64, C.POINTER(C.c_double)],
    "fh_gguf_meta_array_string": [_p, C.c_char_p, _u64, _pp, C.POINTER(_u64)],
    "fh_gguf_tensor_info": [_p, _u64, C.POINTER(GgufTensor)],
    "fh_gguf_tensor_find": [_p, C.c_char_p, C.POINTER(_u64)],
    "fh_gguf_tensor_data": [_p, _u64, _pp, C.POINTER(_sz)],
    "fh_qmatrix_from_gguf_tensor": [_p, _p, C.c_char_p, _pp],
}
STRING_GETTERS = ("fh_last_error", "fh_version")

_lib = None


def load() -> C.CDLL:
    """dlopen the library and attach the prototypes.  No device is touched."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `python -m kalosm_amd.build` "
                          "(there is no CPU fallback for the HIP path)")
    lib = C.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = C.c_int32
    for name in STRING_GETTERS:
        getattr(lib, name).restype = C.c_char_p
        getattr(lib, name).argtypes = []
    _lib = lib
    return lib


def check(status: int) -> None:
    if status != FH_OK:
        raise FusorHipError(status, load().fh_last_error().decode(errors="replace"))
