"""ctypes binding of liboxb_hip.so (the C ABI declared in include/oxb_hip.h).

The library is the product: if it is missing this module raises, it never
substitutes a CPU implementation."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# OXB_HIP_LIBRARY names another build of the same library (comparing two builds on one GPU)
LIB_PATH = os.environ.get("OXB_HIP_LIBRARY") or os.path.join(_HERE, "lib", "liboxb_hip.so")
_lib = None

u8p = C.POINTER(C.c_uint8)
f32p = C.POINTER(C.c_float)
u32p = C.POINTER(C.c_uint32)
u64p = C.POINTER(C.c_uint64)
szp = C.POINTER(C.c_size_t)

_SIGNATURES = {
    "oxb_hip_init": ([C.c_int], C.c_int),
    "oxb_hip_shutdown": ([], None),
    "oxb_hip_device_count": ([], C.c_int),
    "oxb_hip_device_info": ([C.c_char_p, C.c_size_t, szp, szp], C.c_int),
    "oxb_hip_synchronize": ([], C.c_int),
    "oxb_hip_set_stream": ([C.c_void_p], C.c_int),
    "oxb_hip_last_error": ([], C.c_char_p),
    "oxb_hip_upload_q1": ([u64p, u8p, C.c_size_t, C.c_uint32, C.c_uint32], C.c_int),
    "oxb_hip_upload_tq2": ([u64p, u8p, C.c_size_t, C.c_uint32, C.c_uint32], C.c_int),
    "oxb_hip_upload_q1_raw": ([u64p, u8p, C.c_size_t], C.c_int),
    "oxb_hip_upload_tq2_raw": ([u64p, u8p, C.c_size_t], C.c_int),
    "oxb_hip_free_weight": ([C.c_uint64], C.c_int),
    "oxb_hip_weight_info": ([C.c_uint64, C.POINTER(C.c_int), u32p, u32p, szp], C.c_int),
    "oxb_hip_dequant": ([C.c_uint64, f32p, C.c_size_t], C.c_int),
    "oxb_hip_gemv": ([C.c_uint64, f32p, f32p, C.c_uint32, C.c_uint32, C.c_uint32], C.c_int),
    "oxb_hip_gemv_dev": ([C.c_uint64, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32], C.c_int),
    "oxb_hip_profile_gemv": ([u64p, C.c_uint32, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32,
                              C.c_uint32, f32p], C.c_int),
    "oxb_hip_profile_gemv_floor": ([u64p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, f32p], C.c_int),
    "oxb_hip_gemm": ([C.c_uint64, f32p, f32p, C.c_uint32, C.c_uint32, C.c_uint32], C.c_int),
    "oxb_hip_gemm_dev": ([C.c_uint64, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32], C.c_int),
    "oxb_hip_gemm_dev_static": ([C.c_uint64, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32], C.c_int),
    "oxb_hip_profile_gemm": ([C.c_uint64, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32,
                              C.c_uint32, C.c_uint32, f32p], C.c_int),
    "oxb_hip_gemv_q1_g128": ([u8p, C.c_size_t, f32p, C.c_size_t, f32p, C.c_size_t, C.c_uint32, C.c_uint32], C.c_int),
    "oxb_hip_gemv_tq2_g128": ([u8p, C.c_size_t, f32p, C.c_size_t, f32p, C.c_size_t, C.c_uint32, C.c_uint32], C.c_int),
    "oxb_hip_ffn_phase": ([C.c_int, f32p, f32p, f32p, C.c_float, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint32,
                           C.c_uint32, C.c_uint32], C.c_int),
    "oxb_hip_attn_phase": ([C.c_int, f32p, f32p, C.c_float, C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint32, f32p, f32p, f32p], C.c_int),
    "oxb_hip_upload_f32": ([u64p, f32p, C.c_size_t], C.c_int),
    "oxb_hip_free_f32": ([C.c_uint64], C.c_int),
    "oxb_hip_model_create": ([C.c_void_p, u64p], C.c_int),
    "oxb_hip_model_reset": ([C.c_uint64], C.c_int),
    "oxb_hip_model_destroy": ([C.c_uint64], C.c_int),
    "oxb_hip_decode": ([C.c_uint64, f32p, u32p, f32p, u32p], C.c_int),
    "oxb_hip_decode_hidden": ([C.c_uint64, f32p, u32p, f32p], C.c_int),
    "oxb_hip_model_set_lm_head": ([C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint32], C.c_int),
    "oxb_hip_model_set_rope_rows": ([C.c_uint64, C.c_uint32, C.c_uint32, f32p, f32p], C.c_int),
    "oxb_hip_prefill": ([C.c_uint64, C.c_uint32, f32p, C.c_uint32, C.c_uint32, f32p, u32p], C.c_int),
    "oxb_hip_model_uses_graph": ([C.c_uint64], C.c_int),
    "oxb_hip_model_set_attention": ([C.c_uint64, C.c_void_p], C.c_int),
    "oxb_hip_model_get_attention": ([C.c_uint64, C.c_void_p], C.c_int),
    "oxb_hip_model_read_kv": ([C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p,
                               f32p, f32p], C.c_int),
    "oxb_hip_model_kv_reserve": ([C.c_uint64, C.c_uint32, C.c_uint32], C.c_int),
    "oxb_hip_model_kv_release": ([C.c_uint64, C.c_uint32], C.c_int),
    "oxb_hip_model_kv_pool": ([C.c_uint64, C.c_void_p], C.c_int),
    "oxb_hip_model_kv_capacity": ([C.c_uint64, C.c_uint32, u32p], C.c_int),
    "oxb_hip_kv_quantize_rows": ([C.c_int, f32p, C.c_uint32, C.c_uint32, u8p, f32p], C.c_int),
    "oxb_hip_kv_dequantize_rows": ([C.c_int, u8p, f32p, C.c_uint32, C.c_uint32, f32p], C.c_int),
    "oxb_hip_gguf_info": ([C.c_char_p, C.c_void_p], C.c_int),
    "oxb_hip_gguf_metadata": ([C.c_char_p, C.c_char_p, C.c_char_p, C.c_size_t], C.c_int),
    "oxb_hip_gguf_tensor": ([C.c_char_p, C.c_char_p, C.POINTER(C.c_int), u32p, u64p, u64p, u64p], C.c_int),
    "oxb_hip_load_gguf": ([C.c_char_p, C.c_uint32, C.c_uint32, u64p, u64p, C.c_void_p], C.c_int),
    "oxb_hip_upload_embedding": ([u64p, C.c_void_p, C.c_size_t, C.c_int, C.c_uint32, C.c_uint32], C.c_int),
    "oxb_hip_free_embedding": ([C.c_uint64], C.c_int),
    "oxb_hip_embedding_rows": ([C.c_uint64, u32p, C.c_uint32, f32p], C.c_int),
    "oxb_hip_decode_tokens": ([C.c_uint64, C.c_uint64, u32p, u32p, C.c_uint32, u32p], C.c_int),
    "oxb_hip_decode_tokens_sampled": ([C.c_uint64, C.c_uint64, u32p, u32p, C.c_uint32, C.c_void_p, u64p, u32p], C.c_int),
    "oxb_hip_sample_logits": ([f32p, C.c_uint32, C.c_uint32, C.c_void_p, u64p, u32p], C.c_int),
    "oxb_hip_sum_in_order": ([f32p, C.c_uint32, f32p], C.c_int),
    "oxb_hip_set_gemv_packed_min_batch": ([C.c_uint32], C.c_int),
    "oxb_hip_prefill_tokens": ([C.c_uint64, C.c_uint64, C.c_uint32, u32p, C.c_uint32, C.c_uint32, f32p, u32p], C.c_int),
    "oxb_hip_repack_sizes": ([C.c_int, C.c_uint32, C.c_uint32, szp, szp], C.c_int),
    "oxb_hip_repack": ([C.c_int, u8p, C.c_size_t, C.c_uint32, C.c_uint32, u8p, C.c_size_t, u8p, C.c_size_t], C.c_int),
    "oxb_hip_unpack": ([C.c_int, u8p, C.c_size_t, u8p, C.c_size_t, C.c_uint32, C.c_uint32, u8p, C.c_size_t], C.c_int),
}


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with `python -m oxibonsai_amd.build` "
                              "(the native-hip tier has no CPU fallback)")
        L = C.CDLL(LIB_PATH)
        for name, (args, res) in _SIGNATURES.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = res
        _lib = L
    return _lib


def last_error() -> str:
    return lib().oxb_hip_last_error().decode("utf-8", "replace")
