"""Loads libferric_hip.so (the C-ABI library of include/ferric_hip.h) through ctypes.

There is no CPU fallback: if the library has not been built, or no gfx950 device can be
initialised, every entry point of this package raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "libferric_hip.so")

OK, ERR_UNSUPPORTED_TYPE, ERR_SHAPE, ERR_HIP, ERR_ARG, ERR_FORMAT = 0, -1, -2, -3, -4, -5

_vp = C.c_void_p
_sz = C.c_size_t
_u32 = C.c_uint32

# name -> (restype, argtypes); exactly the symbols include/ferric_hip.h declares
SYMBOLS = {
    "fhip_init": (C.c_int, [C.c_int]),
    "fhip_last_error": (C.c_char_p, []),
    "fhip_device_cus": (C.c_int, []),
    "fhip_type_size": (_sz, [_u32, _sz]),
    "fhip_block_bytes": (C.c_int, [_u32, C.POINTER(_sz), C.POINTER(_sz)]),
    "fhip_malloc": (C.c_int, [C.POINTER(_vp), _sz]),
    "fhip_free": (C.c_int, [_vp]),
    "fhip_memcpy_h2d": (C.c_int, [_vp, _vp, _sz, _vp]),
    "fhip_memcpy_d2h": (C.c_int, [_vp, _vp, _sz, _vp]),
    "fhip_memcpy_d2d": (C.c_int, [_vp, _vp, _sz, _vp]),
    "fhip_memcpy_2d_d2d": (C.c_int, [_vp, _sz, _vp, _sz, _sz, _sz, _vp]),
    "fhip_memset": (C.c_int, [_vp, C.c_int, _sz, _vp]),
    "fhip_stream_create": (C.c_int, [C.POINTER(_vp)]),
    "fhip_stream_destroy": (C.c_int, [_vp]),
    "fhip_stream_sync": (C.c_int, [_vp]),
    "fhip_event_create": (C.c_int, [C.POINTER(_vp)]),
    "fhip_event_destroy": (C.c_int, [_vp]),
    "fhip_event_record": (C.c_int, [_vp, _vp]),
    "fhip_event_sync": (C.c_int, [_vp]),
    "fhip_event_elapsed_ms": (C.c_int, [_vp, _vp, C.POINTER(C.c_float)]),
    "fhip_graph_capture_begin": (C.c_int, [_vp]),
    "fhip_graph_capture_end": (C.c_int, [_vp, C.POINTER(_vp)]),
    "fhip_graph_launch": (C.c_int, [_vp, _vp]),
    "fhip_graph_destroy": (C.c_int, [_vp]),
    "fhip_weight_create": (C.c_int, [_u32, _vp, _sz, _sz, _sz, C.POINTER(_vp)]),
    "fhip_weight_create_parts": (C.c_int, [C.c_uint32, _vp, _vp, _sz, _sz, _sz, _vp]),
    "fhip_weight_wrap_device": (C.c_int, [_u32, _vp, _sz, _sz, _sz, C.POINTER(_vp)]),
    "fhip_weight_destroy": (None, [_vp]),
    "fhip_weight_rows": (_sz, [_vp]),
    "fhip_weight_cols": (_sz, [_vp]),
    "fhip_weight_nbytes": (_sz, [_vp]),
    "fhip_weight_type": (_u32, [_vp]),
    "fhip_f16_to_f32": (C.c_int, [_vp, _sz, _vp, _vp]),
    "fhip_dequant_rows": (C.c_int, [_vp, _sz, _sz, _vp, _vp]),
    "fhip_deq_raw": (C.c_int, [_vp, _sz, _sz, _u32, _vp, C.POINTER(_sz)]),
    "fhip_matmul_q": (C.c_int, [_vp, _vp, _sz, _vp, _vp]),
    "fhip_matmul_q_swiglu": (C.c_int, [_vp, _vp, _sz, _vp, _vp]),
    "fhip_swiglu": (C.c_int, [_vp, _sz, _sz, _vp, _vp]),
    "fhip_ffn": (C.c_int, [_vp, _vp, _vp, _sz, _vp, _vp, _vp]),
    "fhip_gemm_q_bf16": (C.c_int, [_vp, _vp, _sz, _vp, _vp]),
    "fhip_moe_topk": (C.c_int, [_vp, _vp, _sz, _sz, _sz, C.c_int, C.c_float, C.c_int, _vp, _vp]),
    "fhip_matmul_q_swiglu_id": (C.c_int, [_vp, _vp, _sz, _vp, _sz, _sz, _vp, _vp]),
    "fhip_matmul_q_relu2_id": (C.c_int, [_vp, _vp, _sz, _vp, _sz, _sz, _vp, _vp]),
    "fhip_matmul_q_id": (C.c_int, [_vp, _vp, _vp, _sz, _sz, _vp, _vp]),
    "fhip_matmul_q_id_wsum": (C.c_int, [_vp, _vp, _sz, _vp, _sz, _sz, _vp, _vp, _vp]),
    "fhip_gguf_parse": (C.c_int, [_vp, _sz, _vp]),
    "fhip_gguf_open": (C.c_int, [C.c_char_p, _vp]),
    "fhip_gguf_close": (None, [_vp]),
    "fhip_gguf_version": (C.c_uint32, [_vp]),
    "fhip_gguf_data_start": (C.c_uint64, [_vp]),
    "fhip_gguf_n_tensors": (_sz, [_vp]),
    "fhip_gguf_tensor": (C.c_int, [_vp, _sz, _vp, _vp, _vp, _vp, _vp]),
    "fhip_gguf_find": (C.c_long, [_vp, C.c_char_p]),
    "fhip_gguf_raw": (C.c_int, [_vp, C.c_char_p, _vp, _vp]),
    "fhip_gguf_n_meta": (_sz, [_vp]),
    "fhip_gguf_meta_key": (C.c_char_p, [_vp, _sz]),
    "fhip_gguf_meta_kind": (C.c_int, [_vp, C.c_char_p, _vp]),
    "fhip_gguf_meta_u64": (C.c_int, [_vp, C.c_char_p, _sz, _vp]),
    "fhip_gguf_meta_i64": (C.c_int, [_vp, C.c_char_p, _sz, _vp]),
    "fhip_gguf_meta_f64": (C.c_int, [_vp, C.c_char_p, _sz, _vp]),
    "fhip_gguf_meta_str": (C.c_int, [_vp, C.c_char_p, _sz, _vp, _vp]),
    "fhip_weight_from_gguf_cat": (C.c_int, [_vp, _vp, _sz, _vp]),
    "fhip_weight_from_gguf": (C.c_int, [_vp, C.c_char_p, _vp]),
    "fhip_cvt_f32_bf16": (C.c_int, [_vp, _sz, _vp, _vp]),
    "fhip_matmul_q_coop": (C.c_int, [_vp, _vp, _sz, _vp, _vp, _vp]),
    "fhip_ffn_coop_ws_bytes": (_sz, [_vp, _vp, _sz]),
    "fhip_ffn_coop": (C.c_int, [_vp, _vp, _vp, _sz, _vp, _vp, _vp]),
    "fhip_matmul_q_f16x2_ws_bytes": (_sz, [_vp, _sz]),
    "fhip_matmul_q_f16x2": (C.c_int, [_vp, _vp, _sz, _vp, _vp, _vp]),
    "fhip_ffn_f16x2_ws_bytes": (_sz, [_vp, _vp, _sz]),
    "fhip_ffn_f16x2": (C.c_int, [_vp, _vp, _vp, _sz, _vp, _vp, _vp]),
    "fhip_rmsnorm": (C.c_int, [_vp, _vp, _sz, _sz, C.c_float, _vp, _vp]),
    "fhip_add_rmsnorm": (C.c_int, [_vp, _vp, _vp, _sz, _sz, C.c_float, _vp, _vp, _vp]),
    "fhip_add": (C.c_int, [_vp, _vp, _sz, _vp, _vp]),
    "fhip_mul_sigmoid": (C.c_int, [_vp, _vp, _sz, _vp, _vp]),
    "fhip_kvq_sizes": (C.c_int, [C.c_int, _sz, _sz, C.POINTER(_sz), C.POINTER(_sz)]),
    "fhip_kvq_append": (C.c_int, [C.c_int, _vp, _sz, _sz, _sz, _vp, C.c_uint32, C.c_int, _sz, _vp, _vp, _vp]),
    "fhip_causal_attention": (C.c_int, [_vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, C.c_float, _vp, _vp]),
    "fhip_kvq_append2": (C.c_int, [C.c_int, _vp, _vp, _sz, _sz, _sz, _vp, C.c_uint32, _sz, _vp, _vp, _vp, _vp, _vp]),
    "fhip_decode_attention_kvq": (C.c_int, [C.c_int, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _vp, _sz, C.c_float, _vp, _vp, _vp]),
    "fhip_qkv_post_packed": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, C.c_int, C.c_float, C.c_float, _vp, _vp, _vp, _vp]),
    "fhip_kvq_dequantize_rows": (C.c_int, [C.c_int, _vp, _vp, _sz, _sz, _sz, _vp, _vp, _vp]),
    "fhip_geglu": (C.c_int, [_vp, _sz, _sz, _vp, _vp]),
    "fhip_rope": (C.c_int, [_vp, _sz, _sz, _sz, _sz, _sz, C.c_float, _vp, _u32, _vp, C.c_int, _vp, _vp]),
    "fhip_kv_append2": (C.c_int, [_vp, _vp, _sz, _sz, _vp, _u32, _vp, _vp, _sz, _vp]),
    "fhip_qkv_post": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, C.c_int, C.c_float, C.c_float, _vp, _vp, _vp,
                                _sz, _vp]),
    "fhip_decode_attention_ws_bytes": (_sz, [_sz, _sz, _sz, _sz]),
    "fhip_decode_attention": (C.c_int, [_vp, _vp, _vp, _sz, _sz, _sz, _sz, _vp, _vp, _vp, _vp]),
    "fhip_qkv_post_attention": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, C.c_int, C.c_float, C.c_float, _vp, _vp, _sz, _sz, _sz,
                                          C.c_float, _vp, _vp, _vp]),
    "fhip_decode_attention_ex": (C.c_int, [_vp, _vp, _vp, _sz, _sz, _sz, _sz, _vp, _sz, C.c_float, _vp, _vp, _vp]),
    "fhip_norm_matmul_q": (C.c_int, [_vp, _vp, _vp, _vp, C.c_float, _vp, _vp, C.c_int, _vp, _vp]),
    "fhip_debug_generic_matvec": (C.c_int, [C.c_int]),
    "fhip_debug_quad_matvec": (C.c_int, [C.c_int]),
    "fhip_debug_gemm_tile": (C.c_int, [C.c_int]),
    "fhip_matvec_precision": (C.c_int, [C.c_int]),
    "fhip_weight_matvec_precision": (C.c_int, [_vp, C.c_int]),
    "fhip_weight_batch_policy": (C.c_int, [_vp, C.c_int]),
    "fhip_ffn_noalloc": (C.c_int, [_vp, _vp, _vp, _sz, _vp, _vp]),
    "fhip_batch_policy": (C.c_int, [C.c_int]),
    "fhip_workspace_bytes": (C.c_size_t, [_vp, _vp, C.c_size_t]),
    "fhip_workspace_bytes_coop": (C.c_size_t, [_vp, _vp, C.c_size_t]),
    "fhip_workspace_reserve": (C.c_int, [_vp, C.c_size_t]),
    "fhip_workspace_release": (None, [_vp]),
    "fhip_debug_read_probe": (C.c_int, [_vp, _sz, _vp, _vp]),
    "fhip_debug_mfma_probe": (C.c_int, [C.c_int, _vp, C.POINTER(C.c_double), _vp]),
    "fhip_debug_matmul_q_loop": (C.c_int, [_vp, _sz, _sz, _vp, C.c_int, _vp, _vp]),
    "fhip_u32_add": (C.c_int, [_vp, _sz, _u32, _vp]),
    "fhip_matvec_q8_0_host": (C.c_int, [_vp, _vp, _sz, _sz, _sz, _vp]),
    "fhip_pool_create": (C.c_int, [_sz, _vp]),
    "fhip_pool_threads": (_sz, [_vp]),
    "fhip_pool_uploads": (_sz, [_vp]),
    "fhip_pool_forget": (None, [_vp]),
    "fhip_pool_destroy": (None, [_vp]),
    "fhip_matvec_q8_0_pooled": (C.c_int, [_vp, _vp, _sz, _vp, _sz, _sz, _sz, _sz, _vp]),
}

_lib = None
_inited = False


class FerricHipError(RuntimeError):
    """A HIP runtime failure or an unusable argument reported by the library."""


def load():
    """dlopen the library and bind every declared symbol (no device is touched)."""
    global _lib
    if _lib is None:
        if not os.path.exists(SO_PATH):
            raise ImportError(f"{SO_PATH} is missing: build it with `python -m ferric_amd.build` (needs hipcc); "
                              "there is no CPU fallback")
        lib = C.CDLL(SO_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)  # AttributeError if the library does not export it
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def last_error():
    return load().fhip_last_error().decode("utf-8", "replace")


def check(rc):
    """Map a return code to the exception the reference's behaviour calls for:
    unsupported type -> ValueError (reference: Err(String)); shape violation -> AssertionError
    (reference: assert!/assert_eq! panic); anything else -> FerricHipError."""
    if rc == OK:
        return
    msg = last_error()
    if rc in (ERR_UNSUPPORTED_TYPE, ERR_FORMAT):
        raise ValueError(msg)
    if rc == ERR_SHAPE:
        raise AssertionError(msg)
    raise FerricHipError(f"[{rc}] {msg}")


def init(device=0):
    """Initialise the device once per process; raises if there is no usable gfx950 GPU."""
    global _inited
    lib = load()
    if not _inited:
        check(lib.fhip_init(device))
        _inited = True
    return lib
