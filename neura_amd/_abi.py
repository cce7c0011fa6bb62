"""ctypes declarations of every symbol include/neura_hip.h exports.

Loading never touches the GPU; only nh_open does.  The library must have been built
in-tree (python -m neura_amd.build); a missing library is an error, never a fallback.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_float, c_int32, c_size_t, c_uint8, c_uint16, c_uint32, c_uint64, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY = os.path.join(HERE, "libneura_hip.so")

NH_F32, NH_F16, NH_Q8_0, NH_Q4_K, NH_Q6_K = 0, 1, 8, 12, 14
NH_Q3_K, NH_Q5_K = 11, 13
NH_OK, NH_E_ARGUMENT, NH_E_DEVICE, NH_E_MEMORY, NH_E_REFUSAL = 0, -1, -2, -3, -4
UINT64_MAX = (1 << 64) - 1


class Epilogue(ctypes.Structure):
    _fields_ = [("residual", c_void_p), ("swiglu", c_int32)]


class ModelConfig(ctypes.Structure):
    _fields_ = [(name, c_uint32) for name in
                ("layers", "hidden", "heads", "kv_heads", "head_dim", "ffn", "vocab", "context", "batch", "max_rows", "window")] + \
               [("rope_base", c_float), ("eps", c_float), ("cache_element", c_int32)]


class TensorTable(ctypes.Structure):
    _fields_ = [("matrix_element", c_int32), ("token_embd", c_uint64), ("output", c_uint64), ("output_norm", c_uint64)] + \
               [(name, POINTER(c_uint64)) for name in
                ("attn_norm", "attn_q", "attn_k", "attn_v", "attn_output", "ffn_norm", "ffn_gate", "ffn_up", "ffn_down")] + \
               [("matrix_elements", POINTER(c_int32))] + [(name, POINTER(c_uint64)) for name in ("attn_q_bias", "attn_k_bias", "attn_v_bias")]


# name -> (restype, argtypes); the single list of what the header declares
SIGNATURES = {
    "nh_open": (c_void_p, [c_int32]),
    "nh_close": (None, [c_void_p]),
    "nh_last_error": (c_char_p, []),
    "nh_alloc": (c_void_p, [c_void_p, c_size_t]),
    "nh_free": (c_int32, [c_void_p, c_void_p]),
    "nh_upload": (c_int32, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "nh_download": (c_int32, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "nh_copy": (c_int32, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "nh_clear": (c_int32, [c_void_p, c_void_p, c_size_t]),
    "nh_sync": (c_int32, [c_void_p]),
    "nh_timer_start": (c_int32, [c_void_p]),
    "nh_timer_stop": (c_int32, [c_void_p, POINTER(c_double)]),
    "nh_profile_begin": (c_int32, [c_void_p]),
    "nh_profile_end": (c_int32, [c_void_p, POINTER(c_double), POINTER(c_uint64), POINTER(c_uint64)]),
    "nh_weights_create": (c_void_p, [c_void_p, c_size_t]),
    "nh_weights_destroy": (None, [c_void_p]),
    "nh_weights_put": (c_int32, [c_void_p, c_size_t, c_void_p, c_size_t]),
    "nh_weights_at": (c_void_p, [c_void_p, c_size_t]),
    "nh_weights_bytes": (c_size_t, [c_void_p]),
    "nh_dequant": (c_int32, [c_void_p, c_int32, c_void_p, c_uint64, c_void_p]),
    "nh_convert_half": (c_int32, [c_void_p, c_void_p, c_uint64, c_void_p]),
    "nh_pack_q8_0": (c_int32, [c_void_p, c_void_p, c_uint64, c_void_p]),
    "nh_gemv": (c_int32, [c_void_p, c_int32, c_void_p, c_uint32, c_uint32, c_void_p, c_uint32, c_void_p, POINTER(Epilogue)]),
    "nh_gemm": (c_int32, [c_void_p, c_int32, c_void_p, c_uint32, c_uint32, c_void_p, c_int32, c_uint32, c_void_p, POINTER(Epilogue)]),
    "nh_rmsnorm": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_uint32, c_uint32, c_void_p, c_void_p]),
    "nh_rope": (c_int32, [c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_void_p, c_float, c_void_p]),
    "nh_cache_write": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32,
                                 c_uint32, c_void_p, c_void_p, c_int32]),
    "nh_attention": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32,
                               c_uint32, c_uint32, c_void_p, c_float, c_void_p]),
    "nh_cache_write_element": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32,
                                         c_uint32, c_void_p, c_void_p, c_int32, c_int32]),
    "nh_attention_element": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32,
                                       c_uint32, c_uint32, c_void_p, c_float, c_void_p, c_int32]),
    "nh_gather": (c_int32, [c_void_p, c_int32, c_void_p, c_uint32, c_uint32, c_void_p, c_uint32, c_uint32, c_void_p, c_void_p]),
    "nh_argmax": (c_int32, [c_void_p, c_void_p, c_uint32, c_uint32, c_void_p]),
    "nh_argmax_static": (c_int32, [c_void_p, c_void_p, c_uint32, c_uint32, c_void_p]),
    "nh_sample": (c_int32, [c_void_p, c_void_p, c_uint32, c_uint32, c_void_p, c_void_p]),
    "nh_model_create": (c_void_p, [c_void_p, POINTER(ModelConfig), c_void_p, POINTER(TensorTable)]),
    "nh_model_destroy": (None, [c_void_p]),
    "nh_decode_step": (c_int32, [c_void_p, POINTER(c_uint32), POINTER(c_uint32), POINTER(c_uint8), c_uint32, POINTER(c_uint32)]),
    "nh_decode_step_sampled": (c_int32, [c_void_p, POINTER(c_uint32), POINTER(c_uint32), POINTER(c_uint8), c_uint32, c_void_p, POINTER(c_uint32)]),
    "nh_prefill": (c_int32, [c_void_p, POINTER(c_uint32), c_uint32, POINTER(c_uint32), POINTER(c_uint8), c_uint32]),
    "nh_model_time_products": (c_int32, [c_void_p, c_uint32, POINTER(c_double), POINTER(c_uint64), POINTER(c_uint64)]),
    "nh_model_reset": (c_int32, [c_void_p, POINTER(c_uint8), c_uint32]),
    "nh_model_logits": (c_int32, [c_void_p, c_void_p]),
    "nh_model_cache_write": (c_int32, [c_void_p, c_uint32, c_int32, c_void_p]),
    "nh_model_cache_read": (c_int32, [c_void_p, c_uint32, c_int32, c_void_p]),
    "nh_model_keep_prefix": (c_int32, [c_void_p, c_uint32]),
    "nh_model_reset_shared": (c_int32, [c_void_p, POINTER(c_uint8), POINTER(c_uint8), c_uint32]),
    "nh_model_shared_write": (c_int32, [c_void_p, c_uint32, c_int32, c_void_p]),
    "nh_model_shared_read": (c_int32, [c_void_p, c_uint32, c_int32, c_void_p]),
    "nh_model_capacity": (c_uint32, [c_void_p]),
    "nh_model_seam_fallbacks": (c_uint32, [c_void_p]),
}

_library = None


def library():
    """The loaded C ABI; raises when the HIP library has not been built."""
    global _library
    if _library is None:
        if not os.path.exists(LIBRARY):
            raise RuntimeError("libneura_hip.so is not built: run `python -m neura_amd.build` (there is no CPU fallback)")
        held = ctypes.CDLL(LIBRARY)
        for name, (restype, argtypes) in SIGNATURES.items():
            function = getattr(held, name)
            function.restype = restype
            function.argtypes = argtypes
        _library = held
    return _library


__all__ = [name for name in dir() if not name.startswith("_")] + ["c_uint16"]
