"""Loads libtwmarlin_hip.so and declares the C ABI of include/twmarlin.h for ctypes.

There is no fallback: if the library is missing, loading raises.  Nothing here
computes on the CPU.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtwmarlin_hip.so")

OK, DEVICE_ERROR, MEMORY_ERROR, SHAPE_ERROR, UNSUPPORTED_OP, INVALID_HANDLE = range(6)
F32, F16, I32, I8, U8 = range(5)

_vp, _u32, _sz, _int = C.c_void_p, C.c_uint32, C.c_size_t, C.c_int

# name -> (restype, argtypes); the list every symbol of include/twmarlin.h must match
SIGNATURES = {
    "twm_version": (C.c_char_p, []),
    "twm_device_count": (_int, []),
    "twm_last_error": (C.c_char_p, []),
    "twm_last_error_kind": (_int, []),
    "twm_stream_create": (_vp, [_vp]),
    "twm_stream_destroy": (_int, [_vp, _vp]),
    "twm_stream_sync": (_int, [_vp, _vp]),
    "twm_cast_f32_to_f16": (_int, [_vp, _vp, _vp, _sz]),
    "twm_cast_f16_to_f32": (_int, [_vp, _vp, _vp, _sz]),
    "twm_ctx_create": (_vp, [_int]),
    "twm_ctx_destroy": (None, [_vp]),
    "twm_ctx_sync": (_int, [_vp]),
    "twm_ctx_set_stream": (_int, [_vp, _vp]),
    "twm_ctx_stream": (_vp, [_vp]),
    "twm_ctx_info": (_int, [_vp, C.c_char_p, _sz]),
    "twm_ctx_set_option": (_int, [_vp, C.c_char_p, _int]),
    "twm_debug_trace": (_int, [_vp, _vp, _u32]),
    "twm_debug_mfma_mix": (_int, [_vp, _int, _int, _int, _int, C.POINTER(C.c_float)]),
    "twm_malloc": (_vp, [_vp, _sz]),
    "twm_free": (_int, [_vp, _vp]),
    "twm_memcpy_h2d": (_int, [_vp, _vp, _vp, _sz]),
    "twm_memcpy_d2h": (_int, [_vp, _vp, _vp, _sz]),
    "twm_memcpy_d2d": (_int, [_vp, _vp, _vp, _sz]),
    "twm_memset_zero": (_int, [_vp, _vp, _sz]),
    "twm_event_create": (_vp, [_vp]),
    "twm_event_destroy": (_int, [_vp, _vp]),
    "twm_event_record": (_int, [_vp, _vp]),
    "twm_event_elapsed_ms": (_int, [_vp, _vp, _vp, C.POINTER(C.c_float)]),
    "twm_quantize_weights_q4_0": (_int, [_vp, _vp, _u32, _u32, _vp]),
    "twm_reorder_to_tw_marlin": (_int, [_vp, _vp, _u32, _u32, _vp, _vp]),
    "twm_quantize_f32_to_tw_marlin": (_int, [_vp, _vp, _int, _u32, _u32, _vp, _vp]),
    "twm_fuse_tw_marlin_n": (_int, [_vp, C.POINTER(_vp), C.POINTER(_vp), _u32, C.POINTER(_u32), _u32, _vp, _vp]),
    "twm_dequant_to_f16": (_int, [_vp, _vp, _vp, _u32, _u32, _vp]),
    "twm_dequant_to_f32": (_int, [_vp, _vp, _vp, _u32, _u32, _vp]),
    "twm_split_qkv": (_int, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32]),
    "twm_argmax_f32": (_int, [_vp, _vp, _u32, _u32, _vp]),
    "twm_split_gate_up": (_int, [_vp, _vp, _vp, _vp, _u32, _u32]),
    "twm_silu_mul": (_int, [_vp, _vp, _vp, _vp, _sz]),
    "twm_swiglu_rows": (_int, [_vp, _vp, _u32, _u32, _int, _vp]),
    "twm_pair_gate_up": (_int, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _vp, _vp]),
    "twm_gemm_tw_marlin_m1": (_int, [_vp, _vp, _vp, _vp, _vp, _u32, _u32]),
    "twm_gemm_tw_marlin_m1_noalloc": (_int, [_vp, _vp, _vp, _vp, _vp, _u32, _u32]),
    "twm_noalloc_scratch_fill": (_int, [_vp, _int]),
    "twm_gemm_tw_marlin_m1_from_buffer": (_int, [_vp, _vp, _vp, _sz, _vp, _sz, _vp, _u32, _u32]),
    "twm_pick_splits_reference": (None, [_u32, _u32, C.POINTER(_u32), C.POINTER(_u32), C.POINTER(_u32)]),
    "twm_weight_upload": (_vp, [_vp, _vp, _vp, _u32, _u32]),
    "twm_weight_from_device": (_vp, [_vp, _vp, _vp, _u32, _u32]),
    "twm_weight_destroy": (None, [_vp]),
    "twm_weight_fuse_n": (_vp, [_vp, _vp, _u32]),
    "twm_weight_dims": (_int, [_vp, C.POINTER(_u32), C.POINTER(_u32)]),
    "twm_weight_bytes": (_sz, [_vp]),
    "twm_weight_tune": (_int, [_vp, _vp, _vp, _u32]),
    "twm_weight_tuned_plan": (_int, [_vp, _u32, _vp]),
    "twm_weight_ensure": (_int, [_vp, _vp, _int]),
    "twm_weight_drop": (_int, [_vp, _vp, _int]),
    "twm_weight_copies": (_int, [_vp]),
    "twm_weight_blob_bytes": (_sz, [_vp]),
    "twm_weight_export": (_int, [_vp, _vp, _vp, _sz]),
    "twm_weight_import": (_vp, [_vp, _vp, _sz]),
    "twm_weight_dequant_f16": (_int, [_vp, _vp, _vp]),
    "twm_gemm": (_int, [_vp, _vp, _vp, _int, _u32, _vp, _u32]),
    "twm_gemm_f16out": (_int, [_vp, _vp, _vp, _int, _u32, _vp, _u32]),
    "twm_gemm_split": (_int, [_vp, _vp, _vp, _int, _u32, C.POINTER(_vp), C.POINTER(_u32), _u32, _u32]),
    "twm_weight_gate_up": (_vp, [_vp, _vp, _vp, _vp, _vp, _u32, _u32]),
    "twm_weight_is_paired": (_int, [_vp]),
    "twm_gemm_swiglu": (_int, [_vp, _vp, _vp, _int, _u32, _vp, _u32]),
    "twm_gemm_geglu": (_int, [_vp, _vp, _vp, _int, _u32, _vp, _u32]),
    "twm_gemm_split_bias": (_int, [_vp, _vp, _vp, _int, _u32, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_u32), _u32, _u32]),
    "twm_bank_from_device": (_vp, [_vp, _vp, _vp, _sz, _sz, _u32, _u32, _u32, _int]),
    "twm_bank_from_device_offsets": (_vp, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _int]),
    "twm_bank_destroy": (None, [_vp]),
    "twm_bank_bytes": (_sz, [_vp]),
    "twm_bank_gemv": (_int, [_vp, _vp, _vp, _int, _u32, _vp, _u32, _int, _vp]),
    "twm_bank_down_axpy": (_int, [_vp, _vp, _vp, _int, _vp, _vp, _u32, _vp]),
    "twm_geglu_rows": (_int, [_vp, _vp, _u32, _u32, _int, _vp]),
    "twm_plan_describe": (_int, [_vp, _u32, _u32, _u32, _int, _int, _vp, _sz]),
    "twm_plan_describe_m1": (_int, [_vp, _u32, _u32, _vp, _sz]),
    "twm_batched_marlin_gate_up": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32]),
    "twm_batched_marlin_down_axpy": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32]),
    "twm_batched_marlin_split_geglu": (_int, [_vp, _vp, _vp, _u32, _u32]),
    "twm_gemm_tw_marlin_m1_indirect": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _vp, _u32, _u32]),
    "twm_pick_splits": (_u32, [_u32, _u32, _u32]),
    "twm_graph_begin": (_int, [_vp]),
    "twm_graph_end": (_vp, [_vp]),
    "twm_graph_launch": (_int, [_vp, _vp]),
    "twm_graph_destroy": (None, [_vp]),
}

_lib = None


def load():
    """Returns the loaded library; raises if it has not been built (python -m tensorwarp_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libtwmarlin_hip.so is missing at %s: build it with `python -m tensorwarp_amd.build` "
                "(there is no CPU fallback)" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib
