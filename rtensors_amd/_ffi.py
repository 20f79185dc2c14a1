"""ctypes binding of librt_hip.so (the C ABI declared in include/rt_hip.h).

There is no CPU fallback: if the library is missing, importing this module raises."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "librt_hip.so")

# every symbol include/rt_hip.h declares
SYMBOLS = [
    "rt_ctx_create", "rt_ctx_destroy", "rt_sync", "rt_last_error", "rt_status_name", "rt_dtype_size", "rt_device_count",
    "rt_alloc", "rt_alloc_uninit", "rt_alloc_from_slice", "rt_free", "rt_copy_from_slice", "rt_copy_range_within",
    "rt_read", "rt_write", "rt_copy", "rt_dump", "rt_equal", "rt_convert",
    "rt_fill_contiguous", "rt_fill_1d_strided", "rt_fill_nd",
    "rt_unary_contiguous", "rt_unary_1d_strided", "rt_unary_nd",
    "rt_scalar_contiguous", "rt_scalar_1d_strided", "rt_scalar_nd", "rt_unary_to", "rt_scalar_to",
    "rt_broadcast", "rt_reduce_flat", "rt_reduce_nd", "rt_reduce_nd_static", "rt_argmax_flat", "rt_argmax_nd", "rt_gather", "rt_matmul", "rt_fused_bias_relu", "rt_fused_l1_forward", "rt_fused_l1_relu_backward",
    "rt_fused_bias_relu_l1", "rt_fused_l1_relu_backward_t", "rt_fused_chain", "rt_debug_check_view", "rt_debug_check_overlap",
    "rt_event_create", "rt_event_record", "rt_event_elapsed_ms", "rt_event_destroy", "rt_mem_stats", "rt_mem_trim",
]

u64, i64, i32, vp = C.c_uint64, C.c_int64, C.c_int32, C.c_void_p
u64p, i64p, i32p, vpp = C.POINTER(C.c_uint64), C.POINTER(C.c_int64), C.POINTER(C.c_int32), C.POINTER(C.c_void_p)



class ChainStep(C.Structure):
    """rt_chain_step of include/rt_hip.h"""
    _fields_ = [("kind", C.c_int32), ("op", C.c_int32), ("operand", C.c_int32), ("reserved", C.c_int32), ("value", C.c_uint8 * 8)]


_SIGS = {
    "rt_ctx_create": [i32, vpp], "rt_ctx_destroy": [vp], "rt_sync": [vp], "rt_dtype_size": [i32], "rt_device_count": [i32p],
    "rt_alloc": [vp, i32, u64, vpp], "rt_alloc_uninit": [vp, i32, u64, vpp], "rt_alloc_from_slice": [vp, i32, vp, u64, vpp],
    "rt_free": [vp, vp], "rt_copy_from_slice": [vp, i32, vp, u64, vp, u64],
    "rt_copy_range_within": [vp, i32, vp, u64, vp, u64, u64, u64, u64],
    "rt_read": [vp, i32, vp, u64, u64, vp], "rt_write": [vp, i32, vp, u64, u64, vp], "rt_copy": [vp, i32, vp, u64, vpp],
    "rt_dump": [vp, i32, vp, u64, vp], "rt_equal": [vp, i32, vp, u64, vp, u64, i32p], "rt_convert": [vp, i32, vp, u64, i32, vp, u64],
    "rt_fill_contiguous": [vp, i32, vp, u64, vp, u64, u64], "rt_fill_1d_strided": [vp, i32, vp, u64, vp, u64, i64, u64],
    "rt_fill_nd": [vp, i32, vp, u64, vp, u64, i32, u64p, i64p],
    "rt_unary_contiguous": [vp, i32, i32, vp, u64, u64, u64], "rt_unary_1d_strided": [vp, i32, i32, vp, u64, u64, i64, u64],
    "rt_unary_nd": [vp, i32, i32, vp, u64, u64, i32, u64p, i64p],
    "rt_scalar_contiguous": [vp, i32, i32, vp, u64, vp, u64, u64], "rt_scalar_1d_strided": [vp, i32, i32, vp, u64, vp, u64, i64, u64],
    "rt_scalar_nd": [vp, i32, i32, vp, u64, vp, u64, i32, u64p, i64p],
    "rt_unary_to": [vp, i32, i32, vp, u64, u64, u64, vp, u64], "rt_scalar_to": [vp, i32, i32, vp, u64, vp, u64, u64, vp, u64],
    "rt_broadcast": [vp, i32, i32, i32, u64p, vp, u64, u64, i64p, vp, u64, u64, i64p, vp, u64, u64, i64p],
    "rt_reduce_flat": [vp, i32, i32, vp, u64, vp, u64, u64, u64],
    "rt_reduce_nd": [vp, i32, i32, vp, u64, u64, i32, u64p, i64p, vp, u64, i32],
    "rt_reduce_nd_static": [vp, i32, i32, vp, u64, u64, i32, u64p, i64p, vp, u64, i32],
    "rt_argmax_flat": [vp, i32, i32, vp, u64, vp, u64, u64, u64],
    "rt_argmax_nd": [vp, i32, i32, vp, u64, u64, i32, u64p, i64p, vp, u64, i32],
    "rt_gather": [vp, i32, vp, u64, u64, i32, u64p, i64p, vp, u64],
    "rt_matmul": [vp, i32, vp, u64, u64, i32, u64p, i64p, i32, vp, u64, u64, i32, u64p, i64p, i32, vp, u64, u64, u64, u64, u64],
    "rt_fused_bias_relu": [vp, i32, vp, u64, vp, u64, vp, u64, u64, u64],
    "rt_fused_l1_forward": [vp, i32, vp, u64, vp, u64, vp, u64, vp, u64, u64],
    "rt_fused_l1_relu_backward": [vp, i32, vp, u64, vp, u64, vp, u64, vp, u64, u64, u64],
    "rt_fused_bias_relu_l1": [vp, i32, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, u64, u64],
    "rt_fused_l1_relu_backward_t": [vp, i32, vp, u64, vp, u64, vp, u64, vp, u64, u64, u64],
    "rt_fused_chain": [vp, i32, i32, vpp, u64p, u64p, u64, i32, C.POINTER(ChainStep), vp, u64, u64],
    "rt_debug_check_view": [u64, i32, u64p, i64p, u64, u64p, i32p, i64p, i64p, i64p],
    "rt_debug_check_overlap": [i32, i32, u64p, u64, i64p, u64, i64p, u64, i32p, i32p],
    "rt_event_create": [vp, vpp], "rt_event_record": [vp, vp], "rt_event_elapsed_ms": [vp, vp, vp, C.POINTER(C.c_float)],
    "rt_event_destroy": [vp, vp], "rt_mem_stats": [vp, u64p, u64p, u64p], "rt_mem_trim": [vp],
}


def load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `python -m rtensors_amd.build` (hipcc, gfx950). "
                          "There is no CPU fallback for this backend.")
    lib = C.CDLL(LIB_PATH)
    for name in SYMBOLS:
        fn = getattr(lib, name)           # AttributeError if the library does not export a declared symbol
        if name in ("rt_last_error", "rt_status_name"):
            fn.restype = C.c_char_p
            fn.argtypes = [] if name == "rt_last_error" else [i32]
        else:
            fn.restype = i32
            fn.argtypes = _SIGS[name]
    return lib


lib = load()
