"""ctypes binding of libtrueno_hip.so (include/trueno_hip.h).  The product's only route to the GPU."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("TRN_HIP_LIBRARY") or os.path.join(_HERE, "libtrueno_hip.so")   # another build, for comparisons

_lib = None

dptr = C.c_uint64
status = C.c_int
vp = C.c_void_p

# name -> argtypes (restype is trn_status unless listed in _RESTYPE)
SIGNATURES = {
    "trn_init": [C.c_uint],
    "trn_device_get_count": [C.POINTER(C.c_int)],
    "trn_device_get": [C.POINTER(C.c_int), C.c_int],
    "trn_device_get_name": [C.c_char_p, C.c_int, C.c_int],
    "trn_device_total_mem": [C.POINTER(C.c_size_t), C.c_int],
    "trn_primary_ctx_retain": [C.POINTER(vp), C.c_int],
    "trn_primary_ctx_release": [C.c_int],
    "trn_ctx_set_current": [vp],
    "trn_ctx_synchronize": [],
    "trn_module_load_data": [C.POINTER(vp), vp],
    "trn_module_unload": [vp],
    "trn_module_get_function": [C.POINTER(vp), vp, C.c_char_p],
    "trn_function_set_rmsnorm": [vp, C.c_uint32, C.c_float],
    "trn_function_set_attention": [vp, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_float],
    "trn_mem_alloc": [C.POINTER(dptr), C.c_size_t],
    "trn_mem_free": [dptr],
    "trn_memcpy_htod": [dptr, vp, C.c_size_t],
    "trn_memcpy_dtoh": [vp, dptr, C.c_size_t],
    "trn_memcpy_htod_async": [dptr, vp, C.c_size_t, vp],
    "trn_memcpy_dtoh_async": [vp, dptr, C.c_size_t, vp],
    "trn_memcpy_dtod": [dptr, dptr, C.c_size_t],
    "trn_memcpy_dtod_async": [dptr, dptr, C.c_size_t, vp],
    "trn_mem_get_info": [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "trn_stream_create": [C.POINTER(vp), C.c_uint],
    "trn_stream_destroy": [vp],
    "trn_stream_synchronize": [vp],
    "trn_launch_kernel": [vp] + [C.c_uint] * 7 + [vp, C.POINTER(vp), C.POINTER(vp)],
    "trn_module_load_builtin": [C.POINTER(vp)],
    "trn_builtin_image": [C.POINTER(vp), C.POINTER(C.c_size_t)],
    "trn_q4k_gemv": [vp, dptr, dptr, dptr, C.c_uint32, C.c_uint32],
    "trn_q5k_gemv": [vp, dptr, dptr, dptr, C.c_uint32, C.c_uint32],
    "trn_q6k_gemv": [vp, dptr, dptr, dptr, C.c_uint32, C.c_uint32],
    "trn_q4k_gemm": [vp, dptr, dptr, dptr, C.c_uint32, C.c_uint32, C.c_uint32],
    "trn_q5k_gemm": [vp, dptr, dptr, dptr, C.c_uint32, C.c_uint32, C.c_uint32],
    "trn_q6k_gemm": [vp, dptr, dptr, dptr, C.c_uint32, C.c_uint32, C.c_uint32],
    "trn_q4k_gemm_as_written": [vp, dptr, dptr, dptr, C.c_uint32, C.c_uint32, C.c_uint32],
    "trn_q5k_gemm_as_written": [vp, dptr, dptr, dptr, C.c_uint32, C.c_uint32, C.c_uint32],
    "trn_q6k_gemm_as_written": [vp, dptr, dptr, dptr, C.c_uint32, C.c_uint32, C.c_uint32],
    "trn_q4k_gemm_noalloc": [vp, dptr, dptr, dptr, C.c_uint32, C.c_uint32, C.c_uint32],
    "trn_q4k_gemm_fused": [vp, dptr, dptr, dptr, C.c_uint32, C.c_uint32, C.c_uint32],
    "trn_gemv_f32": [vp, dptr, dptr, dptr, C.c_uint32, C.c_uint32],
    "trn_q5k_from_ggml": [vp, dptr, dptr, C.c_uint64],
    "trn_incremental_attention": [vp, dptr, dptr, dptr, dptr, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_float],
    "trn_residual_add": [vp, dptr, dptr, dptr, C.c_uint32],
    "trn_fused_swiglu": [vp, dptr, dptr, dptr, C.c_uint32],
    "trn_rmsnorm": [vp, dptr, dptr, dptr, C.c_uint32, C.c_float],
    "trn_fused_residual_rmsnorm": [vp, dptr, dptr, dptr, dptr, C.c_uint32, C.c_float],
    "trn_kquant_gemv_batch": [vp, vp, C.c_uint32],
    "trn_kquant_gemv_plan": [vp, C.c_uint32, vp],
    "trn_q4k_dequant_f32": [vp, dptr, dptr, C.c_uint64, C.c_int],
    "trn_q5k_dequant_f32": [vp, dptr, dptr, C.c_uint64, C.c_int],
    "trn_q6k_dequant_f32": [vp, dptr, dptr, C.c_uint64, C.c_int],
    "trn_q4k_simplified_dequant_f32": [vp, dptr, dptr, C.c_uint64],
    "trn_event_create": [C.POINTER(vp)],
    "trn_event_destroy": [vp],
    "trn_event_record": [vp, vp],
    "trn_event_synchronize": [vp],
    "trn_event_elapsed_ms": [C.POINTER(C.c_float), vp, vp],
    "trn_copy_u128": [vp, dptr, dptr, C.c_uint64],
    "trn_read_u128": [vp, dptr, C.c_uint64, dptr],
    "trn_error_name": [status],
    "trn_error_string": [status],
    "trn_device_cu_count": [C.POINTER(C.c_int)],
    "trn_set_tuning": [C.c_char_p, C.c_int],
}
_RESTYPE = {"trn_error_name": C.c_char_p, "trn_error_string": C.c_char_p}


class GemvDesc(C.Structure):
    """trn_gemv_desc"""
    _fields_ = [("fmt", C.c_uint32), ("k", C.c_uint32), ("n", C.c_uint32), ("flags", C.c_uint32),
                ("y", C.c_uint64), ("w", C.c_uint64), ("x", C.c_uint64),
                ("gamma", C.c_uint64), ("x2", C.c_uint64), ("residual", C.c_uint64),
                ("norm_eps", C.c_float), ("reserved", C.c_uint32)]


class LibraryMissing(OSError):
    pass


def lib() -> C.CDLL:
    """The loaded library.  Raises LibraryMissing if it has not been built
    (build it with `make -C trueno_amd/csrc` or __graft_entry__.build())."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryMissing(f"{LIB_PATH} is not built; run `make -C {os.path.join(_HERE, 'csrc')}`")
        L = C.CDLL(LIB_PATH)
        for name, args in SIGNATURES.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = _RESTYPE.get(name, status)
        _lib = L
    return _lib
