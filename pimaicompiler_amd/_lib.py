"""ctypes binding of libpimhip.so (the C ABI declared in include/pimhip.h).

The library is loaded from this package directory only.  There is no fallback: if the shared object is
missing or an entry point is absent, importing callers get an ImportError / AttributeError.
"""
import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libpimhip.so")

c_void_pp = ctypes.POINTER(ctypes.c_void_p)
c_int64_p = ctypes.POINTER(ctypes.c_int64)
c_int_p = ctypes.POINTER(ctypes.c_int)

# name -> (restype, argtypes); must list every function include/pimhip.h declares.
SIGNATURES = {
    "pimhip_initialize": (ctypes.c_int, [ctypes.c_int]),
    "pimhip_deinitialize": (ctypes.c_int, []),
    "pimhip_last_error": (ctypes.c_char_p, []),
    "pimhip_gemm_broadcast": (ctypes.c_int, [c_int64_p, c_int_p, c_int64_p, c_int_p]),
    "pimhip_get_gemm_type": (ctypes.c_int, [c_int64_p, c_int64_p, c_int_p]),
    "pimhip_execute_gemv": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                                           ctypes.c_int, ctypes.c_void_p]),
    "pimhip_execute_gemv_static": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                  ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                                                  ctypes.c_int, ctypes.c_void_p]),
    "pimhip_execute_gemv_scaled": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                                  ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float,
                                                  ctypes.c_void_p]),
    "pimhip_execute_gemv_cat2": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64,
                                                ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                                                ctypes.c_void_p]),
    "pimhip_probe_stream_read": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]),
    "pimhip_probe_xcc_map": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "pimhip_gemv_status": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]),
    "pimhip_gemv_fallbacks": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64)]),
    "pimhip_set_gemv_spin_limit": (ctypes.c_int, [ctypes.c_uint]),
    "pimhip_execute_dot": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                          ctypes.c_void_p]),
    "pimhip_execute_gemv_group": (ctypes.c_int, [ctypes.c_int, c_void_pp, c_void_pp, c_void_pp, c_void_pp,
                                                 c_int64_p, c_int64_p, c_int_p, ctypes.c_void_p]),
    "pimhip_execute_bmm": (ctypes.c_int, [c_void_pp, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                          ctypes.c_int64, ctypes.c_void_p]),
    "pimhip_execute_add": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                          ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]),
    "pimhip_lstm_plan_create": (ctypes.c_int, [c_void_pp, c_void_pp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                               ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                               ctypes.c_void_p]),
    "pimhip_lstm_plan_destroy": (ctypes.c_int, [ctypes.c_void_p]),
    "pimhip_lstm_forward": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                           ctypes.c_void_p]),
    "pimhip_lstm_plan_status": (ctypes.c_int, [ctypes.c_void_p]),
    "pimhip_lstm_plan_fallbacks": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64), c_int_p]),
    "pimhip_lstm_plan_set_mode": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "pimhip_lstm_plan_set_residual": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "pimhip_lstm_plan_set_measure": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "pimhip_lstm_plan_measured_mode": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, c_int_p]),
    "pimhip_lstm_plan_set_spin_limit": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_uint]),
    "pimhip_decoder_plan_create": (ctypes.c_int, [c_void_pp, c_void_pp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                  ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
                                                  ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]),
    "pimhip_decoder_plan_destroy": (ctypes.c_int, [ctypes.c_void_p]),
    "pimhip_decoder_plan_set_encoder": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]),
    "pimhip_decoder_step": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_void_p, c_void_pp, c_void_pp, c_void_pp, c_void_pp, c_void_pp, c_void_pp,
                                           ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]),
    "pimhip_decoder_plan_status": (ctypes.c_int, [ctypes.c_void_p]),
    "pimhip_decoder_plan_fallbacks": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_int)]),
    "pimhip_decoder_plan_set_spin_limit": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_uint]),
    "pimhip_moe_plan_create": (ctypes.c_int, [c_void_pp, ctypes.c_void_p, ctypes.c_void_p, c_void_pp, c_void_pp, c_void_pp,
                                              c_void_pp, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                                              ctypes.c_int, ctypes.c_void_p]),
    "pimhip_moe_plan_destroy": (ctypes.c_int, [ctypes.c_void_p]),
    "pimhip_moe_ffn_step": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_void_p, ctypes.c_void_p]),
    "pimhip_moe_plan_status": (ctypes.c_int, [ctypes.c_void_p]),
    "pimhip_moe_plan_fallbacks": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64), c_int_p]),
    "pimhip_moe_plan_set_spin_limit": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_uint]),
    "pimhip_rnnt_plan_create": (ctypes.c_int, [c_void_pp, c_void_pp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
                                               ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                               ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]),
    "pimhip_rnnt_plan_destroy": (ctypes.c_int, [ctypes.c_void_p]),
    "pimhip_rnnt_step": (ctypes.c_int, [ctypes.c_void_p] * 9 + [ctypes.c_int, ctypes.c_void_p]),
    "pimhip_rnnt_greedy_decode": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64,
                                                 ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                 ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                 ctypes.c_void_p]),
    "pimhip_rnnt_plan_fallbacks": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64), c_int_p]),
    "pimhip_rnnt_plan_set_spin_limit": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_uint]),
    "pimhip_input_projection": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                               ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p]),
    "pimhip_projection_packed_bytes": (ctypes.c_int, [ctypes.c_int64, ctypes.c_int64, ctypes.POINTER(ctypes.c_uint64)]),
    "pimhip_pack_projection_weight": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                                     ctypes.c_void_p]),
    "pimhip_input_projection_packed": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                      ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p]),
}

# Status codes and enums of include/pimhip.h.
PIMHIP_OK = 0
PIMHIP_ERR_INVALID_ARGUMENT = 1
PIMHIP_ERR_UNSUPPORTED = 2
PIMHIP_ERR_HIP = 3
PIMHIP_ERR_NOT_INITIALIZED = 4
PIMHIP_ERR_TIMEOUT = 5
PIMHIP_ACT_NONE = 0
PIMHIP_ACT_RELU = 1
PIMHIP_I_X_W = 0
PIMHIP_W_X_I = 1
GEMM_UNKNOWN, GEMM_VV, GEMM_MV, GEMM_VM, GEMM_MM = 0, 1, 2, 3, 4

_lib = None


def load():
    """Loads libpimhip.so once and declares every prototype.  Raises ImportError if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is not built; run `python -m pimaicompiler_amd.build` (needs hipcc). "
            "There is no CPU fallback for this path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib
