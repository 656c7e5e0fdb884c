"""Python face of libq8mi.so, the gfx950 Q8_0 x Q8_1 quantized-linear library.

Thin ctypes declarations of every entry point in include/q8mi.h.  This module
never computes anything itself: if the shared library is missing it raises, so
a GPU run cannot silently pass on some other path.
"""
import ctypes as C
import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libq8mi.so")

OK, REJECTED, LAUNCH_ERROR = 0, 1, 2
QK = 32
Q8_0_BYTES = 34
Q8_1_BYTES = 36
D4_BYTES = 144
MAX_GEMV_BATCH = 8


class ArgmaxPair(C.Structure):
    _fields_ = [("value", C.c_float), ("index", C.c_int32)]


_u8p = C.c_void_p  # device pointers travel as plain addresses
_vp = C.c_void_p
_u32 = C.c_uint32
_u64 = C.c_uint64
_int = C.c_int

# name -> (restype, argtypes); mirrors include/q8mi.h one to one
SIGNATURES = {
    "q8mi_last_error": (C.c_char_p, []),
    "q8mi_abi_version": (_int, []),
    "q8mi_q8_1_scratch_bytes": (C.c_size_t, [_u32, _u32]),
    "q8mi_quantize_q8_1": (_int, [_vp, _vp, _u32, _u32, _u32, _vp]),
    "q8mi_gemv": (_int, [_u8p, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_gemv_bf16": (_int, [_u8p, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_gemv_two": (_int, [_u8p, _u8p, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_gemv_silu_mul": (_int, [_u8p, _u8p, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_gemv_add": (_int, [_u8p, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_gemv_add_bf16": (_int, [_u8p, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_gemv_fanout4": (_int, [_u8p] * 4 + [_vp] + [_vp] * 4 + [_u32] * 4 + [_u32, _u32] + [_u32] * 4 + [_vp]),
    "q8mi_q8_1_d4_scratch_bytes": (C.c_size_t, [_u32, _u32]),
    "q8mi_quantize_q8_1_d4": (_int, [_vp, _vp, _u32, _u32, _u32, _vp]),
    "q8mi_gemm": (_int, [_u8p, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_gemm_medium": (_int, [_u8p, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_gemm_add": (_int, [_u8p, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_gemm_bf16": (_int, [_u8p, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_gemm_silu_mul": (_int, [_u8p, _u8p, _vp, _vp, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_silu_mul": (_int, [_vp, _vp, _vp, _u64, _vp]),
    "q8mi_f32_to_bf16": (_int, [_vp, _vp, _u64, _vp]),
    "q8mi_add": (_int, [_vp, _vp, _vp, _u64, _int, _vp]),
    "q8mi_get_row": (_int, [_u8p, _u64, _u64, _u64, _vp, _int, _vp]),
    "q8mi_get_row_from_argmax": (_int, [_u8p, _vp, _u32, _u64, _u64, _vp, _vp]),
    "q8mi_get_rows": (_int, [_u8p, _vp, _u32, _u64, _u64, _vp, _int, _vp]),
    "q8mi_argmax": (_int, [_vp, _u64, _vp, _vp]),
    "q8mi_argmax_to_pair": (_int, [_vp, _u64, _vp, _u32, _vp]),
    "q8mi_argmax_rows_scratch_bytes": (C.c_size_t, [_u32, _u32]),
    "q8mi_argmax_rows": (_int, [_vp, _u32, _u32, _vp, _vp, _vp]),
    "q8mi_lm_head_scratch_bytes": (C.c_size_t, [_u32, _u32, _u32]),
    "q8mi_lm_head_argmax_accept": (_int, [_u8p, _vp, _u32, _u32, _u32, _vp, _int, C.c_int32, _vp, _vp, _vp,
                                          _u32, _vp, _vp]),
    "q8mi_lm_head_argmax_accept_static": (_int, [_u8p, _vp, _u32, _u32, _u32, _vp, _int, C.c_int32, _vp, _vp, _vp,
                                                 _u32, _vp]),
    "q8mi_repack_q8_0_split_host": (_int, [_vp, _u64, _u64, _vp]),
    "q8mi_repack_q8_0_split": (_int, [_vp, _u64, _u64, _vp, _vp]),
    "q8mi_qgemv": (_int, [_vp, _vp, _u32, _vp, _int, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_qgemv_add": (_int, [_vp, _vp, _u32, _vp, _int, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_qgemv_silu_mul": (_int, [_vp, _vp, _vp, _u32, _vp, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_qgemv_fanout4": (_int, [_vp, _vp, _vp, _vp, _vp, _u32, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32,
                                  _u32, _u32, _u32, _u32, _u32, _vp]),
    "q8mi_rms_norm": (_int, [_vp, _vp, _vp, _u32, _u32, _u32, _u32, C.c_float, _vp]),
    "q8mi_rms_norm_quantize_q8_1": (_int, [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, C.c_float, _vp]),
    "q8mi_add_rms_norm": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, C.c_float, _vp]),
    "q8mi_nqgemv": (_int, [_vp, _vp, _vp, C.c_float, _vp, _vp, _int, _u32, _u32, _u32, _vp]),
    "q8mi_nqgemv_silu_mul": (_int, [_vp, _vp, _vp, _vp, C.c_float, _vp, _vp, _u32, _u32, _u32, _vp]),
    "q8mi_nqgemv_fanout4": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, C.c_float, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32,
                                   _u32, _u32, _u32, _vp]),
}

_lib = None


class Q8miError(RuntimeError):
    pass


def lib():
    """The loaded library.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise Q8miError(
                f"{LIB_PATH} is missing: build it first (python kvmem-qw3_amd/q8mi/build.py); "
                "there is no fallback path")
        L = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def last_error():
    m = lib().q8mi_last_error()
    return m.decode() if m else ""


def ok(rc, what=""):
    """Raise unless rc is OK."""
    if rc != OK:
        raise Q8miError(f"{what}: rc={rc} ({last_error()})")
    return rc
