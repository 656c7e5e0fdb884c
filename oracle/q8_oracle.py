"""ctypes binding of oracle/q8_oracle.c (numpy in, numpy out).

Test infrastructure only: imported by tests/, by the smoke check and by the
bench's cpu_baseline leg, never by the shipped GPU path.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libq8oracle.so")

QK = 32
Q8_0_BYTES = 34
Q8_1_BYTES = 36
D4_BYTES = 144

PAIR_DTYPE = np.dtype([("value", np.float32), ("index", np.int32)])


def build(force=False):
    """Compile the oracle with the Makefile beside it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)


class _Pair(C.Structure):
    _fields_ = [("value", C.c_float), ("index", C.c_int32)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        u8p, f32p, u16p, u32p, i32p = (C.POINTER(t) for t in
                                       (C.c_uint8, C.c_float, C.c_uint16, C.c_uint32, C.c_int32))
        u32, u64, i32 = C.c_uint32, C.c_uint64, C.c_int
        sig = {
            "q8o_f32_to_f16": (C.c_uint16, [C.c_float]),
            "q8o_f16_to_f32": (C.c_float, [C.c_uint16]),
            "q8o_f32_to_bf16": (C.c_uint16, [C.c_float]),
            "q8o_bf16_to_f32": (C.c_float, [C.c_uint16]),
            "q8o_quantize_q8_0": (i32, [f32p, u64, u64, u8p]),
            "q8o_repack_split_plane": (i32, [u8p, u64, u64, u8p]),
            "q8o_get_row": (i32, [u8p, u64, u64, f32p]),
            "q8o_rms_norm": (i32, [f32p, f32p, f32p, u32, u32, u32, u32, C.c_float]),
            "q8o_quantize_q8_1": (i32, [f32p, u32, u32, u32, u8p]),
            "q8o_quantize_q8_1_d4": (i32, [f32p, u32, u32, u32, u8p]),
            "q8o_block_dot": (C.c_int32, [u8p, u8p, i32, u32, u32, u32, u32, u32]),
            "q8o_gemv": (i32, [u8p, u8p, f32p, u32, u32, u32, u32, i32]),
            "q8o_gemv_abs": (i32, [u8p, u8p, f32p, u32, u32, u32, u32]),
            "q8o_gemv_bf16": (i32, [u8p, u8p, u16p, u32, u32, u32, u32]),
            "q8o_gemv_two": (i32, [u8p, u8p, u8p, f32p, f32p, u32, u32, u32, u32]),
            "q8o_gemv_silu_mul": (i32, [u8p, u8p, u8p, f32p, u32, u32, u32, u32]),
            "q8o_gemv_add": (i32, [u8p, u8p, f32p, u32, u32, u32, u32]),
            "q8o_gemv_add_bf16": (i32, [u8p, u8p, u16p, u32, u32, u32, u32]),
            "q8o_gemv_fanout4": (i32, [C.POINTER(u8p), u8p, C.POINTER(f32p), u32p, u32, u32, u32p]),
            "q8o_gemm_d4": (i32, [u8p, u8p, f32p, u32, u32, u32, u32, i32]),
            "q8o_gemm_d4_sampled": (i32, [u8p, u8p, u32, u32, u32, u32p, u32p, u32, f32p, f32p]),
            "q8o_argmax_row": (_Pair, [f32p, u64]),
            "q8o_argmax_rows": (i32, [f32p, u32, u32, C.POINTER(_Pair)]),
            "q8o_argmax_rows_scan": (None, [f32p, u32, u32, C.POINTER(_Pair)]),
            "q8o_accept": (u32, [i32p, i32p, u32, C.c_int32, i32p]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def _p(a, ctype):
    return a.ctypes.data_as(C.POINTER(ctype))


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


# ---- conversions ---------------------------------------------------------
def f32_to_f16(v):
    return lib().q8o_f32_to_f16(float(np.float32(v)))


def f32_to_f16_bits(f32_bits):
    """Bit-level entry: uint32 fp32 pattern -> uint16 fp16 pattern."""
    return lib().q8o_f32_to_f16(C.c_float.from_buffer_copy(np.uint32(f32_bits).tobytes()))


def f16_to_f32(h):
    return np.float32(lib().q8o_f16_to_f32(int(h)))


def f32_to_bf16(v):
    return lib().q8o_f32_to_bf16(float(np.float32(v)))


def bf16_to_f32(h):
    return np.float32(lib().q8o_bf16_to_f32(int(h)))


# ---- weights --------------------------------------------------------------
def quantize_q8_0(w):
    """fp32 [rows, cols] -> interleaved GGUF Q8_0 bytes [rows, cols/32*34]."""
    w = _c(w, np.float32)
    rows, cols = w.shape
    out = np.empty((rows, cols // QK * Q8_0_BYTES), np.uint8)
    rc = lib().q8o_quantize_q8_0(_p(w, C.c_float), rows, cols, _p(out, C.c_uint8))
    if rc != 0:
        raise ValueError("q8o_quantize_q8_0 rejected the shape")
    return out


def repack_split_plane(gguf, rows, cols):
    gguf = _c(gguf, np.uint8)
    out = np.empty((rows, cols // QK * Q8_0_BYTES), np.uint8)
    rc = lib().q8o_repack_split_plane(_p(gguf, C.c_uint8), rows, cols, _p(out, C.c_uint8))
    if rc != 0:
        raise ValueError("q8o_repack_split_plane rejected the shape")
    return out


def get_row(w, row, cols):
    w = _c(w, np.uint8)
    out = np.empty(cols, np.float32)
    rc = lib().q8o_get_row(_p(w, C.c_uint8), row, cols, _p(out, C.c_float))
    if rc != 0:
        raise ValueError("q8o_get_row rejected the shape")
    return out


def make_weight(w):
    """fp32 [rows, cols] -> split-plane device-layout bytes."""
    g = quantize_q8_0(w)
    return repack_split_plane(g, w.shape[0], w.shape[1])


# ---- activations ----------------------------------------------------------
def rms_norm(x, weight, eps, cols=None, stride=None):
    """Rows of x ([batch, stride] fp32) normalised over their first `cols` columns."""
    x = _c(np.atleast_2d(x), np.float32)
    weight = _c(weight, np.float32)
    batch = x.shape[0]
    stride = x.shape[1] if stride is None else stride
    cols = x.shape[1] if cols is None else cols
    out = np.zeros((batch, cols), np.float32)
    rc = lib().q8o_rms_norm(_p(x, C.c_float), _p(weight, C.c_float), _p(out, C.c_float), batch, cols, stride,
                            cols, float(eps))
    if rc != 0:
        raise ValueError("q8o_rms_norm rejected the shape")
    return out


def quantize_q8_1(x, cols=None, stride=None):
    x = _c(x, np.float32)
    batch = x.shape[0]
    stride = x.shape[1] if stride is None else stride
    cols = x.shape[1] if cols is None else cols
    out = np.zeros(batch * (cols // QK) * Q8_1_BYTES if cols % QK == 0 else 0, np.uint8)
    rc = lib().q8o_quantize_q8_1(_p(x, C.c_float), batch, cols, stride, _p(out, C.c_uint8))
    return rc, out


def quantize_q8_1_d4(x, cols=None, stride=None):
    x = _c(x, np.float32)
    batch = x.shape[0]
    stride = x.shape[1] if stride is None else stride
    cols = x.shape[1] if cols is None else cols
    out = np.zeros((cols // 128) * batch * D4_BYTES if cols % 128 == 0 else 0, np.uint8)
    rc = lib().q8o_quantize_q8_1_d4(_p(x, C.c_float), batch, cols, stride, _p(out, C.c_uint8))
    return rc, out


def block_dot(w, y, layout, cols, batch, row, j, kb):
    return lib().q8o_block_dot(_p(w, C.c_uint8), _p(y, C.c_uint8), layout, cols, batch, row, j, kb)


# ---- GEMV family ------------------------------------------------------------
def gemv(w, y, rows, cols, batch, stride=None, threads=1):
    stride = rows if stride is None else stride
    dst = np.zeros(batch * stride, np.float32)
    rc = lib().q8o_gemv(_p(w, C.c_uint8), _p(y, C.c_uint8), _p(dst, C.c_float), rows, cols, batch,
                        stride, threads)
    return rc, dst.reshape(batch, stride)


def gemv_abs(w, y, rows, cols, batch, stride=None):
    """sum_kb |d_w*d_x*S| per output (the allowance scale for reordered sums)."""
    stride = rows if stride is None else stride
    dst = np.zeros(batch * stride, np.float32)
    rc = lib().q8o_gemv_abs(_p(w, C.c_uint8), _p(y, C.c_uint8), _p(dst, C.c_float), rows, cols,
                            batch, stride)
    return rc, dst.reshape(batch, stride)


def gemv_bf16(w, y, rows, cols, batch, stride=None):
    stride = rows if stride is None else stride
    dst = np.zeros(batch * stride, np.uint16)
    rc = lib().q8o_gemv_bf16(_p(w, C.c_uint8), _p(y, C.c_uint8), _p(dst, C.c_uint16), rows, cols,
                             batch, stride)
    return rc, dst.reshape(batch, stride)


def gemv_two(w0, w1, y, rows, cols, batch, stride=None):
    stride = rows if stride is None else stride
    d0 = np.zeros(batch * stride, np.float32)
    d1 = np.zeros(batch * stride, np.float32)
    rc = lib().q8o_gemv_two(_p(w0, C.c_uint8), _p(w1, C.c_uint8), _p(y, C.c_uint8),
                            _p(d0, C.c_float), _p(d1, C.c_float), rows, cols, batch, stride)
    return rc, d0.reshape(batch, stride), d1.reshape(batch, stride)


def gemv_silu_mul(wg, wu, y, rows, cols, batch, stride=None):
    stride = rows if stride is None else stride
    dst = np.zeros(batch * stride, np.float32)
    rc = lib().q8o_gemv_silu_mul(_p(wg, C.c_uint8), _p(wu, C.c_uint8), _p(y, C.c_uint8),
                                 _p(dst, C.c_float), rows, cols, batch, stride)
    return rc, dst.reshape(batch, stride)


def gemv_add(w, y, dst, rows, cols, batch, stride=None):
    stride = rows if stride is None else stride
    dst = np.array(dst, np.float32).reshape(-1).copy()
    rc = lib().q8o_gemv_add(_p(w, C.c_uint8), _p(y, C.c_uint8), _p(dst, C.c_float), rows, cols,
                            batch, stride)
    return rc, dst.reshape(batch, stride)


def gemv_add_bf16(w, y, dst, rows, cols, batch, stride=None):
    stride = rows if stride is None else stride
    dst = np.array(dst, np.uint16).reshape(-1).copy()
    rc = lib().q8o_gemv_add_bf16(_p(w, C.c_uint8), _p(y, C.c_uint8), _p(dst, C.c_uint16), rows,
                                 cols, batch, stride)
    return rc, dst.reshape(batch, stride)


def gemv_fanout4(ws, y, rows, cols, batch, strides=None):
    """ws: list of 4 arrays or None; rows: list of 4 ints."""
    u8p, f32p = C.POINTER(C.c_uint8), C.POINTER(C.c_float)
    strides = list(rows) if strides is None else list(strides)
    outs = [np.zeros(batch * max(strides[i], 1), np.float32) for i in range(4)]
    wa = (u8p * 4)(*[(_p(ws[i], C.c_uint8) if ws[i] is not None else u8p()) for i in range(4)])
    da = (f32p * 4)(*[(_p(outs[i], C.c_float) if ws[i] is not None else f32p()) for i in range(4)])
    ra = (C.c_uint32 * 4)(*rows)
    sa = (C.c_uint32 * 4)(*strides)
    rc = lib().q8o_gemv_fanout4(wa, _p(y, C.c_uint8), da, ra, cols, batch, sa)
    return rc, [outs[i].reshape(batch, max(strides[i], 1)) for i in range(4)]


# ---- GEMM ------------------------------------------------------------------
def gemm_d4(w, y, rows, cols, batch, stride=None, threads=1):
    stride = rows if stride is None else stride
    dst = np.zeros(batch * stride, np.float32)
    rc = lib().q8o_gemm_d4(_p(w, C.c_uint8), _p(y, C.c_uint8), _p(dst, C.c_float), rows, cols,
                           batch, stride, threads)
    return rc, dst.reshape(batch, stride)


def gemm_d4_sampled(w, y, rows, cols, batch, rows_idx, js_idx):
    rows_idx = _c(rows_idx, np.uint32)
    js_idx = _c(js_idx, np.uint32)
    out = np.zeros(len(rows_idx), np.float32)
    out_abs = np.zeros(len(rows_idx), np.float32)
    rc = lib().q8o_gemm_d4_sampled(_p(w, C.c_uint8), _p(y, C.c_uint8), rows, cols, batch,
                                   _p(rows_idx, C.c_uint32), _p(js_idx, C.c_uint32),
                                   len(rows_idx), _p(out, C.c_float), _p(out_abs, C.c_float))
    return rc, out, out_abs


# ---- argmax / accept ---------------------------------------------------------
def argmax_row(x):
    x = _c(x, np.float32).reshape(-1)
    r = lib().q8o_argmax_row(_p(x, C.c_float), x.size)
    return np.float32(r.value), int(r.index)


def argmax_rows(x, batch, row_stride):
    x = _c(x, np.float32).reshape(-1)
    out = np.zeros(batch, PAIR_DTYPE)
    rc = lib().q8o_argmax_rows(_p(x, C.c_float), batch, row_stride,
                               out.ctypes.data_as(C.POINTER(_Pair)))
    return rc, out


def argmax_rows_scan(x, batch, row_stride):
    x = _c(x, np.float32).reshape(-1)
    out = np.zeros(batch, PAIR_DTYPE)
    lib().q8o_argmax_rows_scan(_p(x, C.c_float), batch, row_stride,
                               out.ctypes.data_as(C.POINTER(_Pair)))
    return out


def accept(row_tokens, drafts, eos):
    row_tokens = _c(row_tokens, np.int32)
    drafts = _c(drafts, np.int32)
    nxt = C.c_int32(0)
    n = lib().q8o_accept(_p(row_tokens, C.c_int32), _p(drafts, C.c_int32), len(drafts), eos,
                         C.byref(nxt))
    return int(n), int(nxt.value)
