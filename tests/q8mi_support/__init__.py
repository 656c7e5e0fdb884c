"""Instruments of the tests and the bench: seeded synthetic inputs, the int32 block-dot checker and
the kernels that measured ceilings come from (libq8mi_support.so, see q8mi_support.h beside this
file).  Not part of the product: libq8mi.so exports none of this and the package never imports it."""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libq8mi_support.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

_vp, _u32, _u64, _int = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int
SIGNATURES = {
    "q8sup_last_error": (C.c_char_p, []),
    "q8sup_synth_f32": (_int, [_vp, _u64, _u64, _u64, _int, C.c_float, _u32, C.c_float, _int]),
    "q8sup_synth_q8_0_weight": (_int, [_vp, _u64, _u64, _u64, C.c_float, _int]),
    "q8sup_block_dots": (_int, [_vp, _vp, _int, _u32, _u32, _u32, _vp, _vp, _vp, _u32, _vp, _vp]),
    "q8sup_probe_read": (_int, [_vp, _u64, _u32, _vp, _vp]),
    "q8sup_probe_copy": (_int, [_vp, _vp, _u64, _vp]),
    "q8sup_probe_mfma": (_int, [_int, _u32, _vp, C.POINTER(C.c_uint64), _vp]),
    "q8sup_probe_mfma_sink_bytes": (C.c_size_t, []),
}

_lib = None


def build():
    """Compile libq8mi_support.so for gfx950 (same device flags as the product library)."""
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra",
           "-Wno-unused-command-line-argument", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           os.path.join(HERE, "q8mi_support.hip"), "-o", LIB_PATH, "-lpthread"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on q8mi_support.hip:\n" + r.stdout + r.stderr)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; g.build()')")
        L = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def ok(rc, what=""):
    if rc != 0:
        m = lib().q8sup_last_error()
        raise RuntimeError(f"{what}: rc={rc} ({m.decode() if m else ''})")
    return rc


def _threads(threads):
    if threads is None:
        threads = min(16, os.cpu_count() or 1)
    return int(threads)


def normal(rows, cols, seed, scale=1.0, threads=None):
    out = np.empty((rows, cols), np.float32)
    ok(lib().q8sup_synth_f32(out.ctypes.data_as(C.c_void_p), rows, cols, seed, 0, scale, 0, 1.0, _threads(threads)),
       "synth_f32")
    return out


def student_t3(rows, cols, seed, scale=1.0, outlier_ppm=1000, outlier_gain=20.0, threads=None):
    """Unit-variance Student-t(nu=3) with a seeded set of outlier columns (benchmark config 4: 0.1 % of the
    channels at 20 x)."""
    out = np.empty((rows, cols), np.float32)
    ok(lib().q8sup_synth_f32(out.ctypes.data_as(C.c_void_p), rows, cols, seed, 1, scale, outlier_ppm, outlier_gain,
                             _threads(threads)), "synth_f32")
    return out


def q8_0_weight(rows, cols, seed, sigma=0.02, threads=None):
    """N(0, sigma^2) weights, Q8_0-quantized, in split-plane device layout (uint8 [rows, cols/32*34])."""
    out = np.empty((rows, cols // 32 * 34), np.uint8)
    ok(lib().q8sup_synth_q8_0_weight(out.ctypes.data_as(C.c_void_p), rows, cols, seed, sigma, _threads(threads)),
       "synth_q8_0_weight")
    return out
