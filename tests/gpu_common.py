"""Helpers shared by the GPU parity tests: call the C ABI on device buffers."""
import ctypes as C

import numpy as np

import q8mi
from q8mi import hip, ok

NULL = C.c_void_p(0)


def dev(arr):
    return hip.to_device(np.ascontiguousarray(arr))


def quantize_q8_1(x, cols=None, stride=None, stream=NULL):
    """x: fp32 [batch, stride] on host -> (device Q8_1 buffer, host bytes)."""
    x = np.ascontiguousarray(x, np.float32)
    batch = x.shape[0]
    stride = x.shape[1] if stride is None else stride
    cols = x.shape[1] if cols is None else cols
    dx = dev(x)
    n = q8mi.lib().q8mi_q8_1_scratch_bytes(batch, cols)
    dy = hip.DeviceBuffer(n)
    ok(q8mi.lib().q8mi_quantize_q8_1(dx.ptr, dy.ptr, batch, cols, stride, stream), "quantize_q8_1")
    hip.synchronize()
    return dy, dy.download(np.uint8, n)


def quantize_d4(x, cols=None, stride=None, stream=NULL):
    x = np.ascontiguousarray(x, np.float32)
    batch = x.shape[0]
    stride = x.shape[1] if stride is None else stride
    cols = x.shape[1] if cols is None else cols
    dx = dev(x)
    n = q8mi.lib().q8mi_q8_1_d4_scratch_bytes(batch, cols)
    dy = hip.DeviceBuffer(n)
    ok(q8mi.lib().q8mi_quantize_q8_1_d4(dx.ptr, dy.ptr, batch, cols, stride, stream), "quantize_d4")
    hip.synchronize()
    return dy, dy.download(np.uint8, n)


# what -> {"n", "max_rel", "beyond_rel", "max_of_bound", "max_of_floor"}: filled by assert_close_fp32, written out as JSON when the
# test session ends (tests/conftest.py)
TOLERANCE_STATS = {}


def _record(what, err, ref, rel, lim, floor_term):
    """Per check family (the text of `what` up to its first digit): the largest relative error
    seen, how many outputs were beyond rel*|ref| alone, i.e. passed only through the
    sum|t_kb| term of the bound, the largest share of the whole bound any output used, and
    the largest error in units of the sum|t_kb| term (how much of that term is needed)."""
    key = what
    for i, ch in enumerate(what):
        if ch.isdigit():
            key = what[:i].rstrip(" ,=(")
            break
    live = np.abs(ref) > 0
    relerr = np.zeros_like(err)
    relerr[live] = err[live] / np.abs(ref[live])
    s = TOLERANCE_STATS.setdefault(key, {"n": 0, "max_rel": 0.0, "beyond_rel": 0, "max_of_bound": 0.0,
                                         "max_of_floor": 0.0})
    s["n"] += int(err.size)
    s["max_rel"] = max(s["max_rel"], float(relerr.max()) if err.size else 0.0)
    s["beyond_rel"] += int(np.count_nonzero(err > rel * np.abs(ref)))
    ok_lim, ok_floor = lim > 0, floor_term > 0
    if ok_lim.any():
        s["max_of_bound"] = max(s["max_of_bound"], float((err[ok_lim] / lim[ok_lim]).max()))
    if ok_floor.any():
        s["max_of_floor"] = max(s["max_of_floor"], float((err[ok_floor] / floor_term[ok_floor]).max()))


def assert_close_fp32(got, ref, absum, what, rel=1e-5, floor=1e-6):
    """|got - ref| <= rel*|ref| + floor*sum_kb|t_kb|.

    rel is the tolerance the task states for fp32 outputs (1e-5 relative to the
    CPU oracle, ascending block order).  The floor covers outputs whose blocks
    cancel: the GPU adds the same per-block terms in another order, and fp32
    reordering error scales with sum|t_kb|, not with |ref|.
    """
    got = np.asarray(got, np.float64).reshape(-1)
    ref = np.asarray(ref, np.float64).reshape(-1)
    absum = np.asarray(absum, np.float64).reshape(-1)
    err = np.abs(got - ref)
    lim = rel * np.abs(ref) + floor * absum
    _record(what, err, ref, rel, lim, floor * absum)
    bad = np.nonzero(~(err <= lim))[0]
    if bad.size:
        i = bad[0]
        raise AssertionError(
            f"{what}: {bad.size}/{got.size} outputs outside tolerance; first at {i}: "
            f"got {got[i]!r} ref {ref[i]!r} err {err[i]:.3e} lim {lim[i]:.3e}")
    return float((err / np.maximum(np.abs(ref), 1e-30)).max())
