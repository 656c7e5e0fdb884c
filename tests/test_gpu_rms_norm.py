"""GPU parity of the RMS norm in front of the quantizer: q8mi_rms_norm and
q8mi_rms_norm_quantize_q8_1 against the CPU oracle (bit-exact: same order of the sum of squares,
IEEE root and quotient), and the one-launch forms q8mi_nqgemv* against q8mi_rms_norm followed by
the matching q8mi_qgemv* call (bit-exact) and against the oracle's chain (tolerance of the GEMV)."""
import ctypes as C

import numpy as np
import pytest

import q8mi
from gpu_common import NULL, assert_close_fp32, dev
from q8mi import hip, ok
import q8mi_support as synth

pytestmark = pytest.mark.gpu

EPS = 1e-6


def rows_of(n, batch, seed, stride=None):
    rng = np.random.default_rng(seed)
    stride = n if stride is None else stride
    x = (rng.standard_normal((batch, stride)) * rng.uniform(0.05, 30.0, (batch, 1))).astype(np.float32)
    w = rng.uniform(0.2, 2.0, n).astype(np.float32) * rng.choice([-1.0, 1.0], n).astype(np.float32)
    return x, w


def u32(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


@pytest.mark.parametrize("n", [1, 3, 4, 31, 257, 1024, 1027, 5120, 6144, 6148, 17408, 40000])
@pytest.mark.parametrize("batch", [1, 5, 70])
def test_rms_norm_bits(gpu, oracle, n, batch):
    L = gpu.lib()
    stride = n + (8 if n % 4 == 0 else 3)
    x, w = rows_of(n, batch, seed=n + batch, stride=stride)
    ref = oracle.rms_norm(x, w, EPS, cols=n, stride=stride)
    dx, dw = dev(x), dev(w)
    out = hip.DeviceBuffer(4 * batch * n).fill(0xee)
    ok(L.q8mi_rms_norm(dx.ptr, dw.ptr, out.ptr, batch, n, stride, n, EPS, NULL), "rms_norm")
    hip.synchronize()
    got = out.download(np.float32).reshape(batch, n)
    assert np.array_equal(u32(got), u32(ref))


def test_rms_norm_unaligned_pointers_and_padded_output(gpu, oracle):
    L = gpu.lib()
    n, batch = 5120, 3
    x, w = rows_of(n, batch, seed=77)
    ref = oracle.rms_norm(x, w, EPS)
    # every pointer 4 bytes off a 16-byte boundary: the scalar-load variant
    bx = hip.DeviceBuffer(4 * (batch * n + 1)); bx.upload(x, 4)
    bw = hip.DeviceBuffer(4 * (n + 1)); bw.upload(w, 4)
    stride_out = n + 5
    bo = hip.DeviceBuffer(4 * (batch * stride_out + 1)).fill(0xee)
    ok(L.q8mi_rms_norm(bx.at(4), bw.at(4), bo.at(4), batch, n, n, stride_out, EPS, NULL), "rms_norm")
    hip.synchronize()
    got = bo.download(np.uint32)[1:].reshape(batch, stride_out)
    assert np.array_equal(got[:, :n], u32(ref))
    assert np.all(got[:, n:] == 0xeeeeeeee), "nothing is written between the rows"


@pytest.mark.parametrize("cols", [32, 256, 5120, 6144, 8192, 17408])
@pytest.mark.parametrize("batch", [1, 6, 67])
def test_rms_norm_quantize_bits(gpu, oracle, cols, batch):
    L = gpu.lib()
    stride = cols + 16
    x, w = rows_of(cols, batch, seed=3 * cols + batch, stride=stride)
    x[0, :32] = 0.0          # an all-zero block
    ref_n = oracle.rms_norm(x, w, EPS, cols=cols, stride=stride)
    rc, ref_y = oracle.quantize_q8_1(ref_n)
    assert rc == 0
    dx, dw = dev(x), dev(w)
    nbytes = L.q8mi_q8_1_scratch_bytes(batch, cols)
    for with_normalized in (True, False):
        y = hip.DeviceBuffer(nbytes).fill(0xee)
        nrm = hip.DeviceBuffer(4 * batch * cols).fill(0xee)
        ok(L.q8mi_rms_norm_quantize_q8_1(dx.ptr, dw.ptr, nrm.ptr if with_normalized else NULL, y.ptr, batch, cols,
                                         stride, cols, EPS, NULL), "rms_norm_quantize_q8_1")
        hip.synchronize()
        assert np.array_equal(y.download(np.uint8), ref_y)
        if with_normalized:
            assert np.array_equal(nrm.download(np.uint32), u32(ref_n).reshape(-1))
    # and it is what the two separate calls give
    nrm = hip.DeviceBuffer(4 * batch * cols)
    y2 = hip.DeviceBuffer(nbytes).fill(0xdd)
    ok(L.q8mi_rms_norm(dx.ptr, dw.ptr, nrm.ptr, batch, cols, stride, cols, EPS, NULL), "rms_norm")
    ok(L.q8mi_quantize_q8_1(nrm.ptr, y2.ptr, batch, cols, cols, NULL), "quantize_q8_1")
    hip.synchronize()
    assert np.array_equal(y2.download(np.uint8), ref_y)


def test_rms_norm_rejections(gpu):
    L = gpu.lib()
    b = hip.DeviceBuffer(4096)
    assert L.q8mi_rms_norm_quantize_q8_1(b.ptr, b.ptr, NULL, b.ptr, 1, 48, 48, 48, EPS, NULL) == q8mi.REJECTED
    assert L.q8mi_rms_norm(b.ptr, b.ptr, NULL, 1, 64, 64, 64, EPS, NULL) == q8mi.REJECTED
    assert L.q8mi_rms_norm(NULL, b.ptr, b.ptr, 1, 64, 64, 64, EPS, NULL) == q8mi.REJECTED
    ok(L.q8mi_rms_norm(b.ptr, b.ptr, b.ptr, 0, 64, 64, 64, EPS, NULL), "empty batch")


@pytest.mark.parametrize("rows,cols", [(333, 6144), (5120, 5120), (201, 4096), (100, 256), (77, 1024), (150, 2048), (91, 3072), (40, 2304)])
def test_nqgemv_equals_norm_then_qgemv(gpu, oracle, rows, cols):
    L = gpu.lib()
    w = synth.q8_0_weight(rows, cols, seed=rows + cols)
    x, nw = rows_of(cols, 1, seed=rows * 3 + cols)
    dw, dx, dnw = dev(w), dev(x), dev(nw)
    nrm2 = hip.DeviceBuffer(4 * cols)
    two = hip.DeviceBuffer(4 * rows).fill(0xff)
    ok(L.q8mi_rms_norm(dx.ptr, dnw.ptr, nrm2.ptr, 1, cols, cols, cols, EPS, NULL), "rms_norm")
    ok(L.q8mi_qgemv(dw.ptr, nrm2.ptr, cols, two.ptr, 0, rows, cols, 1, rows, NULL), "qgemv")
    for with_normalized in (True, False):
        nrm1 = hip.DeviceBuffer(4 * cols).fill(0xee)
        one = hip.DeviceBuffer(4 * rows).fill(0xee)
        ok(L.q8mi_nqgemv(dw.ptr, dx.ptr, dnw.ptr, EPS, nrm1.ptr if with_normalized else NULL, one.ptr, 0, rows, cols,
                         1, NULL), "nqgemv")
        hip.synchronize()
        assert np.array_equal(one.download(np.uint32), two.download(np.uint32))
        if with_normalized:
            assert np.array_equal(nrm1.download(np.uint32), nrm2.download(np.uint32))
    # against the oracle's chain
    ref_n = oracle.rms_norm(x, nw, EPS)
    assert np.array_equal(nrm2.download(np.uint32), u32(ref_n).reshape(-1))
    rc, y = oracle.quantize_q8_1(ref_n)
    rc, ref = oracle.gemv(w, y, rows, cols, 1)
    rc, absum = oracle.gemv_abs(w, y, rows, cols, 1)
    assert_close_fp32(one.download(np.float32), ref, absum, "nqgemv")
    # bf16 outputs
    one16, two16 = hip.DeviceBuffer(2 * rows).fill(0xee), hip.DeviceBuffer(2 * rows).fill(0xff)
    ok(L.q8mi_nqgemv(dw.ptr, dx.ptr, dnw.ptr, EPS, NULL, one16.ptr, 1, rows, cols, 1, NULL), "nqgemv bf16")
    y = hip.DeviceBuffer(L.q8mi_q8_1_scratch_bytes(1, cols))
    ok(L.q8mi_quantize_q8_1(nrm2.ptr, y.ptr, 1, cols, cols, NULL), "quantize")
    ok(L.q8mi_gemv_bf16(dw.ptr, y.ptr, two16.ptr, rows, cols, 1, rows, NULL), "gemv_bf16")
    hip.synchronize()
    assert np.array_equal(one16.download(np.uint16), two16.download(np.uint16))


def test_nqgemv_fanout4_and_silu_mul(gpu, oracle):
    L = gpu.lib()
    cols = 5120
    rows = (640, 128, 0, 136)
    x, nw = rows_of(cols, 1, seed=11)
    dx, dnw = dev(x), dev(nw)
    ws = [synth.q8_0_weight(max(r, 1), cols, seed=20 + i) for i, r in enumerate(rows)]
    dws = [dev(w) for w in ws]
    ref_n = oracle.rms_norm(x, nw, EPS)
    rc, y = oracle.quantize_q8_1(ref_n)
    nrm = hip.DeviceBuffer(4 * cols).fill(0xee)
    outs = [hip.DeviceBuffer(4 * max(r, 1)).fill(0xee) for r in rows]
    ok(L.q8mi_nqgemv_fanout4(dws[0].ptr, dws[1].ptr, dws[2].ptr, dws[3].ptr, dx.ptr, dnw.ptr, EPS, nrm.ptr,
                             outs[0].ptr, outs[1].ptr, outs[2].ptr, outs[3].ptr, rows[0], rows[1], rows[2], rows[3],
                             cols, 1, NULL), "nqgemv_fanout4")
    hip.synchronize()
    assert np.array_equal(nrm.download(np.uint32), u32(ref_n).reshape(-1))
    nrm2 = dev(ref_n)
    for i, r in enumerate(rows):
        if r == 0:
            assert np.all(outs[i].download(np.uint32) == 0xeeeeeeee)
            continue
        rc, ref = oracle.gemv(ws[i], y, r, cols, 1)
        rc, absum = oracle.gemv_abs(ws[i], y, r, cols, 1)
        assert_close_fp32(outs[i].download(np.float32), ref, absum, f"nqgemv_fanout4 slot {i}")
        two = hip.DeviceBuffer(4 * r)
        ok(L.q8mi_qgemv(dws[i].ptr, nrm2.ptr, cols, two.ptr, 0, r, cols, 1, r, NULL), "qgemv")
        hip.synchronize()
        # on this row length a row's sum does not depend on how the rows are cut into work items
        assert np.array_equal(outs[i].download(np.uint32), two.download(np.uint32)), f"slot {i} against qgemv"
    # the same fan-out in two launches gives the same bits
    two = [hip.DeviceBuffer(4 * max(r, 1)).fill(0xdd) for r in rows]
    ok(L.q8mi_qgemv_fanout4(dws[0].ptr, dws[1].ptr, dws[2].ptr, dws[3].ptr, nrm2.ptr, cols, two[0].ptr, two[1].ptr,
                            two[2].ptr, two[3].ptr, rows[0], rows[1], rows[2], rows[3], cols, 1, rows[0], rows[1],
                            rows[2], rows[3], NULL), "qgemv_fanout4")
    hip.synchronize()
    for i, r in enumerate(rows):
        if r:
            assert np.array_equal(outs[i].download(np.uint32), two[i].download(np.uint32))

    # SwiGLU
    r = 1000
    wg, wu = synth.q8_0_weight(r, cols, seed=31), synth.q8_0_weight(r, cols, seed=32)
    dwg, dwu = dev(wg), dev(wu)
    one, ref_dev = hip.DeviceBuffer(4 * r).fill(0xee), hip.DeviceBuffer(4 * r).fill(0xdd)
    ok(L.q8mi_nqgemv_silu_mul(dwg.ptr, dwu.ptr, dx.ptr, dnw.ptr, EPS, NULL, one.ptr, r, cols, 1, NULL), "nqgemv_silu_mul")
    ok(L.q8mi_qgemv_silu_mul(dwg.ptr, dwu.ptr, nrm2.ptr, cols, ref_dev.ptr, r, cols, 1, r, NULL), "qgemv_silu_mul")
    hip.synchronize()
    assert np.array_equal(one.download(np.uint32), ref_dev.download(np.uint32))
    rc, ref = oracle.gemv_silu_mul(wg, wu, y, r, cols, 1)
    got = one.download(np.float32)
    assert np.all(np.abs(got - ref.reshape(-1)) <= 2e-5 * np.abs(ref.reshape(-1)) + 1e-6)


def test_nqgemv_rejections(gpu):
    L = gpu.lib()
    w = dev(synth.q8_0_weight(64, 8192, seed=1))
    x = hip.DeviceBuffer(4 * 8192 * 2 + 16)
    out = hip.DeviceBuffer(4 * 64 * 2)
    args = lambda cols, batch, xp: (w.ptr, xp, x.ptr, EPS, NULL, out.ptr, 0, 64, cols, batch, NULL)
    assert L.q8mi_nqgemv(*args(8192, 1, x.ptr)) == q8mi.REJECTED      # row too long for the registers
    assert L.q8mi_nqgemv(*args(5120, 2, x.ptr)) == q8mi.REJECTED      # one row only
    assert L.q8mi_nqgemv(*args(5120, 1, x.at(4))) == q8mi.REJECTED    # vector loads need alignment
    assert L.q8mi_nqgemv(*args(5100, 1, x.ptr)) == q8mi.REJECTED      # cols % 32
    assert L.q8mi_nqgemv(*args(1056, 1, x.ptr)) == q8mi.REJECTED      # cols % 256 (weight planes off 16 bytes)
    assert L.q8mi_nqgemv(w.ptr, x.ptr, x.at(32768), EPS, x.ptr, out.ptr, 0, 64, 5120, 1, NULL) == q8mi.REJECTED  # in place


def test_rms_norm_in_place(gpu, oracle):
    """The stand-alone norm (with or without the quantizer) may overwrite its input, long rows included."""
    L = gpu.lib()
    for n in (5120, 17408):
        x, w = rows_of(n, 3, seed=n + 1)
        ref = oracle.rms_norm(x, w, EPS)
        rc, ref_y = oracle.quantize_q8_1(ref)
        dx, dw = dev(x), dev(w)
        ok(L.q8mi_rms_norm(dx.ptr, dw.ptr, dx.ptr, 3, n, n, n, EPS, NULL), "rms_norm in place")
        hip.synchronize()
        assert np.array_equal(dx.download(np.uint32), u32(ref).reshape(-1))
        dx = dev(x)
        y = hip.DeviceBuffer(L.q8mi_q8_1_scratch_bytes(3, n))
        ok(L.q8mi_rms_norm_quantize_q8_1(dx.ptr, dw.ptr, dx.ptr, y.ptr, 3, n, n, n, EPS, NULL), "in place")
        hip.synchronize()
        assert np.array_equal(dx.download(np.uint32), u32(ref).reshape(-1))
        assert np.array_equal(y.download(np.uint8), ref_y)


def test_rms_norm_non_finite_rows(gpu, oracle):
    """A NaN or an infinity in a row makes its scale NaN or zero; whatever comes out must be the
    oracle's bits (normalised values compared as bit patterns, NaNs as NaNs) and its Q8_1 bytes."""
    L = gpu.lib()
    n = 1024
    x, w = rows_of(n, 4, seed=5)
    x[0, 17] = np.nan
    x[1, 500] = np.inf
    x[2, :] = 0.0                      # a zero row: scale = 1/sqrt(eps), outputs zero
    x[3, 3] = -np.inf
    ref = oracle.rms_norm(x, w, EPS)
    rc, ref_y = oracle.quantize_q8_1(ref)
    dx, dw = dev(x), dev(w)
    nrm = hip.DeviceBuffer(4 * 4 * n)
    y = hip.DeviceBuffer(L.q8mi_q8_1_scratch_bytes(4, n))
    ok(L.q8mi_rms_norm_quantize_q8_1(dx.ptr, dw.ptr, nrm.ptr, y.ptr, 4, n, n, n, EPS, NULL), "rms_norm_quantize")
    hip.synchronize()
    got = nrm.download(np.float32).reshape(4, n)
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    keep = ~np.isnan(ref)
    assert np.array_equal(got[keep].view(np.uint32), ref[keep].view(np.uint32))
    assert np.all(got[2] == 0.0)
    # quants and the scale halfword of every block; the sum halfword of a NaN block may differ in payload only
    gy = y.download(np.uint8).reshape(-1, 36)
    ry = ref_y.reshape(-1, 36)
    assert np.array_equal(gy[:, 4:], ry[:, 4:])
    gd, rd = gy[:, :4].copy().view(np.float16), ry[:, :4].copy().view(np.float16)
    assert np.array_equal(np.isnan(gd), np.isnan(rd))
    assert np.array_equal(gd[~np.isnan(rd)], rd[~np.isnan(rd)])


@pytest.mark.parametrize("cols,batch,in_place", [(5120, 1, True), (5120, 8, True), (5120, 5, False), (6144, 3, True),
                                                 (8192, 2, True), (17408, 4, True), (40000, 2, False), (256, 7, True),
                                                 (1027, 3, True), (6148, 2, False), (5120, 300, True)])
def test_add_rms_norm_is_add_then_norm(gpu, oracle, cols, batch, in_place):
    """sum = a + b, then the norm (and the quantizer) of sum, in one launch: the bits of q8mi_add followed
    by q8mi_rms_norm / q8mi_rms_norm_quantize_q8_1, and of the oracle's chain; in place (sum = a) and out
    of place, rows held in registers and rows read twice, vector and scalar loads."""
    L = gpu.lib()
    a, w = rows_of(cols, batch, seed=7 * cols + batch)
    b, _ = rows_of(cols, batch, seed=11 * cols + batch)
    if cols % 32 == 0:
        a[0, :32] = 0.0
        b[0, :32] = 0.0      # an all-zero block after the add
    ref_sum = (a + b).astype(np.float32)
    ref_n = oracle.rms_norm(ref_sum, w, EPS)
    dw, db = dev(w), dev(b)
    quant = cols % 32 == 0
    nbytes = L.q8mi_q8_1_scratch_bytes(batch, cols) if quant else 16
    for with_normalized in ((True, False) if quant else (True,)):
        da = dev(a)
        dsum = da if in_place else hip.DeviceBuffer(4 * batch * cols).fill(0xee)
        nrm = hip.DeviceBuffer(4 * batch * cols).fill(0xee)
        y = hip.DeviceBuffer(nbytes).fill(0xee)
        ok(L.q8mi_add_rms_norm(da.ptr, db.ptr, dsum.ptr, dw.ptr, nrm.ptr if with_normalized else NULL,
                               y.ptr if quant else NULL, batch, cols, cols, cols, EPS, NULL), "add_rms_norm")
        hip.synchronize()
        assert np.array_equal(dsum.download(np.uint32), u32(ref_sum).reshape(-1)), "the sum"
        if not in_place:
            assert np.array_equal(da.download(np.uint32), u32(a).reshape(-1)), "a is left alone"
        if with_normalized:
            assert np.array_equal(nrm.download(np.uint32), u32(ref_n).reshape(-1)), "the normalised rows"
        if quant:
            rc, ref_y = oracle.quantize_q8_1(ref_n)
            assert rc == 0 and np.array_equal(y.download(np.uint8), ref_y), "the Q8_1 blocks"
    # the two launches it replaces
    da2 = dev(a)
    nrm2 = hip.DeviceBuffer(4 * batch * cols)
    ok(L.q8mi_add(da2.ptr, da2.ptr, db.ptr, batch * cols, 0, NULL), "add")
    ok(L.q8mi_rms_norm(da2.ptr, dw.ptr, nrm2.ptr, batch, cols, cols, cols, EPS, NULL), "rms_norm")
    hip.synchronize()
    assert np.array_equal(da2.download(np.uint32), u32(ref_sum).reshape(-1))
    assert np.array_equal(nrm2.download(np.uint32), u32(ref_n).reshape(-1))


def test_add_rms_norm_rejections(gpu):
    L = gpu.lib()
    b, c, d = hip.DeviceBuffer(4096), hip.DeviceBuffer(4096), hip.DeviceBuffer(4096)
    assert L.q8mi_add_rms_norm(b.ptr, c.ptr, b.ptr, c.ptr, NULL, NULL, 1, 64, 64, 64, EPS, NULL) == q8mi.REJECTED   # no output
    assert L.q8mi_add_rms_norm(b.ptr, c.ptr, b.ptr, c.ptr, b.ptr, NULL, 1, 64, 64, 64, EPS, NULL) == q8mi.REJECTED  # normalised over the sum
    assert L.q8mi_add_rms_norm(b.ptr, c.ptr, b.ptr, c.ptr, NULL, d.ptr, 1, 48, 48, 48, EPS, NULL) == q8mi.REJECTED  # Q8_1 of 48 columns
    assert L.q8mi_add_rms_norm(NULL, c.ptr, b.ptr, c.ptr, d.ptr, NULL, 1, 64, 64, 64, EPS, NULL) == q8mi.REJECTED
    ok(L.q8mi_add_rms_norm(b.ptr, c.ptr, b.ptr, c.ptr, d.ptr, NULL, 0, 64, 64, 64, EPS, NULL), "empty batch")
