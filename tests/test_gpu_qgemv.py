"""GPU parity: the GEMV entry points that quantize fp32 activations inside the kernel must give, at
batch 1 bit for bit, what q8mi_quantize_q8_1 followed by the matching GEMV gives (which the other
GPU tests hold against the CPU oracle).  At batch 2 the two routes may run different kernels (the
Q8_1 entry points go to the matrix cores when the launch has few row pairs), which changes the order
of the fp32 sums: there, and on rows above 8192 columns, the fused form is held against the oracle
directly."""
import numpy as np
import pytest

import q8mi
from gpu_common import NULL, assert_close_fp32, dev, quantize_q8_1
from q8mi import hip, ok
import q8mi_support as synth

pytestmark = pytest.mark.gpu


def bits(buf, n, dtype=np.uint32):
    hip.synchronize()
    return buf.download(dtype, n)


@pytest.mark.parametrize("rows,cols", [(33, 17408), (5120, 17408), (700, 12288)])
@pytest.mark.parametrize("batch", [1, 2])
def test_qgemv_long_rows_against_oracle(gpu, oracle, rows, cols, batch):
    L = gpu.lib()
    w = synth.q8_0_weight(rows, cols, seed=rows + cols)
    x = synth.normal(batch, cols, seed=batch * 31 + cols)
    x[0, 64:96] = 0.0
    dw, dx = dev(w), dev(x)
    n = batch * rows
    rc, y = oracle.quantize_q8_1(x)
    rc, ref = oracle.gemv(w, y, rows, cols, batch, threads=8)
    rc, absum = oracle.gemv_abs(w, y, rows, cols, batch)
    one = hip.DeviceBuffer(4 * n).fill(0xee)
    ok(L.q8mi_qgemv(dw.ptr, dx.ptr, cols, one.ptr, 0, rows, cols, batch, rows, NULL), "qgemv")
    hip.synchronize()
    assert_close_fp32(one.download(np.float32), ref, absum, "qgemv long rows")
    base = synth.normal(batch, rows, seed=6)
    acc = dev(base)
    ok(L.q8mi_qgemv_add(dw.ptr, dx.ptr, cols, acc.ptr, 0, rows, cols, batch, rows, NULL), "qgemv_add")
    hip.synchronize()
    assert_close_fp32(acc.download(np.float32), ref.reshape(-1) + base.reshape(-1),
                      absum.reshape(-1) + np.abs(base.reshape(-1)), "qgemv_add long rows")
    # and it is deterministic: a second launch gives the same bits
    two = hip.DeviceBuffer(4 * n).fill(0xdd)
    ok(L.q8mi_qgemv(dw.ptr, dx.ptr, cols, two.ptr, 0, rows, cols, batch, rows, NULL), "qgemv")
    assert np.array_equal(bits(one, n), bits(two, n))


@pytest.mark.parametrize("rows,cols", [(5120, 5120), (300, 2304 // 256 * 256), (129, 6144), (640, 8192), (64, 256)])
@pytest.mark.parametrize("batch", [1, 2, 3, 5, 8])
def test_qgemv_equals_two_step(gpu, oracle, rows, cols, batch):
    """The quantizer inside the GEMV, batch 1 and 2: the bits of quantizer + GEMV at batch 1 and, on
    rows of 4, 5, 6 and 8 KiB (both forms run the kernel whose waves share the rows), at batch 2;
    on other lengths at batch 2 each form is within the tolerance of the oracle.  Declined beyond."""
    L = gpu.lib()
    w = synth.q8_0_weight(rows, cols, seed=rows + cols)
    stride_x = cols + 8
    x = synth.normal(batch, stride_x, seed=batch * 77 + cols)
    x[0, :32] = 0.0                       # an all-zero block
    x[-1, 32:64] = 3000.0                 # a block whose sum overflows fp16 (sum is not used by the dots)
    dw, dx = dev(w), dev(x)
    dy, _ = quantize_q8_1(x, cols=cols, stride=stride_x)
    n = batch * rows
    two = hip.DeviceBuffer(4 * n).fill(0xff)
    one = hip.DeviceBuffer(4 * n).fill(0xee)
    ok(L.q8mi_gemv(dw.ptr, dy.ptr, two.ptr, rows, cols, batch, rows, NULL), "gemv")
    rc = L.q8mi_qgemv(dw.ptr, dx.ptr, stride_x, one.ptr, 0, rows, cols, batch, rows, NULL)
    shared_rows = cols in (4096, 5120, 6144, 8192)
    if batch > 2:
        assert rc == q8mi.REJECTED, "the fused form serves batch 1 and 2 only"
        return
    if rc == q8mi.REJECTED:
        # declined only when the staged activations (plus the per-wave result area) exceed LDS
        steps = (cols // 32 * 2 + 127) // 128
        assert batch * steps * 2304 + 16 * 4096 > 160 * 1024, "a shape that fits LDS must not be declined"
        return
    ok(rc, "qgemv")
    if batch == 2 and not shared_rows:
        hip.synchronize()
        y = dy.download(np.uint8, batch * (cols // 32) * 36)
        rc, ref = oracle.gemv(w, y, rows, cols, batch, threads=8)
        rc, absum = oracle.gemv_abs(w, y, rows, cols, batch)
        assert_close_fp32(one.download(np.float32), ref, absum, "qgemv batch 2")
        assert_close_fp32(two.download(np.float32), ref, absum, "gemv batch 2")
        return
    assert np.array_equal(bits(one, n), bits(two, n))
    # bf16 outputs
    two16, one16 = hip.DeviceBuffer(2 * n).fill(0xff), hip.DeviceBuffer(2 * n).fill(0xee)
    ok(L.q8mi_gemv_bf16(dw.ptr, dy.ptr, two16.ptr, rows, cols, batch, rows, NULL), "gemv_bf16")
    ok(L.q8mi_qgemv(dw.ptr, dx.ptr, stride_x, one16.ptr, 1, rows, cols, batch, rows, NULL), "qgemv bf16")
    assert np.array_equal(bits(one16, n, np.uint16), bits(two16, n, np.uint16))
    # residual add, fp32 and bf16
    base = synth.normal(batch, rows, seed=5)
    a2, a1 = dev(base), dev(base)
    ok(L.q8mi_gemv_add(dw.ptr, dy.ptr, a2.ptr, rows, cols, batch, rows, NULL), "gemv_add")
    ok(L.q8mi_qgemv_add(dw.ptr, dx.ptr, stride_x, a1.ptr, 0, rows, cols, batch, rows, NULL), "qgemv_add")
    assert np.array_equal(bits(a1, n), bits(a2, n))


@pytest.mark.parametrize("batch,rows,cols", [(1, 1000, 1024), (2, 8192, 1024), (1, 600, 5120), (2, 600, 5120)])
def test_qgemv_silu_and_fanout_equal_two_step(gpu, batch, rows, cols):
    L = gpu.lib()
    # 1024 columns at batch 2: rows enough that it stays on the row-pair kernels on both routes;
    # 5120 columns: a row length whose rows the waves of a workgroup share on both routes
    wg, wu = synth.q8_0_weight(rows, cols, seed=1), synth.q8_0_weight(rows, cols, seed=2)
    wk = synth.q8_0_weight(130, cols, seed=3)
    x = synth.normal(batch, cols, seed=40 + batch)
    dg, du, dk, dx = dev(wg), dev(wu), dev(wk), dev(x)
    dy, _ = quantize_q8_1(x)
    n = batch * rows
    two, one = hip.DeviceBuffer(4 * n).fill(0xff), hip.DeviceBuffer(4 * n).fill(0xee)
    ok(L.q8mi_gemv_silu_mul(dg.ptr, du.ptr, dy.ptr, two.ptr, rows, cols, batch, rows, NULL), "silu")
    ok(L.q8mi_qgemv_silu_mul(dg.ptr, du.ptr, dx.ptr, cols, one.ptr, rows, cols, batch, rows, NULL), "qsilu")
    assert np.array_equal(bits(one, n), bits(two, n))
    if batch == 2 and cols == 1024:
        return   # the fan-out below has too few row pairs for the row-pair kernels at batch 2
    outs2 = [hip.DeviceBuffer(4 * batch * r).fill(0xff) for r in (rows, 130, rows)]
    outs1 = [hip.DeviceBuffer(4 * batch * r).fill(0xee) for r in (rows, 130, rows)]
    for fn, xin, extra, outs in ((L.q8mi_gemv_fanout4, dy.ptr, (), outs2), (L.q8mi_qgemv_fanout4, dx.ptr, (cols,), outs1)):
        ok(fn(dg.ptr, dk.ptr, None, du.ptr, xin, *extra, outs[0].ptr, outs[1].ptr, None, outs[2].ptr,
              rows, 130, 0, rows, cols, batch, rows, 130, 0, rows, NULL), "fanout4")
    for o1, o2, r in zip(outs1, outs2, (rows, 130, rows)):
        assert np.array_equal(bits(o1, batch * r), bits(o2, batch * r))


def test_qgemv_rejections(gpu):
    L = gpu.lib()
    b = hip.DeviceBuffer(1 << 16)
    assert L.q8mi_qgemv(b.ptr, b.ptr, 96, b.ptr, 0, 4, 96, 1, 4, NULL) == q8mi.REJECTED      # cols % 256
    assert L.q8mi_qgemv(b.ptr, b.ptr, 256, b.ptr, 0, 4, 256, 9, 4, NULL) == q8mi.REJECTED    # batch > 8
    assert L.q8mi_qgemv(b.ptr, b.ptr, 256, b.ptr, 0, 4, 256, 3, 4, NULL) == q8mi.REJECTED    # batch > 2
    assert L.q8mi_qgemv(b.ptr, b.ptr, 250, b.ptr, 0, 4, 250, 1, 4, NULL) == q8mi.REJECTED    # cols % 32
