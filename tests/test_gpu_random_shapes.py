"""GPU parity on seeded random shapes: every GEMV / GEMM route (dot-product and matrix-core GEMV,
unaligned-plane fallback, ring-staged and 128 x 128 GEMM tiles) against the CPU oracle, with rows,
columns and batches that are ragged against every tile and step size."""
import numpy as np
import pytest

import q8mi
from gpu_common import NULL, assert_close_fp32, dev, quantize_d4, quantize_q8_1
from q8mi import hip, ok
import q8mi_support as synth

pytestmark = pytest.mark.gpu


def shapes(seed, n, max_rows, max_cols, col_step, max_batch):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        rows = int(rng.integers(1, max_rows + 1))
        cols = int(rng.integers(1, max_cols // col_step + 1)) * col_step
        batch = int(rng.integers(1, max_batch + 1))
        out.append((rows, cols, batch))
    return out


@pytest.mark.parametrize("rows,cols,batch", shapes(1, 24, 3000, 8192, 32, 8))
def test_gemv_random_shapes(gpu, oracle, rows, cols, batch):
    L = gpu.lib()
    w = synth.q8_0_weight(rows, cols, seed=rows * 7 + cols)
    x = synth.normal(batch, cols, seed=batch * 5 + rows)
    dw = dev(w)
    dy, y = quantize_q8_1(x)
    stride = rows + 2
    out = hip.DeviceBuffer(4 * batch * stride).fill(0xff)
    ok(L.q8mi_gemv(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, stride, NULL), "gemv")
    hip.synchronize()
    got = out.download(np.float32).reshape(batch, stride)
    rc, ref = oracle.gemv(w, y, rows, cols, batch, threads=8)
    rc, absum = oracle.gemv_abs(w, y, rows, cols, batch)
    assert_close_fp32(got[:, :rows], ref, absum, f"gemv {rows}x{cols} M={batch}")
    assert np.all(got[:, rows:].view(np.uint32) == 0xffffffff), "stores must stay inside the rows"


@pytest.mark.parametrize("rows,cols,batch", shapes(2, 20, 2500, 4096, 128, 300))
def test_gemm_random_shapes(gpu, oracle, rows, cols, batch):
    L = gpu.lib()
    rows = max(rows, 128)                  # below 128 rows the entry point takes Q8_1 activations
    w = synth.q8_0_weight(rows, cols, seed=rows * 11 + cols)
    x = synth.normal(batch, cols, seed=batch * 3 + cols)
    dw = dev(w)
    dy, y = quantize_d4(x)
    stride = rows + 1
    out = hip.DeviceBuffer(4 * batch * stride).fill(0xff)
    ok(L.q8mi_gemm(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, stride, NULL), "gemm")
    hip.synchronize()
    got = out.download(np.float32).reshape(batch, stride)
    rc, ref = oracle.gemm_d4(w, y, rows, cols, batch, threads=8)
    rr, jj = np.meshgrid(np.arange(rows, dtype=np.uint32), np.arange(batch, dtype=np.uint32))
    rc, _, absum = oracle.gemm_d4_sampled(w, y, rows, cols, batch, rr.reshape(-1), jj.reshape(-1))
    assert_close_fp32(got[:, :rows], ref, absum, f"gemm {rows}x{cols} batch {batch}")
    assert np.all(got[:, rows:].view(np.uint32) == 0xffffffff), "stores must stay inside the rows"


def shared_row_cases(seed, n):
    rng = np.random.default_rng(seed)
    out = [(1, 5120, 1), (2, 5120, 2), (3, 4096, 3), (1, 17408, 2), (5, 8192, 4)]   # fewer rows than a workgroup takes
    for _ in range(n):
        out.append((int(rng.integers(1, 700)), int(rng.choice([4096, 5120, 6144, 8192, 17408])), int(rng.integers(1, 5))))
    # every whole number of KiB up to 17 at batch 1 and 2 (each has an instantiation of its own)
    for kib in range(1, 18):
        out.append((int(rng.integers(1, 300)), 1024 * kib, 1))
        out.append((int(rng.integers(1, 300)), 1024 * kib, 2))
    out += [(700, 2048, 3), (431, 3072, 4), (9000, 2048, 4), (17001, 1024, 2), (300, 1024, 3)]   # 1 .. 3 KiB at batch 2 .. 4
    out += [(700, 7168, 3), (333, 12288, 4), (50, 3328, 2), (50, 2560, 1)]   # lengths and batches other kernels serve
    out += [(5120, 15360, 2), (3072, 17408, 1), (2048, 17408, 2)]   # long rows whose pairs leave two workgroups per CU
    return out


@pytest.mark.parametrize("rows,cols,batch", shared_row_cases(3, 15))
def test_gemv_forms_on_rows_with_kernels_of_their_own(gpu, oracle, rows, cols, batch):
    """Rows of 1 to 17 KiB at batch 1..4 (the waves of a workgroup share the row pairs):
    plain store into a padded output, residual add, SwiGLU, and the quantizer-inside forms, with
    row counts that leave single-row pairs and workgroups with fewer pairs than they may take."""
    L = gpu.lib()
    w0 = synth.q8_0_weight(rows, cols, seed=rows * 13 + cols)
    w1 = synth.q8_0_weight(rows, cols, seed=rows * 17 + cols)
    x = synth.normal(batch, cols, seed=batch * 7 + rows)
    dw0, dw1, dx = dev(w0), dev(w1), dev(x)
    dy, y = quantize_q8_1(x)
    rc, ref0 = oracle.gemv(w0, y, rows, cols, batch, threads=8)
    rc, abs0 = oracle.gemv_abs(w0, y, rows, cols, batch)
    stride = rows + 3
    out = hip.DeviceBuffer(4 * batch * stride).fill(0xff)
    ok(L.q8mi_gemv(dw0.ptr, dy.ptr, out.ptr, rows, cols, batch, stride, NULL), "gemv")
    hip.synchronize()
    got = out.download(np.float32).reshape(batch, stride)
    assert_close_fp32(got[:, :rows], ref0, abs0, f"gemv {rows}x{cols} M={batch}")
    assert np.all(got[:, rows:].view(np.uint32) == 0xffffffff), "stores must stay inside the rows"
    # residual add
    base = synth.normal(batch, rows, seed=rows + 1)
    acc = dev(base)
    ok(L.q8mi_gemv_add(dw0.ptr, dy.ptr, acc.ptr, rows, cols, batch, rows, NULL), "gemv_add")
    hip.synchronize()
    rc, refa = oracle.gemv_add(w0, y, base, rows, cols, batch)
    assert_close_fp32(acc.download(np.float32), refa, abs0 + np.abs(base), "gemv_add")
    # SwiGLU against the oracle's own (propagated allowance as in test_gpu_gemv.py)
    rc, ref1 = oracle.gemv(w1, y, rows, cols, batch, threads=8)
    rc, abs1 = oracle.gemv_abs(w1, y, rows, cols, batch)
    rc, refs = oracle.gemv_silu_mul(w0, w1, y, rows, cols, batch)
    os_ = hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    ok(L.q8mi_gemv_silu_mul(dw0.ptr, dw1.ptr, dy.ptr, os_.ptr, rows, cols, batch, rows, NULL), "silu")
    hip.synchronize()
    g, u = ref0.astype(np.float64).reshape(-1), ref1.astype(np.float64).reshape(-1)
    sig = 1.0 / (1.0 + np.exp(-g))
    lim = (1e-5 * np.abs(g * sig * u) + np.abs(u * sig * (1.0 + g * (1.0 - sig))) * (1e-5 * np.abs(g) + 1e-6 * abs0.reshape(-1))
           + np.abs(g * sig) * (1e-5 * np.abs(u) + 1e-6 * abs1.reshape(-1)))
    silu_got = os_.download(np.float32).astype(np.float64)
    assert np.all(np.abs(silu_got - refs.reshape(-1)) <= lim), "silu_mul"
    # the quantizer inside the launch: batch 1 and 2 give the two-step form's bits on rows of up to 8 KiB
    if batch <= 2:
        one = hip.DeviceBuffer(4 * batch * stride).fill(0xff)
        ok(L.q8mi_qgemv(dw0.ptr, dx.ptr, cols, one.ptr, 0, rows, cols, batch, stride, NULL), "qgemv")
        ones = hip.DeviceBuffer(4 * batch * rows).fill(0xee)
        ok(L.q8mi_qgemv_silu_mul(dw0.ptr, dw1.ptr, dx.ptr, cols, ones.ptr, rows, cols, batch, rows, NULL), "qgemv_silu_mul")
        hip.synchronize()
        got1 = one.download(np.float32).reshape(batch, stride)
        if cols <= 8192 and (batch == 1 or cols % 1024 == 0):   # both forms run the same kernel
            assert np.array_equal(got1.view(np.uint32), got.view(np.uint32)), "qgemv against gemv"
            assert np.array_equal(ones.download(np.uint32), os_.download(np.uint32)), "qgemv_silu_mul against gemv_silu_mul"
        else:
            assert_close_fp32(got1[:, :rows], ref0, abs0, "qgemv, another kernel than gemv")
            assert np.all(got1[:, rows:].view(np.uint32) == 0xffffffff)
