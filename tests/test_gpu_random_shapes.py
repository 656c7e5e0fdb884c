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
