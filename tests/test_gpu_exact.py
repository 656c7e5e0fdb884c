"""GPU parity, bit for bit, on the PRODUCTION kernels of every family.

The inputs (tests/exact_inputs.py) have power-of-two scales and small quants, so every per-block
term and every partial sum is exactly representable in fp32 whatever the order a kernel adds them
in.  The fp32 outputs of the dot-product GEMV, the matrix-core GEMV, the 128 x 128 MFMA GEMM (with
and without a K-split last round), the ring-staged GEMM tiles, the register-staged GEMM, the
small-batch D4 route and the fused LM head's logits must therefore EQUAL the CPU oracle's: a wrong
int32 block dot, a dropped or repeated block or a misplaced scale changes the bits.
"""
import ctypes as C

import numpy as np
import pytest

import exact_inputs as ex
import q8mi
from gpu_common import NULL, dev, quantize_d4, quantize_q8_1
from q8mi import hip, ok

pytestmark = pytest.mark.gpu

PAIR = np.dtype([("value", np.float32), ("index", np.int32)])


def same_bits(got, ref, what):
    got = np.ascontiguousarray(got, np.float32)
    ref = np.ascontiguousarray(ref, np.float32)
    if not np.array_equal(got.view(np.uint32), ref.view(np.uint32)):
        bad = np.argwhere(got.view(np.uint32) != ref.view(np.uint32))
        i = tuple(bad[0])
        raise AssertionError(f"{what}: {len(bad)}/{got.size} outputs differ; first at {i}: got {got[i]!r} ref {ref[i]!r}")


def q8_1_exact(oracle, x):
    """Q8_1 blocks of x on the device, checked against the oracle and against the construction."""
    dy, y = quantize_q8_1(x)
    rc, yref = oracle.quantize_q8_1(x)
    assert np.array_equal(y, yref)
    d = y.reshape(x.shape[0], -1, 36)[:, :, :2].copy().view(np.float16).astype(np.float32)
    assert set(np.unique(d)) <= {0.5, 1.0}, "activation scales must be the powers of two put in"
    return dy, y


# rows x cols: 2.5-step rows (5120), whole-step rows (6144, 2048), the longest model rows (17408), few rows
GEMV_SHAPES = [(1000, 5120), (515, 6144), (160, 17408), (37, 2048)]


@pytest.mark.parametrize("rows,cols", GEMV_SHAPES)
@pytest.mark.parametrize("batch", [1, 2, 3, 4, 5, 6, 7, 8])
def test_gemv_bits(gpu, oracle, rows, cols, batch):
    """q8mi_gemv: every batch, so both the dot-product kernels and the matrix-core kernel."""
    w = ex.weight(rows, cols, seed=rows + cols)
    x = ex.activations(batch, cols, seed=batch * 7 + cols)
    dw = dev(w)
    dy, y = q8_1_exact(oracle, x)
    out = hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    ok(q8mi.lib().q8mi_gemv(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, rows, NULL), "gemv")
    hip.synchronize()
    rc, ref = oracle.gemv(w, y, rows, cols, batch)
    same_bits(out.download(np.float32).reshape(batch, rows), ref, f"gemv {rows}x{cols} M={batch}")


@pytest.mark.parametrize("batch", [1, 2, 3, 4, 8])
def test_gemv_fused_forms_bits(gpu, oracle, batch):
    """Residual add (fp32 and bf16), bf16 store, two weights and the four-way fan-out."""
    rows, cols = 300, 5120
    L = q8mi.lib()
    w0, w1 = ex.weight(rows, cols, seed=1), ex.weight(rows, cols, seed=2)
    x = ex.activations(batch, cols, seed=3 + batch)
    dw0, dw1 = dev(w0), dev(w1)
    dy, y = q8_1_exact(oracle, x)
    base = ex.residual(batch, rows, seed=4)
    oa = dev(base)
    ok(L.q8mi_gemv_add(dw0.ptr, dy.ptr, oa.ptr, rows, cols, batch, rows, NULL), "add")
    ob = hip.DeviceBuffer(2 * batch * rows)
    ok(L.q8mi_gemv_bf16(dw0.ptr, dy.ptr, ob.ptr, rows, cols, batch, rows, NULL), "bf16")
    base16 = (base.view(np.uint32) >> 16).astype(np.uint16)     # exact: the residual has few bits
    oab = dev(base16)
    ok(L.q8mi_gemv_add_bf16(dw0.ptr, dy.ptr, oab.ptr, rows, cols, batch, rows, NULL), "add_bf16")
    o0, o1 = hip.DeviceBuffer(4 * batch * rows), hip.DeviceBuffer(4 * batch * rows)
    ok(L.q8mi_gemv_two(dw0.ptr, dw1.ptr, dy.ptr, o0.ptr, o1.ptr, rows, cols, batch, rows, NULL), "two")
    hip.synchronize()
    rc, refa = oracle.gemv_add(w0, y, base, rows, cols, batch)
    same_bits(oa.download(np.float32).reshape(batch, rows), refa, "gemv_add")
    rc, refb = oracle.gemv_bf16(w0, y, rows, cols, batch)
    assert np.array_equal(ob.download(np.uint16).reshape(batch, rows), refb)
    rc, refab = oracle.gemv_add_bf16(w0, y, base16, rows, cols, batch)
    assert np.array_equal(oab.download(np.uint16).reshape(batch, rows), refab)
    rc, r0 = oracle.gemv(w0, y, rows, cols, batch)
    rc, r1 = oracle.gemv(w1, y, rows, cols, batch)
    same_bits(o0.download(np.float32).reshape(batch, rows), r0, "gemv_two/0")
    same_bits(o1.download(np.float32).reshape(batch, rows), r1, "gemv_two/1")

    frows = [96, 0, 17, 130]
    ws = [ex.weight(r, cols, seed=50 + i) if r else None for i, r in enumerate(frows)]
    dws = [dev(v) if v is not None else None for v in ws]
    outs = [hip.DeviceBuffer(4 * batch * max(r, 1)) for r in frows]
    p = lambda b: b.ptr if b is not None else None
    ok(L.q8mi_gemv_fanout4(p(dws[0]), p(dws[1]), p(dws[2]), p(dws[3]), dy.ptr, outs[0].ptr, outs[1].ptr,
                           outs[2].ptr, outs[3].ptr, *frows, cols, batch, *[max(r, 1) for r in frows], NULL), "fanout4")
    hip.synchronize()
    for i, r in enumerate(frows):
        if r:
            rc, ref = oracle.gemv(ws[i], y, r, cols, batch)
            same_bits(outs[i].download(np.float32).reshape(batch, r), ref, f"fanout slot {i}")


@pytest.mark.parametrize("rows,cols", [(700, 5120), (300, 17408)])
@pytest.mark.parametrize("batch", [1, 2])
def test_qgemv_bits(gpu, oracle, rows, cols, batch):
    """Quantizer fused into the GEMV (fp32 activations in): 256-thread form and, for rows above
    8192 columns, the 1024-thread form."""
    w = ex.weight(rows, cols, seed=rows)
    x = ex.activations(batch, cols, seed=cols + batch)
    dw, dx = dev(w), dev(x)
    out = hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    ok(q8mi.lib().q8mi_qgemv(dw.ptr, dx.ptr, cols, out.ptr, 0, rows, cols, batch, rows, NULL), "qgemv")
    hip.synchronize()
    rc, y = oracle.quantize_q8_1(x)
    rc, ref = oracle.gemv(w, y, rows, cols, batch)
    same_bits(out.download(np.float32).reshape(batch, rows), ref, f"qgemv {rows}x{cols} M={batch}")


def gemm(dw, dy, rows, cols, batch, medium=False):
    out = hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    fn = q8mi.lib().q8mi_gemm_medium if medium else q8mi.lib().q8mi_gemm
    ok(fn(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, rows, NULL), "gemm")
    hip.synchronize()
    return out.download(np.float32).reshape(batch, rows)


def d4_exact(oracle, x):
    dy, y = quantize_d4(x)
    rc, yref = oracle.quantize_q8_1_d4(x)
    assert np.array_equal(y, yref)
    return dy, y


# (rows, batch, cols, which kernel serves it)
GEMM_CASES = [
    (2048, 2048, 512, "128 x 128 tiles, direct-to-LDS staging"),
    (1024, 2304, 640, "128 x 128 tiles, register staging (int8 plane 8-byte aligned)"),
    (1000, 33, 1024, "ring tiles, 64 activation rows wide"),
    (12320, 50, 512, "ring tiles, 64 weight rows x 64 activation rows (tall matrix)"),
    (1000, 100, 1024, "ring tiles, 128 activation rows wide"),
    (1000, 200, 5120, "ring tiles, 128 wide, two column tiles"),
    (4000, 29, 5120, "ring tiles, 32 wide, cut in two along K"),
    (1000, 20, 512, "ring tiles, 32 wide, whole K per workgroup"),
    (1000, 5, 5120, "matrix-core GEMV on D4 activations"),
    (1000, 16, 5120, "matrix-core GEMV on D4 activations, 16 rows"),
    (640, 8, 17408, "ring tiles, 32 wide, cut in two along K (long rows)"),
    (8320, 8, 17408, "matrix-core GEMV on D4 activations, two passes of four rows"),
]


@pytest.mark.parametrize("rows,batch,cols,what", GEMM_CASES)
def test_gemm_bits(gpu, oracle, rows, batch, cols, what):
    w = ex.weight(rows, cols, seed=rows + batch)
    x = ex.activations(batch, cols, seed=cols + batch)
    dw = dev(w)
    dy, y = d4_exact(oracle, x)
    got = gemm(dw, dy, rows, cols, batch)
    rc, ref = oracle.gemm_d4(w, y, rows, cols, batch, threads=16)
    same_bits(got, ref, f"gemm {rows}x{batch}x{cols} ({what})")
    if batch <= 64:
        same_bits(gemm(dw, dy, rows, cols, batch, medium=True), ref, f"gemm_medium {rows}x{batch}x{cols}")


def test_gemm_split_last_round_bits(gpu, oracle):
    """640 main tiles on 512 slots: the 128 tiles of the last round are summed from two halves of
    K with fp32 atomic adds onto zero.  Every output of 64 activation rows and a seeded sample of
    the rest equal the oracle."""
    rows, batch, cols = 5120, 2048, 1024
    w = ex.weight(rows, cols, seed=11)
    x = ex.activations(batch, cols, seed=12)
    dw = dev(w)
    dy, y = d4_exact(oracle, x)
    got = gemm(dw, dy, rows, cols, batch)
    js = np.concatenate([np.arange(0, 32), np.arange(batch - 32, batch)]).astype(np.uint32)
    rr, jj = np.meshgrid(np.arange(rows, dtype=np.uint32), js)
    rc, ref, _ = oracle.gemm_d4_sampled(w, y, rows, cols, batch, rr.reshape(-1), jj.reshape(-1))
    same_bits(got[jj.reshape(-1), rr.reshape(-1)], ref, "gemm split last round (64 activation rows)")
    rng = np.random.default_rng(13)
    sr = rng.integers(0, rows, 200000, dtype=np.uint32)
    sj = rng.integers(0, batch, 200000, dtype=np.uint32)
    rc, ref, _ = oracle.gemm_d4_sampled(w, y, rows, cols, batch, sr, sj)
    same_bits(got[sj, sr], ref, "gemm split last round (sample)")


@pytest.mark.parametrize("vocab,batch", [(20000, 1), (20000, 2), (20000, 4), (20000, 8), (70001, 4), (70001, 8)])
def test_lm_head_logits_bits(gpu, oracle, vocab, batch):
    """The fused LM head's logits (dot-product variant; matrix-core variant from 3 rows on weights
    of up to 65536 rows and from 7 rows on taller ones) and its winners against the oracle."""
    cols = 5120
    L = q8mi.lib()
    w = ex.weight(vocab, cols, seed=vocab)
    x = ex.activations(batch, cols, seed=batch)
    dw = dev(w)
    dy, y = q8_1_exact(oracle, x)
    scratch = hip.DeviceBuffer(L.q8mi_lm_head_scratch_bytes(vocab, cols, batch))
    row_out, acc = hip.DeviceBuffer(8 * batch), hip.DeviceBuffer(8)
    logits = hip.DeviceBuffer(4 * batch * vocab).fill(0xff)
    drafts = np.zeros(8, np.int32)
    ok(L.q8mi_lm_head_argmax_accept(dw.ptr, dy.ptr, vocab, cols, batch, drafts.ctypes.data_as(C.c_void_p), 0, 2,
                                    row_out.ptr, acc.ptr, logits.ptr, vocab, scratch.ptr, NULL), "lm_head")
    hip.synchronize()
    rc, ref = oracle.gemv(w, y, vocab, cols, batch, threads=16)
    same_bits(logits.download(np.float32).reshape(batch, vocab), ref, f"lm-head logits, vocab {vocab}, M={batch}")
    want = oracle.argmax_rows_scan(ref, batch, vocab)
    got = row_out.download(PAIR)
    assert np.array_equal(got["index"], want["index"])          # equal logits abound here: lowest id must win
    assert np.array_equal(got["value"].view(np.uint32), want["value"].view(np.uint32))
