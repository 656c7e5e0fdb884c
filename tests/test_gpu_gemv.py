"""GPU parity: GEMV family (batch 1..8) through the C ABI vs the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

import q8mi
from gpu_common import NULL, assert_close_fp32, dev, quantize_q8_1
from q8mi import hip, ok
import q8mi_support as synth

pytestmark = pytest.mark.gpu


def block_dot_check(oracle, dw, w, dy, y, rows, cols, batch, seed, n=4096):
    """Sampled per-block int32 dots: GPU must equal the oracle bit for bit."""
    rng = np.random.default_rng(seed)
    sr = rng.integers(0, rows, n, dtype=np.uint32)
    sj = rng.integers(0, batch, n, dtype=np.uint32)
    sk = rng.integers(0, cols // 32, n, dtype=np.uint32)
    out = hip.DeviceBuffer(4 * n)
    d_sr, d_sj, d_sk = dev(sr), dev(sj), dev(sk)
    ok(synth.lib().q8sup_block_dots(dw.ptr, dy.ptr, 0, rows, cols, batch, d_sr.ptr, d_sj.ptr, d_sk.ptr, n,
                                  out.ptr, NULL), "block_dots")
    hip.synchronize()
    got = out.download(np.int32, n)
    ref = np.array([oracle.block_dot(w, y, 0, cols, batch, int(r), int(j), int(k))
                    for r, j, k in zip(sr, sj, sk)], np.int32)
    assert np.array_equal(got, ref)


# (rows, cols): aligned planes (cols % 256 == 0), ragged step counts, tiny rows; rows of 4, 5, 6, 8
# and 17 KiB have kernels of their own at batch 1..4 (odd row counts end in a single-row pair)
SHAPES = [(5120, 5120), (64, 256), (7, 512), (300, 2304), (129, 6144), (33, 17408), (131, 4096), (75, 8192)]


@pytest.mark.parametrize("rows,cols", SHAPES)
@pytest.mark.parametrize("batch", [1, 2, 3, 4, 5, 6, 7, 8])
def test_gemv_matches_oracle(gpu, oracle, rows, cols, batch):
    w = synth.q8_0_weight(rows, cols, seed=rows * 31 + cols)
    x = synth.normal(batch, cols, seed=batch * 1000 + cols)
    dw = dev(w)
    dy, y = quantize_q8_1(x)
    rc, yref = oracle.quantize_q8_1(x)
    assert np.array_equal(y, yref)
    out = hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    ok(q8mi.lib().q8mi_gemv(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, rows, NULL), "gemv")
    hip.synchronize()
    got = out.download(np.float32).reshape(batch, rows)
    rc, ref = oracle.gemv(w, y, rows, cols, batch)
    rc, absum = oracle.gemv_abs(w, y, rows, cols, batch)
    assert_close_fp32(got, ref, absum, f"gemv {rows}x{cols} M={batch}")
    if batch in (1, 8):
        block_dot_check(oracle, dw, w, dy, y, rows, cols, batch, seed=rows + batch, n=1024)


@pytest.mark.parametrize("rows,cols,batch", [(9001, 17408, 8), (9001, 17408, 3), (40003, 5120, 7), (2049, 8192, 5)])
def test_gemv_matrix_core_splits(gpu, oracle, rows, cols, batch):
    """Both ways the matrix-core kernel splits a workgroup's items over its waves: round-robin with
    every item's sums parked (40003 x 5120 and 2049 x 8192: several units per workgroup, a ragged
    last unit), and contiguous ranges where those sums do not fit LDS beside the activations
    (9001 x 17408: nine units of seventeen items per workgroup next to eight rows of 17408 columns)."""
    w = synth.q8_0_weight(rows, cols, seed=rows + cols)
    x = synth.normal(batch, cols, seed=batch + cols)
    dw = dev(w)
    dy, y = quantize_q8_1(x)
    out = hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    ok(q8mi.lib().q8mi_gemv(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, rows, NULL), "gemv")
    hip.synchronize()
    rc, ref = oracle.gemv(w, y, rows, cols, batch, threads=16)
    rc, absum = oracle.gemv_abs(w, y, rows, cols, batch)
    assert_close_fp32(out.download(np.float32).reshape(batch, rows), ref, absum, f"gemv {rows}x{cols} M={batch}")


@pytest.mark.parametrize("offset", [4, 8, 12])
@pytest.mark.parametrize("batch", [1, 2, 4, 8])
def test_gemv_activations_on_a_4_byte_boundary(gpu, oracle, offset, batch):
    """Q8_1 blocks are only 4-byte aligned by type (36 bytes each): an activation buffer that does
    not start on a 16-byte boundary must give the same results (the lanes then read it from
    global memory instead of a 16-byte-wide LDS staging copy)."""
    rows, cols = 777, 2048
    w = synth.q8_0_weight(rows, cols, seed=5)
    x = synth.normal(batch, cols, seed=6 + batch)
    dw = dev(w)
    _, y = quantize_q8_1(x)
    shifted = hip.DeviceBuffer(len(y) + 16)
    shifted.upload(y, offset)
    L = q8mi.lib()
    out = hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    ok(L.q8mi_gemv(dw.ptr, shifted.ptr + offset, out.ptr, rows, cols, batch, rows, NULL), "gemv")
    hip.synchronize()
    rc, ref = oracle.gemv(w, y, rows, cols, batch)
    rc, absum = oracle.gemv_abs(w, y, rows, cols, batch)
    assert_close_fp32(out.download(np.float32).reshape(batch, rows), ref, absum, f"gemv y+{offset} M={batch}")
    # the fused LM head takes the same buffer
    scratch = hip.DeviceBuffer(L.q8mi_lm_head_scratch_bytes(rows, cols, batch))
    pairs, acc = hip.DeviceBuffer(8 * batch), hip.DeviceBuffer(8)
    drafts = np.zeros(8, np.int32)
    ok(L.q8mi_lm_head_argmax_accept(dw.ptr, shifted.ptr + offset, rows, cols, batch, drafts.ctypes.data_as(C.c_void_p),
                                    0, 0, pairs.ptr, acc.ptr, None, rows, scratch.ptr, NULL), "lm_head")
    hip.synchronize()
    tok = pairs.download(np.dtype([("value", np.float32), ("index", np.int32)]))["index"]
    want = oracle.argmax_rows_scan(ref, batch, rows)["index"]
    assert np.array_equal(tok, want)


@pytest.mark.parametrize("cols", [32, 96, 160, 992])
@pytest.mark.parametrize("batch", [1, 3, 8])
def test_gemv_unaligned_planes(gpu, oracle, cols, batch):
    """cols/32 not a multiple of 8: rows are only 2-byte aligned (fallback kernel)."""
    rows = 37
    w = synth.q8_0_weight(rows, cols, seed=cols)
    x = synth.normal(batch, cols, seed=cols + batch)
    dw = dev(w)
    dy, y = quantize_q8_1(x)
    out = hip.DeviceBuffer(4 * batch * rows)
    ok(q8mi.lib().q8mi_gemv(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, rows, NULL), "gemv")
    hip.synchronize()
    got = out.download(np.float32).reshape(batch, rows)
    rc, ref = oracle.gemv(w, y, rows, cols, batch)
    rc, absum = oracle.gemv_abs(w, y, rows, cols, batch)
    assert_close_fp32(got, ref, absum, f"gemv unaligned cols={cols} M={batch}")


def test_gemv_closed_form(gpu):
    """Reference's own closed form (tests/mixed_linear_parity.cu:205-263): every
    weight block d = 0.5, q = 1 and a constant input x give cols * 0.5 * x."""
    rows, cols = 96, 1024
    nb = cols // 32
    w = np.zeros((rows, nb * 34), np.uint8)
    w[:, :2 * nb] = np.tile(np.frombuffer(np.float16(0.5).tobytes(), np.uint8), nb)
    w[:, 2 * nb:] = 1
    for batch, xv in [(1, 0.25), (4, 2.0)]:
        x = np.full((batch, cols), xv, np.float32)
        dy, _ = quantize_q8_1(x)
        dw = dev(w)
        out = hip.DeviceBuffer(4 * batch * rows)
        ok(q8mi.lib().q8mi_gemv(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, rows, NULL), "gemv")
        hip.synchronize()
        got = out.download(np.float32)
        # x quantizes to q = 127 with d = fp16(x/127): expected = cols * 0.5 * 127 * d_x
        dx = np.float32(np.float16(np.float32(xv) / np.float32(127.0)))
        expect = np.float32(cols * 0.5 * 127.0) * dx
        assert np.allclose(got, expect, rtol=1e-6, atol=0)
        assert abs(expect - cols * 0.5 * xv) <= 1e-3 * cols * 0.5 * xv


def test_gemv_stride_and_rejections(gpu, oracle):
    rows, cols, batch = 70, 512, 3
    stride = rows + 11
    w = synth.q8_0_weight(rows, cols, seed=1)
    x = synth.normal(batch, cols, seed=2)
    dw = dev(w)
    dy, y = quantize_q8_1(x)
    sentinel = np.full(batch * stride, 123.0, np.float32)
    out = dev(sentinel)
    ok(q8mi.lib().q8mi_gemv(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, stride, NULL), "gemv")
    hip.synchronize()
    got = out.download(np.float32).reshape(batch, stride)
    rc, ref = oracle.gemv(w, y, rows, cols, batch, stride=stride)
    rc, absum = oracle.gemv_abs(w, y, rows, cols, batch, stride=stride)
    assert_close_fp32(got[:, :rows], ref[:, :rows], absum[:, :rows], "gemv strided")
    assert np.all(got[:, rows:] == 123.0), "padding between rows must stay untouched"
    L = q8mi.lib()
    assert L.q8mi_gemv(dw.ptr, dy.ptr, out.ptr, rows, 500, batch, stride, NULL) == q8mi.REJECTED
    assert L.q8mi_gemv(dw.ptr, dy.ptr, out.ptr, rows, cols, 0, stride, NULL) == q8mi.REJECTED
    assert L.q8mi_gemv(dw.ptr, dy.ptr, out.ptr, rows, cols, 9, stride, NULL) == q8mi.REJECTED
    assert np.all(out.download(np.float32).reshape(batch, stride)[:, rows:] == 123.0)


# (rows, cols): a streamed row length; rows whose activations stay in registers at batch 1..2; the
# 17 KiB rows shared by the waves of a workgroup at batch 1 (odd row count: a single-row last pair)
@pytest.mark.parametrize("rows,cols", [(200, 2048), (130, 6144), (67, 17408)])
@pytest.mark.parametrize("batch", [1, 2, 3, 4, 5, 8])
def test_gemv_fused_variants(gpu, oracle, batch, rows, cols):
    w0 = synth.q8_0_weight(rows, cols, seed=10)
    w1 = synth.q8_0_weight(rows, cols, seed=11)
    x = synth.normal(batch, cols, seed=12 + batch)
    dw0, dw1 = dev(w0), dev(w1)
    dy, y = quantize_q8_1(x)
    L = q8mi.lib()
    rc, ref0 = oracle.gemv(w0, y, rows, cols, batch)
    rc, ref1 = oracle.gemv(w1, y, rows, cols, batch)
    rc, abs0 = oracle.gemv_abs(w0, y, rows, cols, batch)
    rc, abs1 = oracle.gemv_abs(w1, y, rows, cols, batch)

    # two weights, one activation
    o0, o1 = hip.DeviceBuffer(4 * batch * rows), hip.DeviceBuffer(4 * batch * rows)
    ok(L.q8mi_gemv_two(dw0.ptr, dw1.ptr, dy.ptr, o0.ptr, o1.ptr, rows, cols, batch, rows, NULL), "two")
    hip.synchronize()
    rc, t0, t1 = oracle.gemv_two(w0, w1, y, rows, cols, batch)
    assert np.array_equal(t0, ref0) and np.array_equal(t1, ref1)   # oracle: two == 2 x plain
    assert_close_fp32(o0.download(np.float32), ref0, abs0, "two/0")
    assert_close_fp32(o1.download(np.float32), ref1, abs1, "two/1")

    # SwiGLU: silu(g)*u.  Allowance: propagate the reordering allowance of g and u
    # through the product, plus 1e-5 relative for the exp.
    os_ = hip.DeviceBuffer(4 * batch * rows)
    ok(L.q8mi_gemv_silu_mul(dw0.ptr, dw1.ptr, dy.ptr, os_.ptr, rows, cols, batch, rows, NULL), "silu")
    hip.synchronize()
    got = os_.download(np.float32).astype(np.float64)
    rc, ref = oracle.gemv_silu_mul(w0, w1, y, rows, cols, batch)
    g = ref0.astype(np.float64).reshape(-1)
    u = ref1.astype(np.float64).reshape(-1)
    sig = 1.0 / (1.0 + np.exp(-g))
    silu = g * sig
    dsilu = sig * (1.0 + g * (1.0 - sig))
    lim = (1e-5 * np.abs(silu * u) + np.abs(u * dsilu) * (1e-5 * np.abs(g) + 1e-6 * abs0.reshape(-1))
           + np.abs(silu) * (1e-5 * np.abs(u) + 1e-6 * abs1.reshape(-1)))
    err = np.abs(got - ref.reshape(-1))
    assert np.all(err <= lim), f"silu_mul: max excess {(err - lim).max():.3e}"
    # the oracle's own SwiGLU agrees with float64 math on its g and u
    assert np.allclose(ref.reshape(-1), silu * u, rtol=2e-6, atol=1e-30)

    # residual add (fp32)
    base = synth.normal(batch, rows, seed=99)
    oa = dev(base)
    ok(L.q8mi_gemv_add(dw0.ptr, dy.ptr, oa.ptr, rows, cols, batch, rows, NULL), "add")
    hip.synchronize()
    rc, refa = oracle.gemv_add(w0, y, base, rows, cols, batch)
    assert_close_fp32(oa.download(np.float32), refa, abs0 + np.abs(base), "add")

    # bf16 store and bf16 residual add: compare after rounding; allow one bf16 ulp
    # where the fp32 value sits on a rounding boundary
    ob = hip.DeviceBuffer(2 * batch * rows)
    ok(L.q8mi_gemv_bf16(dw0.ptr, dy.ptr, ob.ptr, rows, cols, batch, rows, NULL), "bf16")
    hip.synchronize()
    rc, refb = oracle.gemv_bf16(w0, y, rows, cols, batch)
    gb = ob.download(np.uint16).astype(np.int32)
    diff = np.abs(gb - refb.reshape(-1).astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.01
    base16 = (base.view(np.uint32) >> 16).astype(np.uint16)
    oab = dev(base16)
    ok(L.q8mi_gemv_add_bf16(dw0.ptr, dy.ptr, oab.ptr, rows, cols, batch, rows, NULL), "add_bf16")
    hip.synchronize()
    rc, refab = oracle.gemv_add_bf16(w0, y, base16, rows, cols, batch)
    diff = np.abs(oab.download(np.uint16).astype(np.int32) - refab.reshape(-1).astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.01


# columns: a streamed row length, one whose activations stay in registers at batch 1..2, and the
# 17 KiB rows that the waves of a workgroup share at batch 1 (odd row counts end in a single-row pair)
@pytest.mark.parametrize("cols", [1024, 5120, 17408])
@pytest.mark.parametrize("batch", [1, 2, 3, 4, 8])
def test_gemv_fanout4(gpu, oracle, batch, cols):
    rows = [96, 0, 17, 130]           # slot 1 is empty, as when the executor passes 3 weights
    ws = [synth.q8_0_weight(r, cols, seed=50 + i) if r else None for i, r in enumerate(rows)]
    x = synth.normal(batch, cols, seed=77)
    dy, y = quantize_q8_1(x)
    dws = [dev(w) if w is not None else None for w in ws]
    strides = [r + 5 for r in rows]
    outs = [hip.DeviceBuffer(4 * batch * s) for s in strides]
    p = lambda b: b.ptr if b is not None else None
    ok(q8mi.lib().q8mi_gemv_fanout4(p(dws[0]), p(dws[1]), p(dws[2]), p(dws[3]), dy.ptr,
                                    outs[0].ptr, outs[1].ptr, outs[2].ptr, outs[3].ptr,
                                    rows[0], rows[1], rows[2], rows[3], cols, batch,
                                    strides[0], strides[1], strides[2], strides[3], NULL), "fanout4")
    hip.synchronize()
    rc, refs = oracle.gemv_fanout4(ws, y, rows, cols, batch, strides)
    assert rc == 0
    for i, r in enumerate(rows):
        if not r:
            continue
        got = outs[i].download(np.float32).reshape(batch, strides[i])[:, :r]
        rc, ab = oracle.gemv_abs(ws[i], y, r, cols, batch)
        assert_close_fp32(got, refs[i][:, :r], ab, f"fanout slot {i}")
    # all-empty fan-out is rejected like the reference's launcher
    assert q8mi.lib().q8mi_gemv_fanout4(None, None, None, None, dy.ptr, None, None, None, None,
                                        0, 0, 0, 0, cols, batch, 0, 0, 0, 0, NULL) == q8mi.REJECTED


def test_gemv_is_deterministic(gpu):
    rows, cols, batch = 4096, 5120, 4
    w = synth.q8_0_weight(rows, cols, seed=3)
    x = synth.normal(batch, cols, seed=4)
    dw = dev(w)
    dy, _ = quantize_q8_1(x)
    out = hip.DeviceBuffer(4 * batch * rows)
    runs = []
    for _ in range(3):
        ok(q8mi.lib().q8mi_gemv(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, rows, NULL), "gemv")
        hip.synchronize()
        runs.append(out.download(np.uint32))
    assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2])
