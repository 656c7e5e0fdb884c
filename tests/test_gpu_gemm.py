"""GPU parity: D4 quantizer + int8 MFMA GEMM through the C ABI vs the CPU oracle."""
import numpy as np
import pytest

import q8mi
from gpu_common import NULL, assert_close_fp32, dev, quantize_d4, quantize_q8_1
from q8mi import hip, ok
import q8mi_support as synth

pytestmark = pytest.mark.gpu


def run_gemm(dw, dy, rows, cols, batch, stride=None, medium=False):
    stride = rows if stride is None else stride
    out = hip.DeviceBuffer(4 * batch * stride).fill(0xff)
    fn = q8mi.lib().q8mi_gemm_medium if medium else q8mi.lib().q8mi_gemm
    ok(fn(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, stride, NULL), "gemm")
    hip.synchronize()
    return out.download(np.float32).reshape(batch, stride)


def d4_block_dots(oracle, dw, w, dy, y, rows, cols, batch, seed, n=2048):
    rng = np.random.default_rng(seed)
    sr = rng.integers(0, rows, n, dtype=np.uint32)
    sj = rng.integers(0, batch, n, dtype=np.uint32)
    sk = rng.integers(0, cols // 32, n, dtype=np.uint32)
    out = hip.DeviceBuffer(4 * n)
    a, b, c = dev(sr), dev(sj), dev(sk)
    ok(synth.lib().q8sup_block_dots(dw.ptr, dy.ptr, 1, rows, cols, batch, a.ptr, b.ptr, c.ptr, n, out.ptr, NULL),
       "block_dots")
    hip.synchronize()
    got = out.download(np.int32)
    ref = np.array([oracle.block_dot(w, y, 1, cols, batch, int(r), int(j), int(k))
                    for r, j, k in zip(sr, sj, sk)], np.int32)
    assert np.array_equal(got, ref)
    assert np.abs(got).max() <= 516128


# (rows M, batch N, cols K): the reference's own parity shapes (tests/mmq_parity.cu:275-295)
REFERENCE_SHAPES = [
    (128, 128, 256), (128, 128, 1024), (128, 128, 2048), (256, 128, 2048), (128, 256, 2048),
    (256, 256, 1024), (384, 256, 2048), (2048, 2048, 2048), (2304, 2048, 2304), (640, 2048, 2304),
    (2048, 2048, 2304), (2304, 2271, 2304), (2048, 2271, 2304), (2304, 223, 2304),
    (2048, 223, 2304), (640, 223, 2304),
]


@pytest.mark.parametrize("rows,batch,cols", REFERENCE_SHAPES)
def test_gemm_reference_shapes(gpu, oracle, rows, batch, cols):
    w = synth.q8_0_weight(rows, cols, seed=rows + cols)
    x = synth.normal(batch, cols, seed=batch + cols + 1)
    dw = dev(w)
    dy, y = quantize_d4(x)
    rc, yref = oracle.quantize_q8_1_d4(x)
    assert np.array_equal(y, yref), "quantized activations must be bit-exact"
    got = run_gemm(dw, dy, rows, cols, batch)
    big = rows * batch > 512 * 512
    if not big:
        rc, ref = oracle.gemm_d4(w, y, rows, cols, batch, threads=8)
        rr, jj = np.meshgrid(np.arange(rows, dtype=np.uint32), np.arange(batch, dtype=np.uint32))
        rc, ref_s, absum = oracle.gemm_d4_sampled(w, y, rows, cols, batch, rr.reshape(-1), jj.reshape(-1))
        assert np.array_equal(ref_s.reshape(batch, rows), ref)
        assert_close_fp32(got, ref, absum, f"gemm {rows}x{batch}x{cols}")
    else:
        rng = np.random.default_rng(rows)
        n = 20000
        sr = rng.integers(0, rows, n, dtype=np.uint32)
        sj = rng.integers(0, batch, n, dtype=np.uint32)
        # always include the corners and the last row / column of every tile edge
        sr[:4] = [0, rows - 1, 0, rows - 1]
        sj[:4] = [0, 0, batch - 1, batch - 1]
        rc, ref_s, absum = oracle.gemm_d4_sampled(w, y, rows, cols, batch, sr, sj)
        assert_close_fp32(got[sj, sr], ref_s, absum, f"gemm {rows}x{batch}x{cols} (sampled)")
    assert np.isfinite(got).all()
    d4_block_dots(oracle, dw, w, dy, y, rows, cols, batch, seed=cols, n=512)


@pytest.mark.parametrize("rows,batch,cols", [(4096, 2048, 256), (4480, 2050, 512), (9000, 1024, 256),
                                             (17408, 2048, 128), (5120, 2048, 512), (5120, 2000, 640),
                                             (17408, 2048, 512)])
def test_gemm_large_tilings(gpu, oracle, rows, batch, cols):
    """Shapes with at least one full round of main tiles on the chip: main tiles only, ragged in
    rows and batch, with a padded output stride; the last three leave a last round of 128 tiles on
    a 256-CU chip, which are computed as two halves of K added into a zeroed output (one with an
    odd number of 128-column super-blocks and a ragged batch)."""
    w = synth.q8_0_weight(rows, cols, seed=rows + 3 * cols)
    x = synth.normal(batch, cols, seed=batch + 5 * cols)
    dw = dev(w)
    dy, y = quantize_d4(x)
    stride = rows + 8
    got = run_gemm(dw, dy, rows, cols, batch, stride=stride)
    assert np.all(got[:, rows:].view(np.uint32) == 0xffffffff), "stores must stay inside the rows"
    assert np.isfinite(got[:, :rows]).all(), "every output must be written"
    rng = np.random.default_rng(rows + batch)
    n = 40000
    sr = rng.integers(0, rows, n, dtype=np.uint32)
    sj = rng.integers(0, batch, n, dtype=np.uint32)
    edge_rows = [0, rows - 1, rows - 33, max(rows - 129, 0), (rows // 128) * 128 - 1, (rows // 128) * 128 % rows]
    sr[:len(edge_rows)] = edge_rows
    sj[:len(edge_rows)] = [0, batch - 1, batch - 1, 0, batch - 1, batch // 2]
    rc, ref_s, absum = oracle.gemm_d4_sampled(w, y, rows, cols, batch, sr, sj)
    assert_close_fp32(got[sj, sr], ref_s, absum, f"gemm {rows}x{batch}x{cols} (sampled)")
    # all rows of two activation rows, to catch a misplaced tile anywhere along the weight rows
    for j in (0, batch - 1):
        rr = np.arange(rows, dtype=np.uint32)
        rc, ref_c, absum_c = oracle.gemm_d4_sampled(w, y, rows, cols, batch, rr, np.full(rows, j, np.uint32))
        assert_close_fp32(got[j, :rows], ref_c, absum_c, f"gemm column {j}")


def test_gemm_split_last_round_is_deterministic(gpu):
    """The tiles of a partly filled last round are summed from two halves of K by two workgroups
    in whichever order they finish: two addends onto zero, so repeated calls agree bit for bit."""
    rows, batch, cols = 5120, 2048, 1024
    dw = dev(synth.q8_0_weight(rows, cols, seed=5))
    dy, _ = quantize_d4(synth.normal(batch, cols, seed=6))
    first = run_gemm(dw, dy, rows, cols, batch)
    for _ in range(3):
        assert np.array_equal(run_gemm(dw, dy, rows, cols, batch).view(np.uint32), first.view(np.uint32))


def test_gemm_narrow_tiles_split_along_k_are_deterministic(gpu, oracle):
    """Up to 32 activation rows on at most one 32-row tile per CU: two workgroups per tile add their
    halves of K into a zeroed output.  Repeated calls agree bit for bit, a poisoned output is fully
    rewritten, the padding of a wider output stride is left alone, and the sums match the oracle."""
    rows, batch, cols = 5120, 29, 5120
    w = synth.q8_0_weight(rows, cols, seed=25)
    dw = dev(w)
    dy, y = quantize_d4(synth.normal(batch, cols, seed=26))
    first = run_gemm(dw, dy, rows, cols, batch, stride=rows + 8)
    assert np.all(first[:, rows:].view(np.uint32) == 0xffffffff)
    for _ in range(3):
        again = run_gemm(dw, dy, rows, cols, batch, stride=rows + 8)
        assert np.array_equal(again.view(np.uint32), first.view(np.uint32))
    rr, jj = np.meshgrid(np.arange(0, rows, 37, dtype=np.uint32), np.arange(batch, dtype=np.uint32))
    rc, ref_s, absum = oracle.gemm_d4_sampled(w, y, rows, cols, batch, rr.reshape(-1), jj.reshape(-1))
    assert_close_fp32(first[jj.reshape(-1), rr.reshape(-1)], ref_s, absum, "narrow tiles, K split")


@pytest.mark.parametrize("rows,cols,batch", [(17408, 1024, 20), (17408, 1024, 32), (17500, 512, 64), (17408, 768, 100)])
def test_gemm_ring_tiles_with_their_k_steps_dealt_out_evenly(gpu, oracle, rows, cols, batch):
    """A few more ring tiles than the chip holds workgroups (544 tiles of 32 x 32 for 512 slots, 272
    or 274 or 544 tiles of 64 x 64 for 256): every workgroup takes an equal range of the K steps of
    all tiles, tiles shared by two workgroups are added into a zeroed output.  Every output against
    the oracle, a wider stride left alone, repeated calls and graph replays bit for bit."""
    w = synth.q8_0_weight(rows, cols, seed=rows + cols + batch)
    dw = dev(w)
    dy, y = quantize_d4(synth.normal(batch, cols, seed=batch + 3))
    rc, ref = oracle.gemm_d4(w, y, rows, cols, batch, threads=8)
    rr, jj = np.meshgrid(np.arange(rows, dtype=np.uint32), np.arange(batch, dtype=np.uint32))
    rc, _, absum = oracle.gemm_d4_sampled(w, y, rows, cols, batch, rr.reshape(-1), jj.reshape(-1))
    stride = rows + 12
    first = run_gemm(dw, dy, rows, cols, batch, stride=stride)
    assert_close_fp32(first[:, :rows], ref, absum, f"gemm ring tiles, K steps dealt out, batch {batch}")
    assert np.all(first[:, rows:].view(np.uint32) == 0xffffffff), "stores must stay inside the rows"
    for _ in range(2):
        assert np.array_equal(run_gemm(dw, dy, rows, cols, batch, stride=stride).view(np.uint32), first.view(np.uint32))
    out = hip.DeviceBuffer(4 * batch * stride).fill(0xff)
    stream = hip.Stream()
    g = hip.Graph(stream)
    with g:
        ok(q8mi.lib().q8mi_gemm(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, stride, stream.handle), "gemm")
    for replay in range(2):
        g.launch()
        stream.synchronize()
        got = out.download(np.float32).reshape(batch, stride)
        assert np.array_equal(got[:, :rows].view(np.uint32), first[:, :rows].view(np.uint32)), f"replay {replay}"
        out.fill(0x7f)
        hip.synchronize()


def test_gemm_split_last_round_replays_in_a_graph(gpu):
    """The two-kernel call (zeroing kernel + GEMM with a K-split last round) captured into a HIP
    graph: every replay, onto an output poisoned in between, gives the eager call's bits."""
    rows, batch, cols = 5120, 2048, 512
    dw = dev(synth.q8_0_weight(rows, cols, seed=15))
    dy, _ = quantize_d4(synth.normal(batch, cols, seed=16))
    eager = run_gemm(dw, dy, rows, cols, batch)
    out = hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    stream = hip.Stream()
    g = hip.Graph(stream)
    with g:
        ok(q8mi.lib().q8mi_gemm(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, rows, stream.handle), "gemm")
    for replay in range(3):
        g.launch()
        stream.synchronize()
        got = out.download(np.float32).reshape(batch, rows)
        assert np.array_equal(got.view(np.uint32), eager.view(np.uint32)), f"replay {replay}"
        out.fill(0x7f)          # eager work between the replays
        hip.synchronize()


# the layer's projections: QKV, O, gate/up (one shape), down
@pytest.mark.parametrize("rows,cols", [(5120, 5120), (8192, 5120), (5120, 6144), (17408, 5120), (5120, 17408)])
def test_gemm_heavy_tail_batch_8192(gpu, oracle, rows, cols):
    """Long-context prefill shapes with heavy-tailed activations: batch 8192, Student-t(3) values
    with 0.1 % of the columns scaled by 20 (outlier channels).  Quantized activations bit-exact on a
    row sample, per-block int32 dots bit-exact and bounded by 32 * 127 * 127, outputs within
    tolerance on a seeded sample."""
    batch = 8192
    w = synth.q8_0_weight(rows, cols, seed=77)
    x = synth.student_t3(batch, cols, seed=78)
    assert np.abs(x).max() > 50.0, "the generator must produce outliers"
    dw = dev(w)
    dy, y = quantize_d4(x)
    pick = np.array([0, 1, 4095, 4096, 8191], np.int64)
    rc, yref = oracle.quantize_q8_1_d4(x[pick])
    yb = y.reshape(cols // 128, batch, 144)
    assert np.array_equal(yb[:, pick, :].reshape(-1), yref), "D4 blocks of the sampled rows must be bit-exact"
    got = run_gemm(dw, dy, rows, cols, batch)
    assert np.isfinite(got).all()
    rng = np.random.default_rng(79)
    n = 30000
    sr = rng.integers(0, rows, n, dtype=np.uint32)
    sj = rng.integers(0, batch, n, dtype=np.uint32)
    rc, ref_s, absum = oracle.gemm_d4_sampled(w, y, rows, cols, batch, sr, sj)
    assert_close_fp32(got[sj, sr], ref_s, absum, "gemm heavy tail (sampled)")
    d4_block_dots(oracle, dw, w, dy, y, rows, cols, batch, seed=80, n=1024)


def test_gemm_prompt_longer_than_a_grid_extent(gpu, oracle):
    """70 000 activation rows in one call (more than a grid's y extent): D4 quantizer bit-exact
    on the whole buffer, GEMM outputs within tolerance on a seeded sample."""
    rows, cols, batch = 256, 256, 70000
    w = synth.q8_0_weight(rows, cols, seed=91)
    x = synth.normal(batch, cols, seed=92)
    dw = dev(w)
    dy, y = quantize_d4(x)
    rc, yref = oracle.quantize_q8_1_d4(x)
    assert np.array_equal(y, yref)
    got = run_gemm(dw, dy, rows, cols, batch)
    rng = np.random.default_rng(93)
    n = 20000
    sr = rng.integers(0, rows, n, dtype=np.uint32)
    sj = np.concatenate([rng.integers(0, batch, n - 4, dtype=np.uint32), np.array([0, 65535, 65536, batch - 1], np.uint32)])
    rc, ref_s, absum = oracle.gemm_d4_sampled(w, y, rows, cols, batch, sr, sj)
    assert_close_fp32(got[sj, sr], ref_s, absum, "gemm, 70000 rows (sampled)")


def test_gemm_reference_tolerance_restated(gpu):
    """tests/mmq_parity.cu:246-254 restated: output vs fp32 dot of the dequantised
    operands within 5e-3 abs or 1e-3 rel, U(-0.5,0.5) weights and U(-1,1) activations."""
    rows, batch, cols = 256, 256, 1024
    rng = np.random.default_rng(0x5EED)
    wf = rng.uniform(-0.5, 0.5, (rows, cols)).astype(np.float32)
    x = rng.uniform(-1, 1, (batch, cols)).astype(np.float32)
    from oracle import q8_oracle as o   # only to build the Q8_0 weight bytes (test input)
    w = o.make_weight(wf)
    dw = dev(w)
    dy, y = quantize_d4(x)
    got = run_gemm(dw, dy, rows, cols, batch)
    nb = cols // 32
    dq_w = (w[:, 2 * nb:].view(np.int8).reshape(rows, nb, 32).astype(np.float32)
            * w[:, :2 * nb].copy().view(np.float16).astype(np.float32)[:, :, None]).reshape(rows, cols)
    yb = y.reshape(cols // 128, batch, 144)
    d4 = yb[:, :, :16].copy().view(np.float32)                      # [sb, j, 4]
    qs = yb[:, :, 16:].view(np.int8).reshape(cols // 128, batch, 4, 32).astype(np.float32)
    dq_x = (qs * d4[..., None]).transpose(1, 0, 2, 3).reshape(batch, cols)
    ref = dq_x @ dq_w.T
    d = np.abs(got - ref)
    assert np.all((d <= 5e-3) | (d <= 1e-3 * np.maximum(np.abs(ref), 1e-6)))


@pytest.mark.parametrize("rows,batch,cols", [(128, 1, 128), (129, 9, 384), (200, 33, 640), (500, 64, 1152),
                                             (1000, 12, 5120)])
def test_gemm_ragged_and_medium(gpu, oracle, rows, batch, cols):
    """Tile-edge handling (rows, batch not multiples of 128; cols/32 % 8 == 4) and the
    medium-batch entry point."""
    w = synth.q8_0_weight(rows, cols, seed=rows * 7 + cols)
    x = synth.normal(batch, cols, seed=batch * 13 + cols)
    dw = dev(w)
    dy, y = quantize_d4(x)
    rc, ref = oracle.gemm_d4(w, y, rows, cols, batch, threads=8)
    rr, jj = np.meshgrid(np.arange(rows, dtype=np.uint32), np.arange(batch, dtype=np.uint32))
    rc, _, absum = oracle.gemm_d4_sampled(w, y, rows, cols, batch, rr.reshape(-1), jj.reshape(-1))
    stride = rows + 3
    got = run_gemm(dw, dy, rows, cols, batch, stride=stride)
    assert_close_fp32(got[:, :rows], ref, absum, "gemm ragged")
    assert np.all(got[:, rows:].view(np.uint32) == 0xffffffff), "stores must stay inside the rows"
    got_m = run_gemm(dw, dy, rows, cols, batch, medium=True)
    assert np.array_equal(got_m.view(np.uint32), got[:, :rows].view(np.uint32))


@pytest.mark.parametrize("rows,cols", [(515, 1024), (5120, 5120), (130, 17408), (4, 256)])
@pytest.mark.parametrize("batch", [1, 3, 4, 7, 8, 9, 12, 13, 16, 17, 29, 32])
def test_gemm_small_batches_stream_the_weights(gpu, oracle, rows, cols, batch):
    """Batches of up to 16 rows on D4 activations are served by the weight-streaming matrix-core
    GEMV (when the activations fit LDS), 17..32 by the narrowest ring tile: same contract as the
    tile kernel."""
    w = synth.q8_0_weight(rows, cols, seed=rows * 5 + cols)
    x = synth.normal(batch, cols, seed=batch * 3 + cols)
    dw = dev(w)
    dy, y = quantize_d4(x)
    rc, ref = oracle.gemm_d4(w, y, rows, cols, batch, threads=8)
    rr, jj = np.meshgrid(np.arange(rows, dtype=np.uint32), np.arange(batch, dtype=np.uint32))
    rc, _, absum = oracle.gemm_d4_sampled(w, y, rows, cols, batch, rr.reshape(-1), jj.reshape(-1))
    stride = rows + 5
    fn = (lambda: run_gemm(dw, dy, rows, cols, batch, stride=stride)) if rows >= 128 else None
    if fn is None:   # rows < 128 take Q8_1 activations through q8mi_gemm; the D4 form goes through gemm_medium
        got = run_gemm(dw, dy, rows, cols, batch, stride=stride, medium=True)
    else:
        got = fn()
    assert_close_fp32(got[:, :rows], ref, absum, f"gemm small batch {batch}")
    assert np.all(got[:, rows:].view(np.uint32) == 0xffffffff), "stores must stay inside the rows"


def test_gemm_small_shapes_take_q8_1(gpu, oracle):
    """rows < 128 or cols % 128 != 0: the entry point expects Q8_1 activations, as the
    reference's launcher does for those shapes (src/kernels_cuda.cu:14545-14552)."""
    for rows, batch, cols in [(64, 20, 256), (300, 11, 160), (16, 32, 96)]:
        w = synth.q8_0_weight(rows, cols, seed=rows)
        x = synth.normal(batch, cols, seed=batch)
        dw = dev(w)
        dy, y = quantize_q8_1(x)
        got = run_gemm(dw, dy, rows, cols, batch)
        ref = np.zeros((batch, rows), np.float32)
        absum = np.zeros((batch, rows), np.float32)
        for j0 in range(0, batch, 8):
            m = min(8, batch - j0)
            ysl = y.reshape(batch, -1)[j0:j0 + m].reshape(-1)
            rc, r = oracle.gemv(w, ysl, rows, cols, m)
            rc, a = oracle.gemv_abs(w, ysl, rows, cols, m)
            ref[j0:j0 + m] = r
            absum[j0:j0 + m] = a
        assert_close_fp32(got, ref, absum, f"gemm small {rows}x{batch}x{cols}")


def test_gemm_equals_gemv_at_block_level(gpu, oracle):
    """Same int8 inputs through GEMV (Q8_1) and GEMM (D4) give the same int32 block
    dots whenever both quantizers agree on q (they do when x/d and x*(127/amax)
    round alike); here both are compared with the oracle instead of each other."""
    rows, batch, cols = 256, 8, 1024
    w = synth.q8_0_weight(rows, cols, seed=1)
    x = synth.normal(batch, cols, seed=2)
    dw = dev(w)
    dy1, y1 = quantize_q8_1(x)
    dy4, y4 = quantize_d4(x)
    q1 = y1.reshape(batch, cols // 32, 36)[:, :, 4:]
    q4 = y4.reshape(cols // 128, batch, 144)[:, :, 16:].reshape(cols // 128, batch, 4, 32)
    q4 = q4.transpose(1, 0, 2, 3).reshape(batch, cols // 32, 32)
    same = (q1 == q4).all(axis=2)
    assert same.mean() > 0.9
    for j, kb in zip(*np.nonzero(same)):
        if (j + kb) % 37:
            continue
        a = oracle.block_dot(w, y1, 0, cols, batch, 3, int(j), int(kb))
        b = oracle.block_dot(w, y4, 1, cols, batch, 3, int(j), int(kb))
        assert a == b


def test_gemm_rejections(gpu):
    L = q8mi.lib()
    b = hip.DeviceBuffer(1 << 16)
    assert L.q8mi_gemm(b.ptr, b.ptr, b.ptr, 128, 100, 4, 128, NULL) == q8mi.REJECTED
    assert L.q8mi_gemm(b.ptr, b.ptr, b.ptr, 0, 128, 4, 128, NULL) == q8mi.REJECTED
    assert L.q8mi_gemm(b.ptr, b.ptr, b.ptr, 128, 128, 0, 128, NULL) == q8mi.REJECTED
    assert L.q8mi_gemm_medium(b.ptr, b.ptr, b.ptr, 128, 160, 4, 128, NULL) == q8mi.REJECTED
    assert L.q8mi_gemm_medium(b.ptr, b.ptr, b.ptr, 128, 128, 65, 128, NULL) == q8mi.REJECTED


@pytest.mark.parametrize("rows,cols", [(1000, 256), (333, 1024), (5120, 5120), (640, 17408), (160, 2304),
                                       (12320, 512), (17408, 1024)])
@pytest.mark.parametrize("batch", [33, 48, 64, 65, 100, 128, 200])
def test_gemm_medium_batches(gpu, oracle, rows, cols, batch):
    """Batches too small to fill the chip with 128 x 128 tiles run 32-row tiles behind a ring of
    LDS stages, 32, 64 or 128 activation rows wide, the narrow ones with K split over the waves:
    rows and batch ragged against every tile width, K shorter and much longer than the ring.  The
    last two matrices are tall enough for the 64-row tiles that batches of 33..128 then take (one
    of them ragged against 64 rows)."""
    w = synth.q8_0_weight(rows, cols, seed=rows * 3 + cols)
    x = synth.normal(batch, cols, seed=batch * 17 + cols)
    x[batch // 2, :128] = 0.0
    dw = dev(w)
    dy, y = quantize_d4(x)
    rc, ref = oracle.gemm_d4(w, y, rows, cols, batch, threads=8)
    rr, jj = np.meshgrid(np.arange(rows, dtype=np.uint32), np.arange(batch, dtype=np.uint32))
    rc, _, absum = oracle.gemm_d4_sampled(w, y, rows, cols, batch, rr.reshape(-1), jj.reshape(-1))
    stride = rows + 7
    got = run_gemm(dw, dy, rows, cols, batch, stride=stride)
    assert_close_fp32(got[:, :rows], ref, absum, f"gemm medium batch {batch}")
    assert np.all(got[:, rows:].view(np.uint32) == 0xffffffff), "stores must stay inside the rows"
    again = run_gemm(dw, dy, rows, cols, batch, stride=stride)
    assert np.array_equal(again.view(np.uint32), got.view(np.uint32)), "deterministic"
    if batch <= 64:
        got_m = run_gemm(dw, dy, rows, cols, batch, medium=True)
        assert np.array_equal(got_m.view(np.uint32), got[:, :rows].view(np.uint32))
