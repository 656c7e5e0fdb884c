"""GPU parity: the tile GEMM's fused stores through the C ABI: residual add (q8mi_gemm_add), bf16
outputs (q8mi_gemm_bf16), the dual-weight SwiGLU form (q8mi_gemm_silu_mul) and the elementwise
q8mi_silu_mul, against the CPU oracle and against the separate launches they replace."""
import numpy as np
import pytest

import q8mi
from gpu_common import NULL, assert_close_fp32, dev, quantize_d4
from q8mi import hip, ok
import q8mi_support as synth

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def gemm(dw, dy, rows, cols, batch):
    out = hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    ok(q8mi.lib().q8mi_gemm(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, rows, NULL), "gemm")
    hip.synchronize()
    return out


def silu64(g, u):
    g, u = np.asarray(g, np.float64), np.asarray(u, np.float64)
    return g / (1.0 + np.exp(-g)) * u


def assert_swiglu_close(got, gref, gabs, uref, uabs, what):
    """silu(g) * u for sums g, u each within the GEMM's tolerance of its oracle value: the bound is
    propagated through the product (|silu'| <= 1.1) plus a few ulp for the fast exponential, whose
    last bit the reference's own __expf does not pin either."""
    got = np.asarray(got, np.float64).reshape(-1)
    gref, uref = np.asarray(gref, np.float64).reshape(-1), np.asarray(uref, np.float64).reshape(-1)
    tg = 1e-5 * np.abs(gref) + 1e-6 * np.asarray(gabs, np.float64).reshape(-1)
    tu = 1e-5 * np.abs(uref) + 1e-6 * np.asarray(uabs, np.float64).reshape(-1)
    want = silu64(gref, uref)
    lim = 1.1 * tg * np.abs(uref) + tu * np.abs(gref) + 1e-6 * np.abs(want)
    bad = np.nonzero(~(np.abs(got - want) <= lim))[0]
    assert bad.size == 0, f"{what}: {bad.size} outputs outside tolerance, first {bad[0]}: got {got[bad[0]]} want {want[bad[0]]}"


def sample_points(rows, batch, n, seed):
    rng = np.random.default_rng(seed)
    sr = rng.integers(0, rows, n, dtype=np.uint32)
    sj = rng.integers(0, batch, n, dtype=np.uint32)
    edges = [(0, 0), (rows - 1, 0), (0, batch - 1), (rows - 1, batch - 1), (rows - 33, batch - 1), (rows // 2, batch // 2),
             (min(63, rows - 1), 0), (min(64, rows - 1), 0)]
    for i, (r, j) in enumerate(edges):
        sr[i], sj[i] = max(r, 0), j
    return sr, sj


# rows of one weight, cols, batch -> which kernel serves it
SILU_SHAPES = [
    (384, 1024, 9),      # matrix-core GEMV on D4 records
    (384, 1024, 16),
    (384, 1024, 20),     # 32 + 32-row ring tiles, one activation group
    (384, 1024, 40),     # two groups
    (384, 1024, 64),
    (1000, 512, 300),    # four groups, ragged rows and batch
    (3328, 512, 512),    # 64 + 64-row main tiles
    (3300, 768, 500),    # main tiles with ragged edges
    (5120, 17408, 12),   # long rows: 12 activation rows do not fit the GEMV's LDS image in one pass
]


@pytest.mark.parametrize("rows,cols,batch", SILU_SHAPES)
def test_gemm_silu_mul(gpu, oracle, rows, cols, batch):
    L = q8mi.lib()
    wg, wu = synth.q8_0_weight(rows, cols, seed=rows + cols), synth.q8_0_weight(rows, cols, seed=rows + cols + 1)
    x = synth.normal(batch, cols, seed=batch + cols)
    dg, du = dev(wg), dev(wu)
    dy, y = quantize_d4(x)
    stride = rows + 8
    out = hip.DeviceBuffer(4 * batch * stride).fill(0xff)
    ok(L.q8mi_gemm_silu_mul(dg.ptr, du.ptr, dy.ptr, out.ptr, rows, cols, batch, stride, NULL), "gemm_silu_mul")
    hip.synchronize()
    got = out.download(np.float32).reshape(batch, stride)
    assert np.all(bits(got[:, rows:]) == 0xffffffff), "stores must stay inside the rows"
    assert np.isfinite(got[:, :rows]).all(), "every output must be written"
    sr, sj = sample_points(rows, batch, 30000, rows + batch)
    rc, gref, gabs = oracle.gemm_d4_sampled(wg, y, rows, cols, batch, sr, sj)
    rc, uref, uabs = oracle.gemm_d4_sampled(wu, y, rows, cols, batch, sr, sj)
    assert_swiglu_close(got[sj, sr], gref, gabs, uref, uabs, f"gemm_silu_mul {rows}x{cols} batch {batch}")
    # all rows of the first and the last activation row: a misplaced tile anywhere along the weight rows
    for j in (0, batch - 1):
        rr = np.arange(rows, dtype=np.uint32)
        jj = np.full(rows, j, np.uint32)
        rc, gref, gabs = oracle.gemm_d4_sampled(wg, y, rows, cols, batch, rr, jj)
        rc, uref, uabs = oracle.gemm_d4_sampled(wu, y, rows, cols, batch, rr, jj)
        assert_swiglu_close(got[j, :rows], gref, gabs, uref, uabs, f"gemm_silu_mul activation row {j}")


@pytest.mark.parametrize("rows,cols,batch", [(384, 1024, 64), (6656, 512, 512)])
def test_gemm_silu_mul_equals_two_gemms_and_silu_mul(gpu, rows, cols, batch):
    """Where the plain GEMM takes tiles of the same kind and sums every output in one piece (no halves
    of K), the dual-weight tile forms the same two sums in the same order: the one-launch form then
    equals q8mi_gemm twice + q8mi_silu_mul bit for bit."""
    L = q8mi.lib()
    dg, du = dev(synth.q8_0_weight(rows, cols, seed=1)), dev(synth.q8_0_weight(rows, cols, seed=2))
    dy, _ = quantize_d4(synth.normal(batch, cols, seed=3))
    g, u = gemm(dg, dy, rows, cols, batch), gemm(du, dy, rows, cols, batch)
    steps = hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    ok(L.q8mi_silu_mul(steps.ptr, g.ptr, u.ptr, batch * rows, NULL), "silu_mul")
    fused = hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    ok(L.q8mi_gemm_silu_mul(dg.ptr, du.ptr, dy.ptr, fused.ptr, rows, cols, batch, rows, NULL), "gemm_silu_mul")
    hip.synchronize()
    assert np.array_equal(bits(fused.download(np.float32)), bits(steps.download(np.float32)))


def test_gemm_silu_mul_prefill_chunk(gpu, oracle):
    """The gate/up projection of a prefill chunk at the model's shape (M=2048, K=5120, N=17408)."""
    rows, cols, batch = 17408, 5120, 2048
    L = q8mi.lib()
    wg, wu = synth.q8_0_weight(rows, cols, seed=11), synth.q8_0_weight(rows, cols, seed=12)
    dg, du = dev(wg), dev(wu)
    dy, y = quantize_d4(synth.normal(batch, cols, seed=13))
    out = hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    ok(L.q8mi_gemm_silu_mul(dg.ptr, du.ptr, dy.ptr, out.ptr, rows, cols, batch, rows, NULL), "gemm_silu_mul")
    hip.synchronize()
    got = out.download(np.float32).reshape(batch, rows)
    assert np.isfinite(got).all()
    sr, sj = sample_points(rows, batch, 20000, 5)
    rc, gref, gabs = oracle.gemm_d4_sampled(wg, y, rows, cols, batch, sr, sj)
    rc, uref, uabs = oracle.gemm_d4_sampled(wu, y, rows, cols, batch, sr, sj)
    assert_swiglu_close(got[sj, sr], gref, gabs, uref, uabs, "gemm_silu_mul prefill chunk")


# rows, cols, batch, in place
ADD_SHAPES = [(384, 1024, 40, True), (384, 1024, 64, False), (1000, 512, 300, True), (6656, 512, 512, True),
              (6656, 512, 500, False), (384, 1024, 12, True), (5120, 5120, 64, True)]


@pytest.mark.parametrize("rows,cols,batch,in_place", ADD_SHAPES)
def test_gemm_add_equals_gemm_then_add(gpu, oracle, rows, cols, batch, in_place):
    """dst = residual + W x in the tile's store: the bits of q8mi_gemm into a temporary followed by
    q8mi_add (what the reference's batched q8_0_matmul_add runs), and within tolerance of the oracle."""
    L = q8mi.lib()
    w = synth.q8_0_weight(rows, cols, seed=rows + 7)
    dw = dev(w)
    dy, y = quantize_d4(synth.normal(batch, cols, seed=batch + 7))
    base = synth.normal(batch, rows, seed=99)
    tmp = gemm(dw, dy, rows, cols, batch)
    want = hip.DeviceBuffer(4 * batch * rows)
    res = dev(base)
    ok(L.q8mi_add(want.ptr, res.ptr, tmp.ptr, batch * rows, 0, NULL), "add")
    dst = res if in_place else hip.DeviceBuffer(4 * batch * rows).fill(0xff)
    keep = dev(base)
    src = dst if in_place else keep
    ok(L.q8mi_gemm_add(dw.ptr, dy.ptr, src.ptr, dst.ptr, rows, cols, batch, rows, NULL), "gemm_add")
    hip.synchronize()
    got = dst.download(np.float32)
    if batch > 16:
        assert np.array_equal(bits(got), bits(want.download(np.float32)))
    if not in_place:
        assert np.array_equal(keep.download(np.float32), base.reshape(-1)), "the residual is left alone"
    sr, sj = sample_points(rows, batch, 20000, 3)
    rc, ref, absum = oracle.gemm_d4_sampled(w, y, rows, cols, batch, sr, sj)
    b = base[sj, sr].astype(np.float64)
    assert_close_fp32(got.reshape(batch, rows)[sj, sr], ref.astype(np.float64) + b, absum + np.abs(b), f"gemm_add {rows}x{cols} batch {batch}")


def test_gemm_add_declines_what_it_cannot_fuse(gpu):
    """Shapes q8mi_gemm sums from two halves of K (and small batches out of place) are declined with
    nothing enqueued, so the caller's two-step route still applies."""
    L = q8mi.lib()
    cases = [(384, 1024, 32, True),      # one 32-row tile per CU at most: cut along K
             (5120, 1024, 2048, True),   # 640 main tiles: the last round of 128 is cut along K
             (17408, 512, 64, True),     # 272 tiles of 64 x 64 for 256 CUs: their K steps are dealt out evenly
             (384, 1024, 12, False)]     # a weight stream adds in place only
    for rows, cols, batch, in_place in cases:
        dw = dev(synth.q8_0_weight(rows, cols, seed=1))
        dy, _ = quantize_d4(synth.normal(batch, cols, seed=2))
        base = synth.normal(batch, rows, seed=3)
        res, other = dev(base), hip.DeviceBuffer(4 * batch * rows).fill(0xff)
        dst = res if in_place else other
        assert L.q8mi_gemm_add(dw.ptr, dy.ptr, res.ptr, dst.ptr, rows, cols, batch, rows, NULL) == q8mi.REJECTED
        hip.synchronize()
        assert np.array_equal(res.download(np.float32), base.reshape(-1))
        assert np.all(bits(other.download(np.float32)) == 0xffffffff)
    dw = dev(synth.q8_0_weight(64, 1024, seed=1))
    assert L.q8mi_gemm_add(dw.ptr, dw.ptr, dw.ptr, dw.ptr, 64, 1024, 40, 64, NULL) == q8mi.REJECTED     # fewer than 128 rows
    assert L.q8mi_gemm_silu_mul(dw.ptr, dw.ptr, dw.ptr, dw.ptr, 256, 384, 40, 256, NULL) == q8mi.REJECTED   # cols % 256
    assert L.q8mi_gemm_bf16(dw.ptr, dw.ptr, dw.ptr, 256, 1024, 8, 256, NULL) == q8mi.REJECTED            # a weight stream


@pytest.mark.parametrize("rows,cols,batch", [(384, 1024, 40), (384, 1024, 64), (1000, 512, 300), (6656, 512, 500)])
def test_gemm_bf16_equals_gemm_then_convert(gpu, rows, cols, batch):
    L = q8mi.lib()
    dw = dev(synth.q8_0_weight(rows, cols, seed=rows + 9))
    dy, _ = quantize_d4(synth.normal(batch, cols, seed=batch + 9))
    tmp = gemm(dw, dy, rows, cols, batch)
    want = hip.DeviceBuffer(2 * batch * rows)
    ok(L.q8mi_f32_to_bf16(tmp.ptr, want.ptr, batch * rows, NULL), "f32_to_bf16")
    stride = rows + 8
    out = hip.DeviceBuffer(2 * batch * stride).fill(0xee)
    ok(L.q8mi_gemm_bf16(dw.ptr, dy.ptr, out.ptr, rows, cols, batch, stride, NULL), "gemm_bf16")
    hip.synchronize()
    got = out.download(np.uint16).reshape(batch, stride)
    assert np.all(got[:, rows:] == 0xeeee)
    assert np.array_equal(got[:, :rows], want.download(np.uint16).reshape(batch, rows))


@pytest.mark.parametrize("n,offset", [(1, 0), (4099, 0), (4099, 1), (1 << 20, 0)])
def test_silu_mul_elementwise(gpu, n, offset):
    """out = silu(gate) * up against float64 (1e-6 relative: a division, a product and the fast
    exponential, whose last bit is not pinned by the reference either); any length and alignment,
    in place over the gate."""
    L = q8mi.lib()
    g = synth.normal(1, n + offset, seed=n) * 4.0
    u = synth.normal(1, n + offset, seed=n + 1)
    g[0, offset] = 0.0
    if n > 3:
        g[0, offset + 1], g[0, offset + 2], g[0, offset + 3] = -80.0, 80.0, -0.0
    dg, du = dev(g), dev(u)
    out = hip.DeviceBuffer(4 * (n + offset + 4)).fill(0xff)
    ok(L.q8mi_silu_mul(out.at(4 * offset), dg.at(4 * offset), du.at(4 * offset), n, NULL), "silu_mul")
    hip.synchronize()
    got = out.download(np.float32)
    want = silu64(g[0, offset:], u[0, offset:])
    assert np.all(bits(got[:offset]) == 0xffffffff) and np.all(bits(got[offset + n:]) == 0xffffffff)
    assert np.all(np.abs(got[offset:offset + n] - want) <= 1e-6 * np.abs(want) + 1e-37)
    ok(L.q8mi_silu_mul(dg.at(4 * offset), dg.at(4 * offset), du.at(4 * offset), n, NULL), "silu_mul in place")
    hip.synchronize()
    assert np.array_equal(bits(dg.download(np.float32)[offset:offset + n]), bits(got[offset:offset + n]))
