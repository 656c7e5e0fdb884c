"""Pins the oracle's dot products, GEMV family and GEMM: brute force, closed forms,
the reference's own tolerance test restated, float64 truth."""
import numpy as np
import pytest

import np_ref


def make(oracle, rows, cols, batch, seed, d4=False):
    rng = np.random.default_rng(seed)
    w = oracle.make_weight((rng.standard_normal((rows, cols)) * 0.02).astype(np.float32))
    x = rng.standard_normal((batch, cols)).astype(np.float32)
    rc, y = (oracle.quantize_q8_1_d4 if d4 else oracle.quantize_q8_1)(x)
    return w, x, y


def test_block_dot_brute_force_and_extremes(oracle):
    rows, cols, batch = 5, 256, 3
    w, x, y = make(oracle, rows, cols, batch, 1)
    _, qw = np_ref.unpack_weight(w, cols)
    _, _, qx = np_ref.unpack_q8_1(y, batch, cols)
    S = np_ref.block_dots(qw, qx)
    for r in range(rows):
        for j in range(batch):
            for kb in range(cols // 32):
                assert oracle.block_dot(w, y, 0, cols, batch, r, j, kb) == S[j, r, kb]
    w4, x4, y4 = make(oracle, rows, cols, batch, 2, d4=True)
    _, qw4 = np_ref.unpack_weight(w4, cols)
    _, qx4 = np_ref.unpack_d4(y4, batch, cols)
    S4 = np_ref.block_dots(qw4, qx4)
    for r in range(rows):
        for j in range(batch):
            for kb in range(cols // 32):
                assert oracle.block_dot(w4, y4, 1, cols, batch, r, j, kb) == S4[j, r, kb]
    # extremes: +-127 * +-127 * 32 = +-516128
    for sw, sx in ((127, 127), (-127, 127), (-127, -127)):
        wq = np.zeros((1, 34), np.uint8)
        wq[0, 2:] = np.int8(sw).view(np.uint8)
        yq = np.zeros(36, np.uint8)
        yq[4:] = np.int8(sx).view(np.uint8)
        assert oracle.block_dot(wq, yq, 0, 32, 1, 0, 0, 0) == sw * sx * 32


def test_gemv_closed_form_of_the_reference(oracle):
    """tests/mixed_linear_parity.cu:205-263: all weight blocks d = 0.5, q = 1 and a constant
    input give cols * 0.5 * x (here through the Q8_1 quantizer: x -> 127 * fp16(x/127))."""
    rows, cols = 9, 2048
    nb = cols // 32
    w = np.zeros((rows, nb * 34), np.uint8)
    w[:, :2 * nb] = np.tile(np.frombuffer(np.float16(0.5).tobytes(), np.uint8), nb)
    w[:, 2 * nb:] = 1
    for batch, xv in ((1, 0.25), (8, 2.0), (3, -1.5)):
        x = np.full((batch, cols), xv, np.float32)
        rc, y = oracle.quantize_q8_1(x)
        rc, out = oracle.gemv(w, y, rows, cols, batch)
        dx = np.float32(np.float16(np.float32(abs(xv)) / np.float32(127)))
        assert np.all(out == np.float32(np.sign(xv) * cols * 0.5 * 127) * dx)
        assert np.allclose(out, cols * 0.5 * xv, rtol=1e-3)
        rc, y4 = oracle.quantize_q8_1_d4(x)
        w128 = np.repeat(w, 15, axis=0)[:128]
        rc, out4 = oracle.gemm_d4(w128, y4, 128, cols, batch)
        assert np.allclose(out4, cols * 0.5 * xv, rtol=1e-6)


@pytest.mark.parametrize("rows,cols,batch", [(4, 32, 1), (7, 256, 8), (33, 1024, 3), (5, 5120, 2)])
def test_gemv_against_float64_truth_and_order(oracle, rows, cols, batch):
    w, x, y = make(oracle, rows, cols, batch, rows + cols)
    dw, qw = np_ref.unpack_weight(w, cols)
    dx, _, qx = np_ref.unpack_q8_1(y, batch, cols)
    rc, out = oracle.gemv(w, y, rows, cols, batch)
    assert rc == 0
    truth = np_ref.linear_f64(dw, qw, dx, qx)
    absum = np.einsum("jrk,rk,jk->jr", np.abs(np_ref.block_dots(qw, qx)).astype(np.float64),
                      dw.astype(np.float64), dx.astype(np.float64))
    nb = cols // 32
    assert np.all(np.abs(out - truth) <= 2.0 ** -23 * nb * absum)           # fp32 accumulation bound
    # the stated order (ascending kb, fma(d_w*d_x, S, acc)) reproduced step by step in numpy
    assert np.array_equal(out, np_ref.linear_f32_ascending(dw, qw, dx, qx))
    rc, ab = oracle.gemv_abs(w, y, rows, cols, batch)
    assert np.allclose(ab, absum, rtol=1e-6)
    # dropping one block, or transposing the operands, must be visible at this tolerance
    wrong = truth - (dw[:, 0][None, :] * dx[:, 0][:, None] * np_ref.block_dots(qw, qx)[:, :, 0])
    assert np.any(np.abs(out - wrong) > 2.0 ** -23 * nb * absum)


def test_gemv_dst_indexing_and_threads(oracle):
    rows, cols, batch = 10, 128, 3
    w, x, y = make(oracle, rows, cols, batch, 5)
    rc, a = oracle.gemv(w, y, rows, cols, batch)
    rc, b = oracle.gemv(w, y, rows, cols, batch, stride=rows + 6)
    assert np.array_equal(a, b[:, :rows]) and np.all(b[:, rows:] == 0)
    rc, c = oracle.gemv(w, y, rows, cols, batch, threads=4)
    assert np.array_equal(a, c)
    # element (j, r) is row r of W against activation row j
    dw, qw = np_ref.unpack_weight(w, cols)
    dx, _, qx = np_ref.unpack_q8_1(y, batch, cols)
    t = np_ref.linear_f64(dw, qw, dx, qx)
    assert np.allclose(a, t, rtol=1e-5, atol=1e-7) and not np.allclose(a.T[:batch, :batch], t[:batch, :batch])
    for bad in ((rows, 100, 1), (rows, cols, 0), (rows, cols, 9)):
        assert oracle.gemv(w, y, *bad)[0] == -1


def test_fused_variants_are_compositions(oracle):
    rows, cols, batch = 24, 512, 4
    w0, x, y = make(oracle, rows, cols, batch, 7)
    w1, _, _ = make(oracle, rows, cols, batch, 8)
    rc, p0 = oracle.gemv(w0, y, rows, cols, batch)
    rc, p1 = oracle.gemv(w1, y, rows, cols, batch)
    rc, t0, t1 = oracle.gemv_two(w0, w1, y, rows, cols, batch)
    assert np.array_equal(t0, p0) and np.array_equal(t1, p1)
    rc, s = oracle.gemv_silu_mul(w0, w1, y, rows, cols, batch)
    g = p0.astype(np.float64)
    want = g / (1 + np.exp(-g)) * p1.astype(np.float64)
    assert np.allclose(s, want, rtol=3e-7, atol=1e-30)
    base = np.random.default_rng(0).standard_normal((batch, rows)).astype(np.float32)
    rc, a = oracle.gemv_add(w0, y, base, rows, cols, batch)
    assert np.array_equal(a, base + p0)
    rc, b16 = oracle.gemv_bf16(w0, y, rows, cols, batch)
    want16 = np.array([oracle.f32_to_bf16(v) for v in p0.reshape(-1)], np.uint16).reshape(batch, rows)
    assert np.array_equal(b16, want16)
    base16 = (base.view(np.uint32) >> 16).astype(np.uint16)
    rc, ab = oracle.gemv_add_bf16(w0, y, base16, rows, cols, batch)
    basef = (base16.astype(np.uint32) << 16).view(np.float32)
    wantab = np.array([oracle.f32_to_bf16(v) for v in (basef + p0).reshape(-1)], np.uint16).reshape(batch, rows)
    assert np.array_equal(ab, wantab)
    # fan-out: slot-wise plain GEMV; null / empty slots skipped; all-empty rejected
    w2 = oracle.make_weight((np.random.default_rng(3).standard_normal((5, cols)) * 0.02).astype(np.float32))
    rc, outs = oracle.gemv_fanout4([w0, None, w2, w1], y, [rows, 0, 5, rows], cols, batch, [rows, 0, 9, rows + 2])
    assert rc == 0
    assert np.array_equal(outs[0], p0) and np.array_equal(outs[3][:, :rows], p1)
    assert np.array_equal(outs[2][:, :5], oracle.gemv(w2, y, 5, cols, batch)[1]) and np.all(outs[2][:, 5:] == 0)
    assert oracle.gemv_fanout4([None] * 4, y, [0, 0, 0, 0], cols, batch)[0] == -1


# a subset of the reference's parity shapes (tests/mmq_parity.cu:275-295) that runs in seconds on CPU
@pytest.mark.parametrize("rows,batch,cols", [(128, 128, 256), (128, 128, 1024), (256, 128, 2048), (640, 223, 2304)])
def test_gemm_reference_tolerance_restated(oracle, rows, batch, cols):
    """tests/mmq_parity.cu:137-143, 246-254: U(-0.5,0.5) weights, U(-1,1) activations; result vs the
    fp32 dot of the dequantised operands within 5e-3 abs or 1e-3 rel."""
    rng = np.random.default_rng(0x5EED + rows)
    wf = rng.uniform(-0.5, 0.5, (rows, cols)).astype(np.float32)
    x = rng.uniform(-1, 1, (batch, cols)).astype(np.float32)
    w = oracle.make_weight(wf)
    rc, y = oracle.quantize_q8_1_d4(x)
    rc, out = oracle.gemm_d4(w, y, rows, cols, batch, threads=8)
    assert rc == 0
    dw, qw = np_ref.unpack_weight(w, cols)
    dy, qy = np_ref.unpack_d4(y, batch, cols)
    deq_w = (qw.astype(np.float32) * dw[:, :, None]).reshape(rows, cols)
    deq_x = (qy.astype(np.float32) * dy[:, :, None]).reshape(batch, cols)
    ref = deq_x @ deq_w.T
    d = np.abs(out - ref)
    assert np.all((d <= 5e-3) | (d <= 1e-3 * np.maximum(np.abs(ref), 1e-6)))
    # and against float64 truth of the Q8 semantics, at the fp32 accumulation bound
    truth = np_ref.linear_f64(dw, qw, dy, qy)
    absum = np.einsum("jrk,rk,jk->jr", np.abs(np_ref.block_dots(qw, qy)).astype(np.float64),
                      dw.astype(np.float64), dy.astype(np.float64))
    assert np.all(np.abs(out - truth) <= 2.0 ** -23 * (cols // 32) * absum)
    if rows * batch <= 128 * 128:
        assert np.array_equal(out, np_ref.linear_f32_ascending(dw, qw, dy, qy))
    # sampled variant returns the same numbers
    sr = rng.integers(0, rows, 100, dtype=np.uint32)
    sj = rng.integers(0, batch, 100, dtype=np.uint32)
    rc, s, ab = oracle.gemm_d4_sampled(w, y, rows, cols, batch, sr, sj)
    assert np.array_equal(s, out[sj, sr]) and np.allclose(ab, absum[sj, sr], rtol=1e-6)


def test_gemm_gates(oracle):
    w, x, y = make(oracle, 128, 256, 4, 1, d4=True)
    assert oracle.gemm_d4(w, y, 128, 160, 4)[0] == -1
    assert oracle.gemm_d4(w, y, 0, 256, 4)[0] == -1
    assert oracle.gemm_d4(w, y, 128, 256, 0)[0] == -1


def test_heavy_tail_headroom(oracle):
    """Config-4 style activations: int32 block dots stay within +-516128 and the
    scales stay finite in fp32 (D4) while Q8_1's fp16 s may overflow to inf."""
    rng = np.random.default_rng(11)
    x = (rng.standard_t(3, (32, 1024)) / np.sqrt(3)).astype(np.float32)
    x[:, rng.choice(1024, 2, replace=False)] *= 20
    w = oracle.make_weight((rng.standard_normal((128, 1024)) * 0.02).astype(np.float32))
    rc, y = oracle.quantize_q8_1_d4(x)
    _, qw = np_ref.unpack_weight(w, 1024)
    dy, qy = np_ref.unpack_d4(y, 32, 1024)
    assert np.abs(np_ref.block_dots(qw, qy)).max() <= 516128
    assert np.isfinite(dy).all()
    rc, out = oracle.gemm_d4(w, y, 128, 1024, 32)
    assert np.isfinite(out).all()
