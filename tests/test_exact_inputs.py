"""CPU check of the inputs behind the bit-for-bit GPU tests (tests/exact_inputs.py): the oracle's
quantizers return the powers of two and the integers that were put in, and the oracle's fp32 GEMV /
GEMM equal integer arithmetic, also with the blocks added in a shuffled order."""
import numpy as np
import pytest

import exact_inputs as ex


def planes(w, cols):
    nb = cols // 32
    d = w[:, :2 * nb].copy().view(np.float16).astype(np.float64)
    q = w[:, 2 * nb:].view(np.int8).astype(np.int64).reshape(w.shape[0], nb, 32)
    return d, q


@pytest.mark.parametrize("cols", [256, 5120, 17408])
def test_sums_are_exact_in_any_order(oracle, cols):
    rows, batch = 24, 3
    w = ex.weight(rows, cols, seed=cols)
    x = ex.activations(batch, cols, seed=cols + 1)
    nb = cols // 32
    rc, y = oracle.quantize_q8_1(x)
    yb = y.reshape(batch, nb, 36)
    dx = yb[:, :, :2].copy().view(np.float16).astype(np.float64).reshape(batch, nb)
    qx = yb[:, :, 4:].view(np.int8).astype(np.int64)
    assert set(np.unique(dx)) <= {0.5, 1.0}
    assert np.array_equal(qx * dx[..., None], x.reshape(batch, nb, 32).astype(np.float64))
    assert np.all(np.abs(qx).max(axis=2) == 127)
    dw, qw = planes(w, cols)
    S = np.einsum("rki,jki->jrk", qw, qx)                       # int64 block dots
    assert np.abs(S).max() <= ex.W_QMAX * 127 + 31 * ex.W_QMAX * ex.X_QMAX
    terms = S * dw[None, :, :] * dx[:, None, :]                   # exact in float64
    units = terms * 1024.0
    assert np.array_equal(units, np.rint(units)) and np.abs(units).sum(axis=2).max() < 2 ** 24
    rc, ref = oracle.gemv(w, y, rows, cols, batch)
    assert np.array_equal(ref.astype(np.float64), terms.sum(axis=2))
    # fp32 accumulation in a shuffled block order gives the same bits
    perm = np.random.default_rng(5).permutation(nb)
    acc = np.zeros((batch, rows), np.float32)
    for kb in perm:
        acc = (acc + terms[:, :, kb].astype(np.float32)).astype(np.float32)
    assert np.array_equal(acc.view(np.uint32), ref.view(np.uint32))
    # D4 flavour: same integers, scales as fp32 powers of two, same sums
    if cols % 128 == 0:
        rc, y4 = oracle.quantize_q8_1_d4(x)
        y4 = y4.reshape(cols // 128, batch, 144)
        d4 = y4[:, :, :16].copy().view(np.float32).astype(np.float64)         # [sb, j, 4]
        q4 = y4[:, :, 16:].view(np.int8).astype(np.int64).reshape(cols // 128, batch, 4, 32)
        assert np.array_equal(d4.transpose(1, 0, 2).reshape(batch, nb), dx)
        assert np.array_equal(q4.transpose(1, 0, 2, 3).reshape(batch, nb, 32), qx)
        rc, ref4 = oracle.gemm_d4(w, y4.reshape(-1), rows, cols, batch)
        assert np.array_equal(ref4.view(np.uint32), ref.view(np.uint32))


def test_residual_keeps_the_sums_exact():
    r = ex.residual(4, 100, seed=1)
    assert np.array_equal(r * 1024.0, np.rint(r * 1024.0)) and np.abs(r).max() <= 4.0
    # representable in bf16 after truncation?  no: the bf16 tests truncate it themselves; what
    # matters here is that |residual| * 1024 + the largest sum of block terms stays below 2^24
    assert 4096 + ex.MAX_BLOCKS * (ex.W_QMAX * 127 + 31 * ex.W_QMAX * ex.X_QMAX) * 4 < 2 ** 24
