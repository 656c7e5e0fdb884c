"""Pins the oracle's RMS norm without running the reference: float64 truth, closed forms that a
dropped term / wrong divisor / misplaced eps would break, the power-of-two scaling law, and an
independent numpy restatement of its summation order (bit-exact)."""
from fractions import Fraction

import numpy as np
import pytest

SIZES = [1, 3, 4, 31, 257, 1024, 1027, 5120, 6144, 17408]


def rows_of(n, batch, seed):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((batch, n)) * rng.uniform(0.05, 30.0, (batch, 1))).astype(np.float32)
    w = rng.uniform(0.2, 2.0, n).astype(np.float32) * rng.choice([-1.0, 1.0], n).astype(np.float32)
    return x, w


@pytest.mark.parametrize("n", SIZES)
def test_against_float64_truth(oracle, n):
    x, w = rows_of(n, 3, seed=n)
    eps = 1e-6
    got = oracle.rms_norm(x, w, eps)
    x64 = x.astype(np.float64)
    truth = x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + eps) * w.astype(np.float64)
    # sum of squares: relative error of about sqrt(log2 n) ulp; root, quotient and two products: 3 more
    assert np.all(np.abs(got - truth) <= 6 * 2.0 ** -24 * np.abs(truth) + 1e-40)


def test_closed_forms(oracle):
    n = 4096
    w = np.arange(1, n + 1, dtype=np.float32)
    # constant 0.5: mean of squares 0.25 exactly, eps 0 -> scale 2 -> out = w
    out = oracle.rms_norm(np.full((1, n), 0.5, np.float32), w, 0.0)
    assert np.array_equal(out[0], w)
    # alternating +-1: mean 1; eps 3 -> scale 0.5 exactly -> out = +-w/2 (eps inside the root, after the mean)
    x = np.where(np.arange(n) % 2 == 0, 1.0, -1.0).astype(np.float32)[None, :]
    out = oracle.rms_norm(x, w, 3.0)
    assert np.array_equal(out[0], x[0] * 0.5 * w)
    # one spike of 64 in 4096 zeros: mean = 1 -> only that output is non-zero and equals 64 * w
    x = np.zeros((1, n), np.float32)
    x[0, 1234] = 64.0
    out = oracle.rms_norm(x, w, 0.0)
    assert out[0, 1234] == 64.0 * w[1234] and np.count_nonzero(out) == 1
    # the divisor is the row length, not the padded length: n = 3, x = (2, 2, 2) -> mean 4 -> scale 0.5
    out = oracle.rms_norm(np.full((1, 3), 2.0, np.float32), np.ones(3, np.float32), 0.0)
    assert np.array_equal(out[0], np.ones(3, np.float32))


@pytest.mark.parametrize("n", [257, 5120])
def test_power_of_two_scaling_law(oracle, n):
    """x -> 4x with eps -> 16 eps multiplies every intermediate by a power of two: same output bits."""
    x, w = rows_of(n, 2, seed=5 * n)
    a = oracle.rms_norm(x, w, 1e-5)
    b = oracle.rms_norm(4.0 * x, w, np.float32(1e-5) * np.float32(16.0))
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_rows_and_strides(oracle):
    x, w = rows_of(96, 4, seed=9)
    wide = np.full((4, 128), 7.0, np.float32)
    wide[:, :96] = x
    a = oracle.rms_norm(x, w, 1e-6)
    b = oracle.rms_norm(wide, w, 1e-6, cols=96, stride=128)
    assert np.array_equal(a, b)
    for j in range(4):
        assert np.array_equal(a[j], oracle.rms_norm(x[j:j + 1], w, 1e-6)[0])


def fma32(a, b, c):
    """round_fp32(a * b + c) for fp32 arrays: the product is exact in float64; the rare sums whose
    float64 rounding lands on an fp32 tie (double rounding) are redone exactly."""
    s = a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)
    r = s.astype(np.float32)
    tie = (s.view(np.uint64) & np.uint64((1 << 29) - 1)) == np.uint64(1 << 28)
    for i in np.flatnonzero(tie):
        exact = Fraction(float(a.flat[i])) * Fraction(float(b.flat[i])) + Fraction(float(c.flat[i]))
        lo, hi = np.nextafter(r.flat[i], -np.inf), np.nextafter(r.flat[i], np.inf)
        r.flat[i] = min((lo, r.flat[i], hi), key=lambda v: abs(Fraction(float(v)) - exact))
    return r


def numpy_restatement(x, w, eps):
    n = x.size
    padded = -(-n // 1024) * 1024
    v = np.zeros(padded, np.float32)
    v[:n] = x
    v = v.reshape(-1, 256, 4)                       # [trip][partial][element]
    q = v[:, :, 0] * v[:, :, 0]
    for e in (1, 2, 3):
        q = fma32(v[:, :, e], v[:, :, e], q)
    p = np.zeros(256, np.float32)
    for trip in q:
        p = p + trip
    while p.size > 1:
        p = p[0::2] + p[1::2]
    scale = np.float32(1.0) / np.sqrt(p[0] / np.float32(n) + np.float32(eps))
    return (x * scale) * w


@pytest.mark.parametrize("n", SIZES)
def test_summation_order_restated_in_numpy(oracle, n):
    x, w = rows_of(n, 2, seed=100 + n)
    got = oracle.rms_norm(x, w, 1e-6)
    for j in range(2):
        assert np.array_equal(got[j].view(np.uint32), numpy_restatement(x[j], w, 1e-6).view(np.uint32))
