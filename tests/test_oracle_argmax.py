"""Pins the oracle's argmax variants and the greedy accept rule."""
import itertools

import numpy as np
import pytest


def textbook(row):
    best, idx = -np.inf, -1
    for i, v in enumerate(row):
        if v > best:
            best, idx = v, i
    return np.float32(best), idx


@pytest.mark.parametrize("n", [1, 2, 255, 256, 257, 1024, 1025, 5000])
def test_argmax_row_textbook(oracle, n):
    rng = np.random.default_rng(n)
    r = rng.standard_normal(n).astype(np.float32)
    v, i = oracle.argmax_row(r)
    assert i == int(np.argmax(r)) and v == r.max()
    r[[0, n // 2, n - 1]] = r.max() + 1                       # ties -> lowest index
    assert oracle.argmax_row(r)[1] == 0
    r2 = np.full(n, -np.inf, np.float32)
    assert oracle.argmax_row(r2) == (np.float32(-np.inf), -1)   # nothing above -inf
    r3 = rng.standard_normal(n).astype(np.float32)
    r3[::3] = np.nan                                           # NaN never wins a `>`
    v, i = oracle.argmax_row(r3)
    assert (v, i) == textbook(r3)
    if n > 1:
        assert not np.isnan(v)


def test_argmax_row_empty(oracle):
    assert oracle.argmax_row(np.zeros(0, np.float32)) == (np.float32(-np.inf), -1)


@pytest.mark.parametrize("row_stride", [1, 100, 256, 257, 1000, 248320])
def test_argmax_rows_nan_free_equals_scan(oracle, row_stride):
    rng = np.random.default_rng(row_stride)
    batch = 4
    x = rng.standard_normal((batch, row_stride)).astype(np.float32)
    x[1, [0, row_stride // 2, row_stride - 1]] = 10.0         # ties
    x[2, :] = 0.0                                              # all equal -> index 0
    rc, got = oracle.argmax_rows(x, batch, row_stride)
    assert rc == 0
    scan = oracle.argmax_rows_scan(x, batch, row_stride)
    assert np.array_equal(got["index"], scan["index"]) and np.array_equal(got["value"], scan["value"])
    assert np.array_equal(got["index"], np.argmax(x, axis=1))


def test_argmax_rows_documented_differences(oracle):
    """The two-stage network (src/kernels_cuda.cu:1765-1802) differs from the scan on rows
    with nothing above -inf (it returns index 0, not -1) and keeps a NaN that sits in the
    lower slot of a comparison; both follow from its rule 'a valid index beats none, then >'."""
    x = np.full((1, 600), -np.inf, np.float32)
    rc, got = oracle.argmax_rows(x, 1, 600)
    assert got["index"][0] == 0 and got["value"][0] == -np.inf
    assert oracle.argmax_rows_scan(x, 1, 600)["index"][0] == -1
    # NaN at column 0 is never displaced (nothing is > NaN); by hand: slot 0 survives every level
    x = np.arange(600, dtype=np.float32)[None, :].copy()
    x[0, 0] = np.nan
    rc, got = oracle.argmax_rows(x, 1, 600)
    assert got["index"][0] == 0 and np.isnan(got["value"][0])
    # NaN at column 1 loses at stride 1 only if slot 0 holds something; before that it has
    # absorbed slots 3, 5, ... ; slot 0 holds max of even slots of block 0 -> the winner of
    # block 0 is the best even column, then later blocks win on value
    x = np.zeros((1, 256), np.float32)
    x[0, 1] = np.nan
    x[0, 7] = 5.0            # odd column: compared against the NaN chain and lost
    x[0, 6] = 3.0
    rc, got = oracle.argmax_rows(x, 1, 256)
    assert got["index"][0] == 6 and got["value"][0] == 3.0
    assert oracle.argmax_rows(x, 1, 0)[0] == -1
    assert oracle.argmax_rows(np.zeros((1, 1), np.float32), 1, 1024 * 256 + 1)[0] == -1


def test_accept_brute_force(oracle):
    """src/qwen_native_backend.cpp:15948-15960, 16048-16052 over every (M, prefix) pair and
    every match pattern of up to 7 drafts."""
    eos = 99
    for m in range(1, 9):
        n = m - 1
        tokens = np.arange(10, 10 + m, dtype=np.int32)
        for pattern in itertools.product([True, False], repeat=n):
            drafts = np.array([tokens[i] if ok else tokens[i] + 1000 for i, ok in enumerate(pattern)], np.int32)
            want = 0
            while want < n and pattern[want]:
                want += 1
            got, nxt = oracle.accept(tokens, drafts, eos)
            assert got == want and nxt == tokens[want]
    # a negative argmax (empty row) stands for eos, both when compared and when emitted
    tokens = np.array([-1, 5, -1], np.int32)
    assert oracle.accept(tokens, np.array([eos, 5], np.int32), eos) == (2, eos)
    assert oracle.accept(tokens, np.array([7, 5], np.int32), eos) == (0, eos)
