"""GPU parity: argmax kernels and the fused LM head + greedy accept, bit-exact."""
import ctypes as C

import numpy as np
import pytest

import q8mi
from gpu_common import NULL, assert_close_fp32, dev, quantize_q8_1
from q8mi import hip, ok
import q8mi_support as synth

pytestmark = pytest.mark.gpu

PAIR = np.dtype([("value", np.float32), ("index", np.int32)])


def adversarial_rows(n, seed):
    rng = np.random.default_rng(seed)
    rows = []
    r = rng.standard_normal(n).astype(np.float32)
    rows.append(r.copy())
    t = r.copy(); m = t.max(); t[[n // 3, n // 2, n - 1]] = m + 1.0     # ties of the maximum
    rows.append(t)
    rows.append(np.full(n, -np.inf, np.float32))                          # nothing above -inf
    t = np.full(n, -np.inf, np.float32); t[n - 1] = -1e30
    rows.append(t)
    rows.append(np.zeros(n, np.float32))                                  # all equal
    t = np.zeros(n, np.float32); t[1::2] = -0.0
    rows.append(t)
    t = r.copy(); t[::5] = np.nan                                         # NaN never wins a `>`
    rows.append(t)
    t = r.copy(); t[0] = np.nan; t[n - 1] = np.nan; t[255 % n] = np.nan
    rows.append(t)
    t = r.copy(); t[n // 2] = np.inf
    rows.append(t)
    return np.stack(rows)


@pytest.mark.parametrize("n", [1, 31, 256, 1024, 1025, 32771, 81919, 81920, 81923, 248320, 262147])
def test_argmax_single_row(gpu, oracle, n):
    rows = adversarial_rows(n, seed=n)
    L = q8mi.lib()
    out2 = hip.DeviceBuffer(8)
    pairs = hip.DeviceBuffer(8 * 4)
    for i, r in enumerate(rows):
        dx = dev(r)
        ok(L.q8mi_argmax(dx.ptr, n, out2.ptr, NULL), "argmax")
        ok(L.q8mi_argmax_to_pair(dx.ptr, n, pairs.ptr, i % 4, NULL), "argmax_to_pair")
        hip.synchronize()
        got = out2.download(np.int32)
        v, idx = oracle.argmax_row(r)
        assert got[0] == idx, f"row {i}: index {got[0]} != {idx}"
        assert got[1] == np.float32(v).view(np.int32), f"row {i}: value bits differ"
        p = pairs.download(PAIR)[i % 4]
        assert p["index"] == idx and p["value"].view(np.int32) == np.float32(v).view(np.int32)


@pytest.mark.parametrize("n", [5, 1027, 70001, 100003])
def test_argmax_single_row_off_a_16_byte_boundary(gpu, oracle, n):
    """Rows on a 16-byte boundary are scanned four elements per load, others one by one: same result."""
    rows = adversarial_rows(n, seed=n + 7)
    L = q8mi.lib()
    out2 = hip.DeviceBuffer(8)
    for i, r in enumerate(rows):
        for offset in (4, 8, 12):
            shifted = hip.DeviceBuffer(4 * n + 16)
            shifted.upload(r, offset)
            ok(L.q8mi_argmax(shifted.ptr + offset, n, out2.ptr, NULL), "argmax")
            hip.synchronize()
            got = out2.download(np.int32)
            v, idx = oracle.argmax_row(r)
            assert got[0] == idx and got[1] == np.float32(v).view(np.int32), f"row {i}, offset {offset}"


def test_argmax_empty_row(gpu):
    out2 = hip.DeviceBuffer(8)
    ok(q8mi.lib().q8mi_argmax(out2.ptr, 0, out2.ptr, NULL), "argmax")
    hip.synchronize()
    got = out2.download(np.int32)
    assert got[0] == -1 and got[1] == np.float32(-np.inf).view(np.int32)


@pytest.mark.parametrize("row_stride", [1, 255, 256, 257, 5000, 248320])
def test_argmax_rows_matches_reference_network(gpu, oracle, row_stride):
    rows = adversarial_rows(row_stride, seed=row_stride + 1)
    batch = rows.shape[0]
    L = q8mi.lib()
    scratch = hip.DeviceBuffer(L.q8mi_argmax_rows_scratch_bytes(batch, row_stride))
    res = hip.DeviceBuffer(8 * batch)
    dx = dev(rows)
    ok(L.q8mi_argmax_rows(dx.ptr, batch, row_stride, scratch.ptr, res.ptr, NULL), "argmax_rows")
    hip.synchronize()
    got = res.download(PAIR)
    rc, ref = oracle.argmax_rows(rows, batch, row_stride)
    assert rc == 0
    assert np.array_equal(got["index"], ref["index"])
    assert np.array_equal(got["value"].view(np.int32), ref["value"].view(np.int32))


def test_argmax_rows_rejections(gpu):
    L = q8mi.lib()
    b = hip.DeviceBuffer(64)
    assert L.q8mi_argmax_rows(b.ptr, 2, 0, b.ptr, b.ptr, NULL) == q8mi.REJECTED
    assert L.q8mi_argmax_rows(b.ptr, 2, 1024 * 256 + 1, b.ptr, b.ptr, NULL) == q8mi.REJECTED


def run_lm_head(w_dev, y_dev, vocab, cols, batch, drafts, eos, want_logits=False, on_device=False):
    L = q8mi.lib()
    scratch = hip.DeviceBuffer(L.q8mi_lm_head_scratch_bytes(vocab, cols, batch))
    row_out = hip.DeviceBuffer(8 * batch)
    acc = hip.DeviceBuffer(8)
    logits = hip.DeviceBuffer(4 * batch * vocab) if want_logits else None
    d = np.ascontiguousarray(drafts, np.int32)
    if on_device:
        dd = dev(d) if d.size else None
        dptr = dd.ptr if dd is not None else None
    else:
        dptr = d.ctypes.data_as(C.c_void_p) if d.size else None
    ok(L.q8mi_lm_head_argmax_accept(w_dev.ptr, y_dev.ptr, vocab, cols, batch, dptr, 1 if on_device else 0,
                                    eos, row_out.ptr, acc.ptr, logits.ptr if logits else None, vocab,
                                    scratch.ptr, NULL), "lm_head")
    hip.synchronize()
    pairs = row_out.download(PAIR)
    a = acc.download(np.int32)
    lg = logits.download(np.float32).reshape(batch, vocab) if want_logits else None
    return pairs, int(a[0]), int(a[1]), lg


@pytest.mark.parametrize("batch", [1, 2, 4, 6, 8])
def test_lm_head_fused_matches_unfused_and_oracle(gpu, oracle, batch):
    vocab, cols = 20000, 1024
    w = synth.q8_0_weight(vocab, cols, seed=500)
    x = synth.normal(batch, cols, seed=600 + batch)
    dw = dev(w)
    dy, y = quantize_q8_1(x)
    rc, ref_logits = oracle.gemv(w, y, vocab, cols, batch)
    ref_pairs = oracle.argmax_rows_scan(ref_logits, batch, vocab)
    ref_tokens = ref_pairs["index"]
    rng = np.random.default_rng(batch)
    for prefix in range(batch):            # forced-match prefix of every possible length
        drafts = rng.integers(0, vocab, batch - 1).astype(np.int32)
        drafts[:prefix] = ref_tokens[:prefix]
        if prefix < batch - 1 and drafts[prefix] == ref_tokens[prefix]:
            drafts[prefix] = (drafts[prefix] + 1) % vocab
        exp_len, exp_next = oracle.accept(ref_tokens, drafts, eos=2)
        assert exp_len == prefix
        for on_device in (False, True):
            pairs, n_acc, nxt, lg = run_lm_head(dw, dy, vocab, cols, batch, drafts, 2,
                                                want_logits=(prefix == 0), on_device=on_device)
            assert np.array_equal(pairs["index"], ref_tokens), "row argmax tokens differ"
            assert n_acc == exp_len and nxt == exp_next
            # winning logits are the GPU's own fp32 values: within tolerance of the oracle's
            assert np.allclose(pairs["value"], ref_pairs["value"], rtol=1e-5, atol=1e-6)
            if lg is not None:
                # the winners are the kernel's own logits; every logit is within the GEMV's tolerance
                # of the oracle's, and one row (where head and GEMV add in the same order) equals the
                # plain GEMV's bit for bit
                assert np.array_equal(pairs["value"].view(np.uint32),
                                      lg[np.arange(batch), pairs["index"]].view(np.uint32))
                rc, mag = oracle.gemv_abs(w, y, vocab, cols, batch)
                assert_close_fp32(lg, ref_logits, mag, f"fused head logits, batch {batch}")
                if batch == 1:
                    out = hip.DeviceBuffer(4 * batch * vocab)
                    ok(q8mi.lib().q8mi_gemv(dw.ptr, dy.ptr, out.ptr, vocab, cols, batch, vocab, NULL), "gemv")
                    hip.synchronize()
                    plain = out.download(np.float32).reshape(batch, vocab)
                    assert np.array_equal(lg.view(np.uint32), plain.view(np.uint32))


def test_lm_head_ties_and_eos(gpu, oracle):
    """Duplicate weight rows give exactly equal logits: the lowest token id must win,
    whichever workgroup met it first."""
    vocab, cols, batch = 6000, 512, 3
    w = synth.q8_0_weight(vocab, cols, seed=9)
    x = synth.normal(batch, cols, seed=10)
    dy, y = quantize_q8_1(x)
    rc, logits = oracle.gemv(w, y, vocab, cols, batch)
    top = int(np.argmax(logits[0]))
    for dup in (5, 4097, 5999):
        if dup != top:
            w[dup] = w[top]
    dw = dev(w)
    rc, logits = oracle.gemv(w, y, vocab, cols, batch)
    ref = oracle.argmax_rows_scan(logits, batch, vocab)
    assert ref["index"][0] == min(top, 5)
    pairs, n_acc, nxt, _ = run_lm_head(dw, dy, vocab, cols, batch, ref["index"][:2], eos=7)
    assert np.array_equal(pairs["index"], ref["index"])
    assert n_acc == 2 and nxt == ref["index"][2]


def test_lm_head_rejections(gpu):
    L = q8mi.lib()
    b = hip.DeviceBuffer(1 << 16)
    d = np.zeros(8, np.int32).ctypes.data_as(C.c_void_p)
    args = lambda rows, cols, batch: (b.ptr, b.ptr, rows, cols, batch, d, 0, 0, b.ptr, b.ptr, None, rows, b.ptr, NULL)
    assert L.q8mi_lm_head_argmax_accept(*args(100, 500, 2)) == q8mi.REJECTED
    assert L.q8mi_lm_head_argmax_accept(*args(100, 512, 0)) == q8mi.REJECTED
    assert L.q8mi_lm_head_argmax_accept(*args(100, 512, 9)) == q8mi.REJECTED
    assert L.q8mi_lm_head_argmax_accept(*args(0, 512, 2)) == q8mi.REJECTED


# ---- the real LM head: 248 320 tokens x 5120 columns (1.35 GB of weights) ------------------------
FULL_VOCAB, FULL_COLS = 248320, 5120


@pytest.fixture(scope="module")
def full_head(gpu):
    w = synth.q8_0_weight(FULL_VOCAB, FULL_COLS, seed=4242)
    return w, dev(w)


@pytest.mark.parametrize("batch", [1, 2, 4, 6, 8])
def test_lm_head_full_vocabulary(gpu, oracle, full_head, batch):
    """The model's LM head.  The oracle runs the whole 248 320 x 5120 head (row-parallel, well under
    a second per activation row): (1) its argmax is the expected token of each verify row, (2) the
    plain GEMV's logits and the fused head's own optional logits are held against it on every row,
    (3) the fused head must return those tokens and the accept length of every forced-match prefix."""
    L = gpu.lib()
    w, dw = full_head
    x = synth.normal(batch, FULL_COLS, seed=700 + batch)
    dy, y = quantize_q8_1(x)
    rc, ref = oracle.gemv(w, y, FULL_VOCAB, FULL_COLS, batch, threads=16)
    rc, absum = oracle.gemv_abs(w, y, FULL_VOCAB, FULL_COLS, batch)
    ref_pairs = oracle.argmax_rows_scan(ref, batch, FULL_VOCAB)
    tokens = ref_pairs["index"]
    # top-2 gaps of this seed are far above the fp32 tolerance, so the tokens are unambiguous
    top2 = np.partition(ref, -2, axis=1)[:, -2:]
    assert np.all(top2[:, 1] - top2[:, 0] > 1e-4 * np.abs(top2[:, 1]))
    logits_dev = hip.DeviceBuffer(4 * batch * FULL_VOCAB)
    ok(L.q8mi_gemv(dw.ptr, dy.ptr, logits_dev.ptr, FULL_VOCAB, FULL_COLS, batch, FULL_VOCAB, NULL), "gemv")
    hip.synchronize()
    assert_close_fp32(logits_dev.download(np.float32), ref, absum, "LM-head logits, plain GEMV, every row")
    rng = np.random.default_rng(batch)
    for prefix in sorted({0, batch // 2, batch - 1}):
        drafts = rng.integers(0, FULL_VOCAB, batch - 1).astype(np.int32)
        drafts[:prefix] = tokens[:prefix]
        if prefix < batch - 1 and drafts[prefix] == tokens[prefix]:
            drafts[prefix] = (drafts[prefix] + 1) % FULL_VOCAB
        exp_len, exp_next = oracle.accept(tokens, drafts, eos=2)
        assert exp_len == prefix
        pairs, n_acc, nxt, lg = run_lm_head(dw, dy, FULL_VOCAB, FULL_COLS, batch, drafts, 2, want_logits=(prefix == 0),
                                            on_device=(prefix % 2 == 1))
        assert np.array_equal(pairs["index"], tokens), "row argmax tokens differ"
        assert n_acc == exp_len and nxt == exp_next
        want = ref[np.arange(batch), tokens]
        assert np.all(np.abs(pairs["value"] - want) <= 1e-5 * np.abs(want) + 1e-6 * absum[np.arange(batch), tokens])
        if lg is not None:
            assert_close_fp32(lg, ref, absum, "LM-head logits, fused head, every row")
            assert np.array_equal(pairs["value"].view(np.uint32), lg[np.arange(batch), tokens].view(np.uint32))


@pytest.mark.parametrize("batch", [3, 5, 8])
def test_lm_head_several_rounds_ragged(gpu, oracle, batch):
    """A head whose workgroups take their units in several whole rounds and a partial one (97 or 98
    units of two items per workgroup), with a row count that is no multiple of four: tokens, accept
    result and every logit against the oracle, with and without the optional logits."""
    vocab, cols = 100003, 2048
    w = synth.q8_0_weight(vocab, cols, seed=1300)
    x = synth.normal(batch, cols, seed=1310 + batch)
    dw = dev(w)
    dy, y = quantize_q8_1(x)
    rc, ref = oracle.gemv(w, y, vocab, cols, batch, threads=16)
    rc, absum = oracle.gemv_abs(w, y, vocab, cols, batch)
    tokens = oracle.argmax_rows_scan(ref, batch, vocab)["index"]
    top2 = np.partition(ref, -2, axis=1)[:, -2:]
    assert np.all(top2[:, 1] - top2[:, 0] > 1e-4 * np.abs(top2[:, 1]))
    for prefix, want_logits in ((0, True), (batch - 1, False)):
        drafts = np.full(batch - 1, 7, np.int32)
        drafts[:prefix] = tokens[:prefix]
        if prefix < batch - 1 and drafts[prefix] == tokens[prefix]:
            drafts[prefix] = 8
        exp_len, exp_next = oracle.accept(tokens, drafts, eos=2)
        pairs, n_acc, nxt, lg = run_lm_head(dw, dy, vocab, cols, batch, drafts, 2, want_logits=want_logits, on_device=False)
        assert np.array_equal(pairs["index"], tokens), "row argmax tokens differ"
        assert (n_acc, nxt) == (exp_len, exp_next)
        if lg is not None:
            assert_close_fp32(lg, ref, absum, f"fused head logits, ragged head, batch {batch}")
            assert np.array_equal(pairs["value"].view(np.uint32), lg[np.arange(batch), tokens].view(np.uint32))


@pytest.mark.parametrize("batch", [2, 4, 7])
def test_lm_head_rows_without_a_number(gpu, oracle, batch):
    """Logits that are NaN never win and a verify row with nothing above -inf has no token (-1, read
    as eos by the accept rule), whichever lane, wave or workgroup meets them first: weight rows
    with a NaN scale at both ends and in the middle of the vocabulary, and one activation row whose
    every block scale is NaN.  Batch 2 runs the dot-product kernel, 4 and 7 the matrix-core one."""
    vocab, cols, eos = 20000, 1024, 3
    dead = batch - 2                       # the activation row whose logits are all NaN
    w = synth.q8_0_weight(vocab, cols, seed=31).copy()
    x = synth.normal(batch, cols, seed=32 + batch)
    dy, y = quantize_q8_1(x)
    y = y.copy()
    nb = cols // 32
    rc, clean = oracle.gemv(w, y, vocab, cols, batch)
    tops = [int(np.argmax(clean[j])) for j in range(batch)]
    nan_rows = sorted({0, 1, 63, 64, 4095, 4096, 9999, vocab - 2, vocab - 1, tops[0], tops[-1]})
    nan16 = np.frombuffer(np.uint16(0x7e00).tobytes(), np.uint8)
    wv = w.reshape(vocab, nb * 34)
    for r in nan_rows:
        wv[r, 0:2] = nan16                 # fp16 NaN scale of the row's first block
    y.reshape(batch, nb, 36)[dead, :, 0:2] = nan16
    dw, dyp = dev(w), dev(y)
    rc, logits = oracle.gemv(w, y, vocab, cols, batch)
    assert np.isnan(logits[:, nan_rows]).all() and np.isnan(logits[dead]).all()
    want_tok, want_val = [], []
    for j in range(batch):
        row = np.where(np.isnan(logits[j]), -np.inf, logits[j])
        t = int(np.argmax(row)) if np.isfinite(row).any() else -1
        want_tok.append(t)
        want_val.append(row[t] if t >= 0 else -np.inf)
    assert want_tok[dead] == -1 and want_tok[-1] != tops[-1]
    live = [j for j in range(batch) if j != dead]
    for prefix in sorted({0, dead, batch - 1}):
        drafts = np.array([(t if t >= 0 else eos) for t in want_tok[:batch - 1]], np.int32)
        if prefix < batch - 1:
            drafts[prefix] = (drafts[prefix] + 1) % vocab
        for on_device in (False, True):
            pairs, n_acc, nxt, _ = run_lm_head(dw, dyp, vocab, cols, batch, drafts, eos, on_device=on_device)
            assert list(pairs["index"]) == want_tok
            assert pairs["value"][dead] == -np.inf
            assert np.allclose(pairs["value"][live], np.array(want_val)[live], rtol=1e-5, atol=1e-6)
            assert n_acc == prefix
            assert nxt == (want_tok[prefix] if want_tok[prefix] >= 0 else eos)
