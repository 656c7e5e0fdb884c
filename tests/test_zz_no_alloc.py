"""GPU test of the LM-head entry point that allocates nothing (q8mi_lm_head_argmax_accept_static:
its per-workgroup partials live in a static device array of the library) against the entry point
that takes a caller-allocated scratch buffer: same row winners, same accept result, same optional
logits, bit for bit, on two calls in a row of which the second is smaller (fewer vocabulary rows,
fewer verify rows), so that partials left over from the first call would show if they were read."""
import ctypes as C

import numpy as np
import pytest

import q8mi
import q8mi_support as synth
from gpu_common import NULL, dev, quantize_q8_1
from q8mi import hip, ok

pytestmark = pytest.mark.gpu

PAIR = np.dtype([("value", np.float32), ("index", np.int32)])


def run(entry, dw, dy, vocab, cols, batch, drafts, eos, scratch):
    L = q8mi.lib()
    row_out, acc = hip.DeviceBuffer(8 * batch).fill(0xff), hip.DeviceBuffer(8).fill(0xff)
    logits = hip.DeviceBuffer(4 * batch * vocab).fill(0xff)
    d = np.ascontiguousarray(drafts, np.int32)
    dptr = d.ctypes.data_as(C.c_void_p) if d.size else None
    if entry == "static":
        ok(L.q8mi_lm_head_argmax_accept_static(dw.ptr, dy.ptr, vocab, cols, batch, dptr, 0, eos, row_out.ptr, acc.ptr,
                                               logits.ptr, vocab, NULL), "lm_head static")
    else:
        ok(L.q8mi_lm_head_argmax_accept(dw.ptr, dy.ptr, vocab, cols, batch, dptr, 0, eos, row_out.ptr, acc.ptr,
                                        logits.ptr, vocab, scratch.ptr, NULL), "lm_head")
    hip.synchronize()
    return row_out.download(PAIR), acc.download(np.int32), logits.download(np.uint32)


def test_static_scratch_entry_point_matches_the_allocating_one(gpu, oracle):
    L = q8mi.lib()
    cols = 1024
    # first call: many workgroups and eight verify rows; second: a smaller head and three rows
    for vocab, batch, seed in ((60000, 8, 1), (3000, 3, 2)):
        w = synth.q8_0_weight(vocab, cols, seed=900 + seed)
        x = synth.normal(batch, cols, seed=910 + seed)
        dw = dev(w)
        dy, y = quantize_q8_1(x)
        rc, ref_logits = oracle.gemv(w, y, vocab, cols, batch, threads=8)
        tokens = oracle.argmax_rows_scan(ref_logits, batch, vocab)["index"]
        drafts = tokens[:batch - 1].copy()
        drafts[-1] = (drafts[-1] + 1) % vocab          # all but the last draft match
        scratch = hip.DeviceBuffer(L.q8mi_lm_head_scratch_bytes(vocab, cols, batch))
        want_pairs, want_acc, want_logits = run("alloc", dw, dy, vocab, cols, batch, drafts, 2, scratch)
        got_pairs, got_acc, got_logits = run("static", dw, dy, vocab, cols, batch, drafts, 2, None)
        assert np.array_equal(got_pairs["index"], want_pairs["index"])
        assert np.array_equal(got_pairs["value"].view(np.uint32), want_pairs["value"].view(np.uint32))
        assert np.array_equal(got_acc, want_acc)
        assert np.array_equal(got_logits, want_logits)
        # and both agree with the oracle's tokens and accept length
        assert np.array_equal(got_pairs["index"], tokens)
        exp_len, exp_next = oracle.accept(tokens, drafts, eos=2)
        assert exp_len == batch - 2 and (int(got_acc[0]), int(got_acc[1])) == (exp_len, exp_next)


def test_static_scratch_entry_point_rejections(gpu):
    L = q8mi.lib()
    b = hip.DeviceBuffer(1 << 16)
    d = np.zeros(8, np.int32).ctypes.data_as(C.c_void_p)
    args = lambda rows, cols, batch: (b.ptr, b.ptr, rows, cols, batch, d, 0, 0, b.ptr, b.ptr, None, rows, NULL)
    assert L.q8mi_lm_head_argmax_accept_static(*args(100, 512, 9)) == q8mi.REJECTED     # more rows than the array holds
    assert "batch" in q8mi.last_error()
    assert L.q8mi_lm_head_argmax_accept_static(*args(100, 500, 2)) == q8mi.REJECTED
    assert L.q8mi_lm_head_argmax_accept_static(*args(0, 512, 2)) == q8mi.REJECTED


def mem_free():
    free, total = C.c_size_t(0), C.c_size_t(0)
    hip.check(hip.rt().hipMemGetInfo(C.byref(free), C.byref(total)), "hipMemGetInfo")
    return free.value


def test_static_scratch_entry_point_under_capture(gpu):
    """After one eager call of the same shape and batch (the first launch of a kernel instantiation
    asks the runtime for its LDS grant and occupancy), the call is captured into a HIP graph and
    replayed with eager work of another shape in between: every replay gives the eager call's
    bits, and the device's free memory does not change over the replays and the eager calls
    between them (nothing is allocated)."""
    L = q8mi.lib()
    vocab, cols, batch = 40000, 1024, 5
    dw = dev(synth.q8_0_weight(vocab, cols, seed=951))
    dy, _ = quantize_q8_1(synth.normal(batch, cols, seed=952))
    other_w = dev(synth.q8_0_weight(5000, cols, seed=953))
    other_y, _ = quantize_q8_1(synth.normal(2, cols, seed=954))
    drafts = np.array([1, 2, 3, 4], np.int32)
    dptr = drafts.ctypes.data_as(C.c_void_p)
    row_out, acc = hip.DeviceBuffer(8 * batch), hip.DeviceBuffer(8)
    o_rows, o_acc = hip.DeviceBuffer(16), hip.DeviceBuffer(8)
    stream = hip.Stream()

    def call(s):
        ok(L.q8mi_lm_head_argmax_accept_static(dw.ptr, dy.ptr, vocab, cols, batch, dptr, 0, 2, row_out.ptr, acc.ptr,
                                               None, vocab, s), "lm_head static")

    def other():
        ok(L.q8mi_lm_head_argmax_accept_static(other_w.ptr, other_y.ptr, 5000, cols, 2, dptr, 0, 2, o_rows.ptr, o_acc.ptr,
                                               None, 5000, stream.handle), "lm_head static, other shape")

    call(stream.handle)
    other()
    stream.synchronize()
    want_rows, want_acc = row_out.download(np.uint32).copy(), acc.download(np.int32).copy()
    g = hip.Graph(stream)
    with g:
        call(stream.handle)
    before = None
    for rep in range(5):
        if rep == 1:
            before = mem_free()      # after the runtime has set the graph up with its first launch
        row_out.fill(0xff)
        acc.fill(0xff)
        hip.synchronize()
        g.launch()
        stream.synchronize()
        assert np.array_equal(row_out.download(np.uint32), want_rows)
        assert np.array_equal(acc.download(np.int32), want_acc)
        other()                      # overwrites the shared partials between replays
        stream.synchronize()
    assert mem_free() == before
