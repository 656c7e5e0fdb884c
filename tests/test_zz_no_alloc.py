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
