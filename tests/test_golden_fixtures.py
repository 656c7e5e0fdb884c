"""Golden fixtures (tests/golden/q8_fixtures.npz, written by tests/golden/make_fixtures.py
from an independent numpy restatement): the CPU oracle and the GPU library must both
reproduce them.  Integer and byte results bit for bit; fp32 results within
1e-5 relative (+1e-6 of the summed block magnitudes) of the float64 truth."""
import ctypes as C
import os

import numpy as np
import pytest

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "q8_fixtures.npz")
ROWS, COLS, BATCH = 24, 256, 3
PAIR = np.dtype([("value", np.float32), ("index", np.int32)])


@pytest.fixture(scope="module")
def fx():
    with np.load(FIX, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def close(got, truth, mag, what, rel=1e-5, floor=1e-6):
    got, truth, mag = (np.asarray(a, np.float64) for a in (got, truth, mag))
    lim = rel * np.abs(truth) + floor * mag + 1e-30
    bad = ~(np.abs(got - truth) <= lim)
    assert not bad.any(), f"{what}: {bad.sum()} outside tolerance, first {np.argwhere(bad)[0]}"


# ---------------------------------------------------------------- CPU: oracle vs fixtures
def test_oracle_weight_formats(oracle, fx):
    gguf = oracle.quantize_q8_0(fx["w_f32"])
    assert np.array_equal(gguf.reshape(ROWS, -1), fx["w_gguf"])
    split = oracle.repack_split_plane(fx["w_gguf"], ROWS, COLS)
    assert np.array_equal(split.reshape(ROWS, -1), fx["w_split"])


def test_oracle_activation_quantizers(oracle, fx):
    rc, y = oracle.quantize_q8_1(fx["x_f32"])
    assert rc == 0 and np.array_equal(y, fx["x_q8_1"])
    rc, y4 = oracle.quantize_q8_1_d4(fx["x_f32"])
    assert rc == 0 and np.array_equal(y4, fx["x_d4"])


def test_oracle_block_dots(oracle, fx):
    for layout, ykey, skey in ((0, "x_q8_1", "dots_q8_1"), (1, "x_d4", "dots_d4")):
        for j in range(BATCH):
            for r in range(ROWS):
                for kb in range(COLS // 32):
                    assert oracle.block_dot(fx["w_split"], fx[ykey], layout, COLS, BATCH, r, j, kb) == \
                        fx[skey][j, r, kb]


def test_oracle_linear_outputs(oracle, fx):
    w, w2, y = fx["w_split"], fx["w2_split"], fx["x_q8_1"]
    rc, out = oracle.gemv(w, y, ROWS, COLS, BATCH)
    assert rc == 0
    # same order, same fused multiply-add: bit for bit
    assert np.array_equal(out.view(np.uint32), fx["gemv_f32_ascending"].view(np.uint32))
    close(out, fx["gemv_f64"], fx["gemv_abs_f64"], "gemv vs float64")
    rc, out4 = oracle.gemm_d4(w, fx["x_d4"], ROWS, COLS, BATCH)
    assert rc == 0
    assert np.array_equal(out4.view(np.uint32), fx["gemm_d4_f32_ascending"].view(np.uint32))
    close(out4, fx["gemm_d4_f64"], fx["gemv_abs_f64"], "gemm vs float64")
    rc, silu = oracle.gemv_silu_mul(w, w2, y, ROWS, COLS, BATCH)
    g, u = fx["gemv_f64"], fx["up_f64"]
    mag = fx["gemv_abs_f64"] * np.abs(u) * 1.1 + np.abs(g) * np.abs(u) + np.abs(fx["silu_mul_f64"])
    close(silu, fx["silu_mul_f64"], mag, "silu_mul vs float64", rel=2e-5, floor=2e-6)
    rc, acc = oracle.gemv_add(w, y, fx["residual_f32"].copy(), ROWS, COLS, BATCH)
    close(acc, fx["add_f64"], fx["gemv_abs_f64"] + np.abs(fx["residual_f32"]), "gemv_add vs float64")


def test_oracle_argmax_and_accept(oracle, fx):
    logits = fx["logits"]
    for i, row in enumerate(logits):
        value, index = oracle.argmax_row(row)
        assert index == fx["argmax_index"][i]
        assert np.float32(value).view(np.uint32) == fx["argmax_value"][i].view(np.uint32)
    scan = oracle.argmax_rows_scan(logits, logits.shape[0], logits.shape[1])
    assert np.array_equal(scan["index"], fx["argmax_index"])
    for tok, dr, (m, eos, acc, nxt) in zip(fx["accept_tokens"], fx["accept_drafts"], fx["accept_meta"]):
        got = oracle.accept(tok[:m], dr[:m - 1], eos=int(eos))
        assert tuple(int(v) for v in got) == (int(acc), int(nxt))


# ---------------------------------------------------------------- GPU: library vs fixtures
@pytest.mark.gpu
def test_gpu_formats_and_dots(gpu, fx):
    from gpu_common import NULL, dev, quantize_d4, quantize_q8_1
    import q8mi_support as synth
    from q8mi import hip, ok
    L = gpu.lib()
    split = np.empty_like(fx["w_split"])
    ok(L.q8mi_repack_q8_0_split_host(fx["w_gguf"].ctypes.data_as(C.c_void_p), ROWS, COLS,
                                     split.ctypes.data_as(C.c_void_p)), "repack host")
    assert np.array_equal(split, fx["w_split"])
    dsplit = hip.DeviceBuffer(split.nbytes)
    ok(L.q8mi_repack_q8_0_split(dev(fx["w_gguf"]).ptr, ROWS, COLS, dsplit.ptr, NULL), "repack device")
    hip.synchronize()
    assert np.array_equal(dsplit.download(np.uint8).reshape(ROWS, -1), fx["w_split"])
    dy, y = quantize_q8_1(fx["x_f32"])
    assert np.array_equal(y, fx["x_q8_1"])
    dy4, y4 = quantize_d4(fx["x_f32"])
    assert np.array_equal(y4, fx["x_d4"])
    jj, rr, kk = np.meshgrid(np.arange(BATCH), np.arange(ROWS), np.arange(COLS // 32), indexing="ij")
    n = jj.size
    sr, sj, sk = (dev(a.reshape(-1).astype(np.uint32)) for a in (rr, jj, kk))
    for layout, ybuf, skey in ((0, dy, "dots_q8_1"), (1, dy4, "dots_d4")):
        out = hip.DeviceBuffer(4 * n)
        ok(synth.lib().q8sup_block_dots(dsplit.ptr, ybuf.ptr, layout, ROWS, COLS, BATCH, sr.ptr, sj.ptr, sk.ptr, n, out.ptr,
                             NULL), "block_dots")
        hip.synchronize()
        assert np.array_equal(out.download(np.int32, n).reshape(BATCH, ROWS, -1), fx[skey])


@pytest.mark.gpu
def test_gpu_linear_outputs(gpu, fx):
    from gpu_common import NULL, dev
    from q8mi import hip, ok
    L = gpu.lib()
    w, w2, y = dev(fx["w_split"]), dev(fx["w2_split"]), dev(fx["x_q8_1"])
    out = hip.DeviceBuffer(4 * BATCH * ROWS)
    mag = fx["gemv_abs_f64"]

    def result():
        hip.synchronize()
        return out.download(np.float32).reshape(BATCH, ROWS)

    ok(L.q8mi_gemv(w.ptr, y.ptr, out.ptr, ROWS, COLS, BATCH, ROWS, NULL), "gemv")
    close(result(), fx["gemv_f64"], mag, "gemv")
    close(result(), fx["gemv_f32_ascending"], mag, "gemv vs ascending fp32")
    ok(L.q8mi_gemm(w.ptr, y.ptr, out.ptr, ROWS, COLS, BATCH, ROWS, NULL), "gemm")   # rows < 128: Q8_1 layout
    close(result(), fx["gemv_f64"], mag, "gemm (Q8_1 layout)")
    ok(L.q8mi_gemv_silu_mul(w.ptr, w2.ptr, y.ptr, out.ptr, ROWS, COLS, BATCH, ROWS, NULL), "silu_mul")
    g, u = fx["gemv_f64"], fx["up_f64"]
    smag = mag * np.abs(u) * 1.1 + np.abs(g) * np.abs(u) + np.abs(fx["silu_mul_f64"])
    close(result(), fx["silu_mul_f64"], smag, "silu_mul", rel=2e-5, floor=2e-6)
    acc = dev(fx["residual_f32"])
    ok(L.q8mi_gemv_add(w.ptr, y.ptr, acc.ptr, ROWS, COLS, BATCH, ROWS, NULL), "gemv_add")
    hip.synchronize()
    close(acc.download(np.float32).reshape(BATCH, ROWS), fx["add_f64"], mag + np.abs(fx["residual_f32"]), "gemv_add")


@pytest.mark.gpu
def test_gpu_gemm_d4_fixture(gpu, fx):
    """The D4 GEMM needs rows >= 128: the fixture's 24 weight rows are tiled 6 times."""
    from gpu_common import NULL, dev
    from q8mi import hip, ok
    L = gpu.lib()
    reps = 6
    w = dev(np.tile(fx["w_split"], (reps, 1)))
    y4 = dev(fx["x_d4"])
    rows = ROWS * reps
    out = hip.DeviceBuffer(4 * BATCH * rows)
    ok(L.q8mi_gemm(w.ptr, y4.ptr, out.ptr, rows, COLS, BATCH, rows, NULL), "gemm d4")
    hip.synchronize()
    got = out.download(np.float32).reshape(BATCH, reps, ROWS)
    for r in range(reps):
        close(got[:, r], fx["gemm_d4_f64"], fx["gemv_abs_f64"], "gemm d4")
        close(got[:, r], fx["gemm_d4_f32_ascending"], fx["gemv_abs_f64"], "gemm d4 vs ascending fp32")


@pytest.mark.gpu
def test_gpu_argmax_and_accept(gpu, fx):
    from gpu_common import NULL, dev, quantize_q8_1
    from q8mi import hip, ok
    L = gpu.lib()
    logits = fx["logits"]
    n = logits.shape[1]
    for i, row in enumerate(logits):
        res = hip.DeviceBuffer(8)
        ok(L.q8mi_argmax(dev(row).ptr, n, res.ptr, NULL), "argmax")
        hip.synchronize()
        out = res.download(np.int32, 2)
        assert out[0] == fx["argmax_index"][i]
        assert out[1:2].view(np.uint32)[0] == fx["argmax_value"][i:i + 1].view(np.uint32)[0]
    # accept through the fused LM head: activation row j lights up column j only, and the weight
    # row of token[j] is the only one that reads column j, so row j's argmax is token[j]
    vocab, cols = 4096, 256
    for tok, dr, (m, eos, acc, nxt) in zip(fx["accept_tokens"], fx["accept_drafts"], fx["accept_meta"]):
        m = int(m)
        tokens = tok[:m] % vocab
        if (tok[:m] < 0).any():
            continue     # rows without a token cannot come out of a finite LM head; covered on the CPU side
        drafts = np.where(dr[:m - 1] == tok[:m - 1], tokens[:m - 1], (tokens[:m - 1] + 1) % vocab).astype(np.int32)
        w = np.zeros((vocab, cols // 32 * 34), np.uint8)
        d = np.zeros((vocab, cols // 32), np.float16)
        q = np.zeros((vocab, cols), np.int8)
        x = np.zeros((m, cols), np.float32)
        for j in range(m):
            x[j, j] = 1.0
            d[tokens[j], 0] = 1.0
            q[tokens[j], j] = 100
        w[:, :2 * (cols // 32)] = d.view(np.uint8)
        w[:, 2 * (cols // 32):] = q.view(np.uint8)
        dy, _ = quantize_q8_1(x)
        scratch = hip.DeviceBuffer(L.q8mi_lm_head_scratch_bytes(vocab, cols, m))
        rows_out, acc_out = hip.DeviceBuffer(8 * m), hip.DeviceBuffer(8)
        dd = np.ascontiguousarray(drafts, np.int32)
        ok(L.q8mi_lm_head_argmax_accept(dev(w).ptr, dy.ptr, vocab, cols, m,
                                        dd.ctypes.data_as(C.c_void_p) if dd.size else None, 0, int(eos),
                                        rows_out.ptr, acc_out.ptr, None, vocab, scratch.ptr, NULL), "lm_head")
        hip.synchronize()
        got_rows = rows_out.download(PAIR)
        a = acc_out.download(np.int32)
        assert got_rows["index"].tolist() == tokens.tolist()
        assert (int(a[0]), int(a[1])) == (int(acc), int(tokens[int(acc)]))
