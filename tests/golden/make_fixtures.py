#!/usr/bin/env python3
"""Writes tests/golden/q8_fixtures.npz: small input/expected-output vectors for every
stage of the Q8_0 x Q8_1 path.

The expected values come from tests/np_ref.py (an independent numpy restatement of the
block formats) and from plain Python loops for argmax and accept; neither the C oracle nor
the GPU library is used, so the fixtures pin both.  Inputs come from numpy's PCG64 and are
stored in the file, so regenerating is never needed to run the tests.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import np_ref  # noqa: E402

F32 = np.float32
OUT = os.path.join(HERE, "q8_fixtures.npz")


def activations(rng, batch, cols):
    x = rng.standard_normal((batch, cols)).astype(F32)
    x[0, 0:32] = 0.0                                   # all-zero block: d = 0, q = 0
    x[0, 32:64] = F32(0.37)                            # constant block: q = 127, s = fp16(32 c)
    x[0, 64:96] = np.arange(32, dtype=F32)             # ramp: q_i = rn(i * 127 / 31)
    x[0, 96:128] = -np.arange(32, dtype=F32) * F32(1e-3)
    x[1, 0:32] = F32(3000.0)                           # s = 96000 overflows fp16 -> +inf
    x[1, 32:64] = F32(-3000.0)                         # -inf
    x[1, 64:96] = F32(1e-7) * rng.standard_normal(32).astype(F32)   # fp16-subnormal scale
    x[1, 96:128] = np.where(np.arange(32) % 2 == 0, F32(0.5), F32(-0.5))   # rounding ties x/d = +-127
    x[2, 0:32] = np.linspace(-2.5, 2.5, 32, dtype=F32) # half-way cases after scaling
    return x


def argmax_single(row):
    """max by '>', ties -> lowest index, nothing above -inf -> (-inf, -1)
    (src/kernels_cuda.cu:1693-1734)."""
    best, idx = -np.inf, -1
    for i, v in enumerate(row):
        if v > best:
            best, idx = v, i
    return F32(best), idx


def accept(tokens, drafts, eos):
    """src/qwen_native_backend.cpp:15948-15960, 16048-16052."""
    n = 0
    for i, d in enumerate(drafts):
        t = tokens[i] if tokens[i] >= 0 else eos
        if t != d:
            break
        n += 1
    nxt = tokens[n] if tokens[n] >= 0 else eos
    return n, nxt


def main():
    rng = np.random.default_rng(20240607)
    rows, cols, batch = 24, 256, 3
    out = {}

    # weights
    w = (rng.standard_normal((rows, cols)) * 0.02).astype(F32)
    w[0, :32] = 0.0
    w[1, :32] = F32(0.01)
    w2 = (rng.standard_normal((rows, cols)) * 0.02).astype(F32)
    d16, q = np_ref.quantize_q8_0(w)
    d16b, qb = np_ref.quantize_q8_0(w2)
    out["w_f32"], out["w2_f32"] = w, w2
    out["w_gguf"] = np_ref.gguf_blocks(d16, q)
    out["w_split"] = np_ref.split_plane(d16, q)
    out["w2_split"] = np_ref.split_plane(d16b, qb)

    # activations in both layouts
    x = activations(rng, batch, cols)
    out["x_f32"] = x
    out["x_q8_1"] = np_ref.quantize_q8_1(x)
    out["x_d4"] = np_ref.quantize_d4(x)

    # int32 block dots and linear outputs
    dw, qw = np_ref.unpack_weight(out["w_split"], cols)
    dw2, qw2 = np_ref.unpack_weight(out["w2_split"], cols)
    dx, _, qx = np_ref.unpack_q8_1(out["x_q8_1"], batch, cols)
    dx4, qx4 = np_ref.unpack_d4(out["x_d4"], batch, cols)
    S = np_ref.block_dots(qw, qx)
    out["dots_q8_1"] = S.astype(np.int32)
    out["dots_d4"] = np_ref.block_dots(qw, qx4).astype(np.int32)
    out["gemv_f64"] = np_ref.linear_f64(dw, qw, dx, qx)
    out["gemv_abs_f64"] = np.einsum("jrk,rk,jk->jr", np.abs(S).astype(np.float64), dw.astype(np.float64),
                                    dx.astype(np.float64))
    out["gemv_f32_ascending"] = np_ref.linear_f32_ascending(dw, qw, dx, qx)
    out["gemm_d4_f64"] = np_ref.linear_f64(dw, qw, dx4, qx4)
    out["gemm_d4_f32_ascending"] = np_ref.linear_f32_ascending(dw, qw, dx4, qx4)
    g = out["gemv_f64"]
    u = np_ref.linear_f64(dw2, qw2, dx, qx)
    out["up_f64"] = u
    out["silu_mul_f64"] = g / (1.0 + np.exp(-g)) * u
    resid = rng.standard_normal((batch, rows)).astype(F32)
    out["residual_f32"] = resid
    out["add_f64"] = resid.astype(np.float64) + g

    # argmax rows: plain, ties, -inf rows, a single element
    n = 3000
    logits = rng.standard_normal((6, n)).astype(F32)
    logits[1, 17] = logits[1, 2900] = F32(9.0)          # tie: lowest index
    logits[2, :] = -np.inf                              # nothing above -inf
    logits[3, :] = -np.inf
    logits[3, 2999] = F32(-1e30)                        # the only finite value, last position
    logits[4, 0] = F32(50.0)                            # first position
    logits[5, 1023] = logits[5, 1024] = logits[5, 2047] = F32(7.5)   # ties across scanner boundaries
    out["logits"] = logits
    pairs = [argmax_single(r) for r in logits]
    out["argmax_value"] = np.array([p[0] for p in pairs], F32)
    out["argmax_index"] = np.array([p[1] for p in pairs], np.int32)

    # accept: every (rows, matching prefix) pair with forced matches, plus rows without a token
    cases = []
    for m in range(1, 9):
        tokens = rng.integers(0, 248320, m).astype(np.int32)
        for prefix in range(m):
            drafts = rng.integers(0, 248320, m - 1).astype(np.int32)
            drafts[:prefix] = tokens[:prefix]
            if prefix < m - 1 and drafts[prefix] == tokens[prefix]:
                drafts[prefix] += 1
            cases.append((tokens, drafts, 151645))
    cases.append((np.array([5, -1, 9], np.int32), np.array([5, 151645], np.int32), 151645))   # -1 reads as eos
    cases.append((np.array([-1], np.int32), np.array([], np.int32), 7))
    cases.append((np.array([4, 4, -1], np.int32), np.array([4, 4], np.int32), 7))              # next = eos
    tok = np.full((len(cases), 8), -2, np.int32)
    dr = np.full((len(cases), 7), -2, np.int32)
    meta = np.zeros((len(cases), 4), np.int32)          # rows, eos, accepted, next
    for i, (t, d, eos) in enumerate(cases):
        tok[i, :len(t)] = t
        dr[i, :len(d)] = d
        a, nx = accept(list(t), list(d), eos)
        meta[i] = (len(t), eos, a, nx)
    out["accept_tokens"], out["accept_drafts"], out["accept_meta"] = tok, dr, meta

    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT}: {os.path.getsize(OUT)} bytes, {len(out)} arrays")


if __name__ == "__main__":
    main()
