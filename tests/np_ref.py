"""Independent numpy restatement of the Q8 block formats, used to pin the C
oracle (two implementations written separately must agree bit for bit) and to
write the golden fixtures.  Vectorised, float32 arithmetic via numpy scalars'
IEEE semantics; no code shared with oracle/q8_oracle.c."""
import numpy as np

F32 = np.float32


def quantize_q8_0(w):
    """fp32 [rows, cols] -> (fp16 scales [rows, nb], int8 quants [rows, nb, 32]).
    Rule of the reference's host quantizer (tests/mmq_parity.cu:54-80)."""
    rows, cols = w.shape
    b = w.reshape(rows, cols // 32, 32).astype(F32)
    amax = np.abs(b).max(axis=2)
    d = amax / F32(127.0)
    with np.errstate(divide="ignore"):
        d_inv = np.where(d == 0, F32(0), F32(1.0) / d).astype(F32)
    q = np.rint(b * d_inv[:, :, None]).clip(-127, 127).astype(np.int8)
    return d.astype(np.float16), q


def split_plane(d16, q):
    """(scales, quants) -> split-plane row bytes [rows, nb*34]."""
    rows, nb = d16.shape
    out = np.empty((rows, nb * 34), np.uint8)
    out[:, :2 * nb] = d16.view(np.uint8).reshape(rows, 2 * nb)
    out[:, 2 * nb:] = q.reshape(rows, nb * 32).view(np.uint8)
    return out


def gguf_blocks(d16, q):
    """(scales, quants) -> interleaved GGUF Q8_0 bytes [rows, nb*34]."""
    rows, nb = d16.shape
    out = np.empty((rows, nb, 34), np.uint8)
    out[:, :, :2] = d16.view(np.uint8).reshape(rows, nb, 2)
    out[:, :, 2:] = q.view(np.uint8)
    return out.reshape(rows, nb * 34)


def butterfly_sum(b):
    """b: [..., 32] float32 -> the reference's xor-butterfly sum (offsets 16,8,4,2,1)."""
    a = (b[..., :16] + b[..., 16:]).astype(F32)
    a = (a[..., :8] + a[..., 8:]).astype(F32)
    a = (a[..., :4] + a[..., 4:]).astype(F32)
    a = (a[..., :2] + a[..., 2:]).astype(F32)
    return (a[..., 0] + a[..., 1]).astype(F32)


def quantize_q8_1(x):
    """fp32 [batch, cols] (finite values) -> Q8_1 bytes, src/mmvq_q8.cu:82-112."""
    batch, cols = x.shape
    nb = cols // 32
    b = x.reshape(batch, nb, 32).astype(F32)
    amax = np.abs(b).max(axis=2)
    s = butterfly_sum(b)
    d = (amax / F32(127.0)).astype(F32)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        q = np.where(amax[:, :, None] == 0, F32(0), np.rint(b / d[:, :, None]))
    out = np.empty((batch, nb, 36), np.uint8)
    with np.errstate(over="ignore"):
        out[:, :, 0:2] = d.astype(np.float16).view(np.uint8).reshape(batch, nb, 2)
        out[:, :, 2:4] = s.astype(np.float16).view(np.uint8).reshape(batch, nb, 2)
    out[:, :, 4:] = q.astype(np.int8).view(np.uint8)
    return out.reshape(-1)


def quantize_d4(x):
    """fp32 [batch, cols] -> D4 bytes ordered (k/128)*batch + j, src/mmvq_q8.cu:668-722."""
    batch, cols = x.shape
    nsb = cols // 128
    b = x.reshape(batch, nsb, 4, 32).astype(F32)
    amax = np.abs(b).max(axis=3)
    with np.errstate(divide="ignore"):
        d_inv = np.where(amax == 0, F32(0), F32(127.0) / amax).astype(F32)
        d = np.where(amax == 0, F32(0), F32(1.0) / d_inv).astype(F32)
    q = np.rint(b * d_inv[..., None]).astype(np.int8)
    out = np.empty((nsb, batch, 144), np.uint8)
    out[:, :, :16] = d.transpose(1, 0, 2).copy().view(np.uint8).reshape(nsb, batch, 16)
    out[:, :, 16:] = q.transpose(1, 0, 2, 3).reshape(nsb, batch, 128).view(np.uint8)
    return out.reshape(-1)


def unpack_weight(w_split, cols):
    rows = w_split.shape[0]
    nb = cols // 32
    d = w_split[:, :2 * nb].copy().view(np.float16).astype(F32)               # [rows, nb]
    q = w_split[:, 2 * nb:].copy().view(np.int8).reshape(rows, nb, 32)
    return d, q


def unpack_q8_1(y, batch, cols):
    nb = cols // 32
    b = np.asarray(y, np.uint8).reshape(batch, nb, 36)
    d = b[:, :, 0:2].copy().view(np.float16).reshape(batch, nb).astype(F32)
    s = b[:, :, 2:4].copy().view(np.float16).reshape(batch, nb)
    q = b[:, :, 4:].copy().view(np.int8)
    return d, s, q


def unpack_d4(y, batch, cols):
    nsb = cols // 128
    b = np.asarray(y, np.uint8).reshape(nsb, batch, 144)
    d = b[:, :, :16].copy().view(F32).reshape(nsb, batch, 4).transpose(1, 0, 2).reshape(batch, nsb * 4)
    q = b[:, :, 16:].copy().view(np.int8).reshape(nsb, batch, 4, 32).transpose(1, 0, 2, 3)
    return d, q.reshape(batch, nsb * 4, 32)


def block_dots(qw, qx):
    """int8 [rows, nb, 32] x int8 [batch, nb, 32] -> int64 S[batch, rows, nb]."""
    return np.einsum("rkt,jkt->jrk", qw.astype(np.int64), qx.astype(np.int64))


def linear_f64(dw, qw, dx, qx):
    """Exact-ish truth: sum_kb d_w*d_x*S in float64 -> [batch, rows]."""
    S = block_dots(qw, qx).astype(np.float64)
    return np.einsum("jrk,rk,jk->jr", S, dw.astype(np.float64), dx.astype(np.float64))


def linear_f32_ascending(dw, qw, dx, qx):
    """The oracle's order restated: acc = fma(d_w*d_x, S, acc) for kb ascending.
    fma is emulated in float64 (the product of two fp32 by a 20-bit integer is
    exact in 53 bits only up to rounding of the final add; see the test that uses
    this for the allowance)."""
    S = block_dots(qw, qx)
    batch, rows, nb = S.shape
    acc = np.zeros((batch, rows), F32)
    for kb in range(nb):
        d = (dx[:, kb][:, None] * dw[:, kb][None, :]).astype(F32)            # fp32 product, rounded
        t = d.astype(np.float64) * S[:, :, kb].astype(np.float64) + acc.astype(np.float64)
        acc = t.astype(F32)
    return acc
