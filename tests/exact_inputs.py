"""Inputs whose Q8_0 x Q8_1 / D4 results are exact in fp32 in ANY summation order.

Every weight scale and every activation scale is a power of two and the quants are small, so each
per-block term d_w * d_x * S is an integer multiple of 2^-10 below 2^15 of those units, and the sum
of the up to 544 blocks of a row stays below 2^24 units: every partial sum a kernel can form, in
whatever order and grouping, is exactly representable.  A kernel that computes the right int32
block dots and applies the right scales therefore returns the oracle's bits, and one that drops,
repeats or misplaces a block does not.
"""
import numpy as np

W_EXPS = (-9, -8)      # weight scales 2^-9, 2^-8 (exact fp16 values)
X_EXPS = (-1, 0)       # activation scales 2^-1, 2^0
W_QMAX = 15            # weight quants in [-15, 15]
X_QMAX = 7             # activation quants in [-7, 7], plus one +-127 per block (it fixes the scale)
MAX_BLOCKS = 544       # 17408 columns: 544 * (15*127 + 31*15*7) * 4 < 2^24


def weight(rows, cols, seed):
    """Split-plane Q8_0 rows (uint8 [rows, cols/32*34]) with power-of-two scales."""
    nb = cols // 32
    assert cols % 32 == 0 and nb <= MAX_BLOCKS
    rng = np.random.default_rng(seed)
    d = np.ldexp(np.float32(1.0), rng.integers(W_EXPS[0], W_EXPS[1] + 1, (rows, nb))).astype(np.float16)
    q = rng.integers(-W_QMAX, W_QMAX + 1, (rows, nb * 32)).astype(np.int8)
    w = np.empty((rows, nb * 34), np.uint8)
    w[:, :2 * nb] = d.view(np.uint8).reshape(rows, 2 * nb)
    w[:, 2 * nb:] = q.view(np.uint8)
    return w


def activations(batch, cols, seed):
    """fp32 [batch, cols]: x = q * 2^k per 32-block with max|q| = 127, so both quantizers
    (amax/127 and 127/amax forms) return scale 2^k and the integers q exactly."""
    nb = cols // 32
    rng = np.random.default_rng(seed)
    q = rng.integers(-X_QMAX, X_QMAX + 1, (batch, nb, 32)).astype(np.float32)
    pos = rng.integers(0, 32, (batch, nb))
    sign = rng.choice(np.array([-127.0, 127.0], np.float32), (batch, nb))
    np.put_along_axis(q, pos[..., None], sign[..., None], axis=2)
    k = rng.integers(X_EXPS[0], X_EXPS[1] + 1, (batch, nb, 1))
    return np.ldexp(q, k).astype(np.float32).reshape(batch, cols)


def residual(batch, rows, seed):
    """A residual stream on the same 2^-10 grid, small enough to keep the sums exact."""
    rng = np.random.default_rng(seed)
    return (rng.integers(-4096, 4097, (batch, rows)).astype(np.float32) / np.float32(1024.0)).astype(np.float32)
