"""GPU parity: dequantizing row gather (embedding lookup), bit-exact.

Every output is fp16 * int8, exact in fp32, so the oracle and the kernels must agree on bits
(reference kernels: src/kernels_cuda.cu:2075-2190)."""
import numpy as np
import pytest

import q8mi
from gpu_common import NULL, dev
from q8mi import REJECTED, hip, ok

pytestmark = pytest.mark.gpu

PAIR = np.dtype([("value", np.float32), ("index", np.int32)])


def make(oracle, rows, cols, seed):
    rng = np.random.default_rng(seed)
    w = rng.standard_normal((rows, cols)).astype(np.float32) * 0.05
    w[0, :32] = 0.0                                   # a block with scale zero
    w[rows - 1, -32:] = 3000.0 * np.sign(w[rows - 1, -32:])   # large scale
    return oracle.make_weight(w)


def bf16(oracle, v):
    return np.array([oracle.f32_to_bf16(float(x)) for x in v], np.uint16)


@pytest.mark.parametrize("rows,cols", [(64, 32), (33, 96), (500, 1024), (2000, 5120), (40, 17408)])
def test_get_row_and_rows(gpu, oracle, rows, cols):
    w = make(oracle, rows, cols, seed=rows + cols)
    dw = dev(w)
    L = q8mi.lib()
    out = hip.DeviceBuffer(cols * 4)
    outb = hip.DeviceBuffer(cols * 2)
    for r in (0, rows // 2, rows - 1):
        want = oracle.get_row(w, r, cols)
        ok(L.q8mi_get_row(dw.ptr, r, rows, cols, out.ptr, 0, NULL), "get_row")
        ok(L.q8mi_get_row(dw.ptr, r, rows, cols, outb.ptr, 1, NULL), "get_row bf16")
        hip.synchronize()
        assert np.array_equal(out.download(np.uint32), want.view(np.uint32)), f"row {r}"
        assert np.array_equal(outb.download(np.uint16), bf16(oracle, want)), f"row {r} bf16"
    assert L.q8mi_get_row(dw.ptr, rows, rows, cols, out.ptr, 0, NULL) == REJECTED

    rng = np.random.default_rng(3)
    ids = rng.integers(0, rows, 37).astype(np.uint64)
    ids[5] = ids[6] = rows - 1                        # repeats
    ids[9] = rows + 7                                 # outside the matrix: a row of zeros
    dids = dev(ids)
    many = hip.DeviceBuffer(len(ids) * cols * 4)
    manyb = hip.DeviceBuffer(len(ids) * cols * 2)
    ok(L.q8mi_get_rows(dw.ptr, dids.ptr, len(ids), rows, cols, many.ptr, 0, NULL), "get_rows")
    ok(L.q8mi_get_rows(dw.ptr, dids.ptr, len(ids), rows, cols, manyb.ptr, 1, NULL), "get_rows bf16")
    hip.synchronize()
    got = many.download(np.uint32).reshape(len(ids), cols)
    gotb = manyb.download(np.uint16).reshape(len(ids), cols)
    for j, r in enumerate(ids):
        want = oracle.get_row(w, int(r), cols) if r < rows else np.zeros(cols, np.float32)
        assert np.array_equal(got[j], want.view(np.uint32)), f"slot {j} row {r}"
        assert np.array_equal(gotb[j], bf16(oracle, want)), f"slot {j} row {r} bf16"


def test_get_row_from_argmax_slot(gpu, oracle):
    rows, cols = 3000, 5120
    w = make(oracle, rows, cols, seed=11)
    dw = dev(w)
    L = q8mi.lib()
    pairs = np.zeros(5, PAIR)
    pairs["index"] = [17, -1, rows, rows - 1, 2 ** 31 - 1]
    dp = dev(pairs.view(np.uint8))
    out = hip.DeviceBuffer(cols * 4)
    for slot, tok in enumerate(pairs["index"]):
        ok(L.q8mi_get_row_from_argmax(dw.ptr, dp.ptr, slot, rows, cols, out.ptr, NULL), "from_argmax")
        hip.synchronize()
        want = oracle.get_row(w, int(tok), cols) if 0 <= tok < rows else np.zeros(cols, np.float32)
        assert np.array_equal(out.download(np.uint32), want.view(np.uint32)), f"slot {slot}"


def test_argmax_then_embedding_chain(gpu, oracle):
    """The decode tail: argmax of a logits row lands in a pair slot, the next token's embedding
    row is gathered from that slot without a host round trip."""
    rows, cols = 4096, 1024
    w = make(oracle, rows, cols, seed=12)
    dw = dev(w)
    L = q8mi.lib()
    rng = np.random.default_rng(13)
    logits = rng.standard_normal(rows).astype(np.float32)
    dl = dev(logits)
    dp = hip.DeviceBuffer(8 * 2)
    out = hip.DeviceBuffer(cols * 4)
    ok(L.q8mi_argmax_to_pair(dl.ptr, rows, dp.ptr, 1, NULL), "argmax_to_pair")
    ok(L.q8mi_get_row_from_argmax(dw.ptr, dp.ptr, 1, rows, cols, out.ptr, NULL), "from_argmax")
    hip.synchronize()
    _, tok = oracle.argmax_row(logits)
    assert np.array_equal(out.download(np.uint32), oracle.get_row(w, tok, cols).view(np.uint32))


def test_get_rows_long_prompt(gpu, oracle):
    """A prompt's worth of rows in one call: 100 000 ids (more than a grid's y extent)."""
    rows, cols = 512, 256
    w = make(oracle, rows, cols, seed=14)
    dw = dev(w)
    n = 100000
    ids = np.random.default_rng(15).integers(0, rows, n).astype(np.uint64)
    dids = dev(ids)
    out = hip.DeviceBuffer(n * cols * 4)
    ok(q8mi.lib().q8mi_get_rows(dw.ptr, dids.ptr, n, rows, cols, out.ptr, 0, NULL), "get_rows")
    hip.synchronize()
    got = out.download(np.uint32).reshape(n, cols)
    table = np.stack([oracle.get_row(w, r, cols) for r in range(rows)]).view(np.uint32)
    assert np.array_equal(got, table[ids.astype(np.int64)])


def test_get_rows_rejections(gpu):
    L = q8mi.lib()
    buf = hip.DeviceBuffer(4096)
    assert L.q8mi_get_row(buf.ptr, 0, 4, 48, buf.ptr, 0, NULL) == REJECTED          # cols % 32
    assert L.q8mi_get_row(buf.ptr, 0, 4, 0, buf.ptr, 0, NULL) == REJECTED
    assert L.q8mi_get_row(buf.ptr, 0, 4, 64, buf.ptr + 4, 0, NULL) == REJECTED      # output alignment
    assert L.q8mi_get_rows(buf.ptr, 0, 3, 4, 64, buf.ptr, 0, NULL) == REJECTED      # null id array
    assert L.q8mi_get_rows(buf.ptr, 0, 0, 4, 64, buf.ptr, 0, NULL) == q8mi.OK       # empty batch
