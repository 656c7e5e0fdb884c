"""GPU parity at the shapes of benchmark config 3: the prefill chunk M = 2048 on the two FFN
projections, K=5120 -> N=17408 (2176 main tiles: four full rounds and a quarter round whose tiles
are cut in two along K) and K=17408 -> N=5120 (640 tiles: one round and a K-split quarter round),
i.e. exactly the launches bench.py times.  Reference shape: src/mmq_q8.cu:2394-2420 (128 x 128
tiles over rows x batch)."""
import numpy as np
import pytest

from gpu_common import NULL, assert_close_fp32, dev
from q8mi import hip, ok
import q8mi_support as synth
import q8mi

pytestmark = pytest.mark.gpu

M = 2048


@pytest.mark.parametrize("rows,cols", [(17408, 5120), (5120, 17408)])
def test_prefill_chunk_m2048(gpu, oracle, rows, cols):
    L = q8mi.lib()
    w = synth.q8_0_weight(rows, cols, seed=rows + 1, sigma=0.02)
    x = synth.normal(M, cols, seed=cols + 2)
    dw, dx = dev(w), dev(x)
    y_bytes = L.q8mi_q8_1_d4_scratch_bytes(M, cols)
    dy = hip.DeviceBuffer(y_bytes)
    ok(L.q8mi_quantize_q8_1_d4(dx.ptr, dy.ptr, M, cols, cols, NULL), "quantize_d4")
    hip.synchronize()
    y = dy.download(np.uint8, y_bytes)
    # quantized activations: bit-exact on a seeded sample of rows (first, last, tile edges, random)
    rng = np.random.default_rng(rows)
    pick = np.unique(np.concatenate([[0, 1, 127, 128, 1023, 1024, M - 1], rng.integers(0, M, 57)])).astype(np.int64)
    rc, yref = oracle.quantize_q8_1_d4(x[pick])
    assert np.array_equal(y.reshape(cols // 128, M, 144)[:, pick, :].reshape(-1), yref), "D4 blocks differ"

    out = hip.DeviceBuffer(4 * M * rows)
    runs = []
    for poison in (0xff, 0x7f):               # a poisoned output must be fully rewritten, twice alike
        out.fill(poison)
        ok(L.q8mi_gemm(dw.ptr, dy.ptr, out.ptr, rows, cols, M, rows, NULL), "gemm")
        hip.synchronize()
        runs.append(out.download(np.float32).reshape(M, rows))
    got = runs[0]
    assert np.array_equal(got.view(np.uint32), runs[1].view(np.uint32)), "two calls must agree bit for bit"
    assert np.isfinite(got).all(), "every output must be written"

    n = 60000
    sr = rng.integers(0, rows, n, dtype=np.uint32)
    sj = rng.integers(0, M, n, dtype=np.uint32)
    sr[:6] = [0, rows - 1, 0, rows - 1, rows - 129, 127]
    sj[:6] = [0, 0, M - 1, M - 1, M - 129, 128]
    rc, ref, absum = oracle.gemm_d4_sampled(w, y, rows, cols, M, sr, sj)
    assert_close_fp32(got[sj, sr], ref, absum, "prefill chunk M=2048 (sampled)")
    # every weight row for two activation rows: a misplaced or missing tile anywhere shows up
    for j in (0, M - 1):
        rr = np.arange(rows, dtype=np.uint32)
        rc, ref_c, absum_c = oracle.gemm_d4_sampled(w, y, rows, cols, M, rr, np.full(rows, j, np.uint32))
        assert_close_fp32(got[j], ref_c, absum_c, "prefill chunk M=2048 (activation row)")
    # and every activation row for two weight rows (first tile, last tile)
    for r in (0, rows - 1):
        jj = np.arange(M, dtype=np.uint32)
        rc, ref_r, absum_r = oracle.gemm_d4_sampled(w, y, rows, cols, M, np.full(M, r, np.uint32), jj)
        assert_close_fp32(got[:, r], ref_r, absum_r, "prefill chunk M=2048 (weight row)")
