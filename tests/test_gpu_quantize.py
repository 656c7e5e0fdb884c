"""GPU parity: activation quantizers vs the CPU oracle, bit-exact."""
import numpy as np
import pytest

from gpu_common import quantize_d4, quantize_q8_1
import q8mi_support as synth

pytestmark = pytest.mark.gpu


def special_rows(cols):
    """Rows that exercise the corners of the quantizers."""
    rng = np.random.default_rng(5)
    rows = []
    rows.append(np.zeros(cols, np.float32))                       # all-zero blocks -> d = 0, q = 0
    rows.append(np.full(cols, 0.75, np.float32))                  # constant block -> q = 127
    rows.append(np.full(cols, -3.0, np.float32))
    rows.append(np.tile(np.arange(32, dtype=np.float32), cols // 32))   # ramp
    r = rng.standard_normal(cols).astype(np.float32) * 1e-42      # fp32 denormals
    rows.append(r)
    r = rng.standard_normal(cols).astype(np.float32) * 3e4        # block sums beyond fp16 range -> s = inf
    rows.append(r)
    r = rng.standard_normal(cols).astype(np.float32)
    r[::7] *= 1e6                                                  # d beyond fp16 normal range for Q8_1
    rows.append(r)
    r = rng.standard_normal(cols).astype(np.float32)              # ties at .5 after scaling
    r[:32] = np.arange(32, dtype=np.float32) * 0.5
    r[31] = 63.5
    rows.append(r)
    r = rng.standard_normal(cols).astype(np.float32)
    r[5] = np.inf
    r[40] = -np.inf
    r[70] = np.nan
    rows.append(r)
    return np.stack(rows)


@pytest.mark.parametrize("batch,cols", [(1, 32), (1, 5120), (3, 6144), (8, 17408), (5, 96), (2, 1056)])
def test_quantize_q8_1_bit_exact(gpu, oracle, batch, cols):
    x = synth.normal(batch, cols, seed=100 + batch + cols)
    _, got = quantize_q8_1(x)
    rc, ref = oracle.quantize_q8_1(x)
    assert rc == 0
    assert np.array_equal(got, ref), f"{(got != ref).sum()} differing bytes"


def test_quantize_q8_1_special_values(gpu, oracle):
    x = special_rows(256)
    _, got = quantize_q8_1(x)
    rc, ref = oracle.quantize_q8_1(x)
    g = got.reshape(-1, 36)
    r = ref.reshape(-1, 36)
    # quants and d must match bit for bit; s too unless it is a NaN (payload is unspecified)
    assert np.array_equal(g[:, 4:], r[:, 4:])
    assert np.array_equal(g[:, :2], r[:, :2])
    gs = g[:, 2:4].copy().view(np.float16).reshape(-1)
    rs = r[:, 2:4].copy().view(np.float16).reshape(-1)
    nan = np.isnan(rs)
    assert np.array_equal(np.isnan(gs), nan)
    assert np.array_equal(g[:, 2:4][~nan], r[:, 2:4][~nan])


def test_quantize_q8_1_strided_and_unaligned(gpu, oracle):
    # stride larger than cols, and a stride that breaks 16-byte alignment of rows
    for stride, cols in [(5120 + 64, 5120), (1000 + 3, 992)]:
        x = synth.normal(4, stride, seed=stride)
        _, got = quantize_q8_1(x, cols=cols, stride=stride)
        rc, ref = oracle.quantize_q8_1(x, cols=cols, stride=stride)
        assert rc == 0 and np.array_equal(got, ref)


def test_quantize_q8_1_rejects_ragged_cols(gpu):
    import q8mi
    from q8mi import hip
    buf = hip.DeviceBuffer(4096)
    assert q8mi.lib().q8mi_quantize_q8_1(buf.ptr, buf.ptr, 1, 33, 33, None) == q8mi.REJECTED
    assert q8mi.lib().q8mi_quantize_q8_1_d4(buf.ptr, buf.ptr, 1, 160, 160, None) == q8mi.REJECTED


@pytest.mark.parametrize("batch,cols", [(1, 128), (7, 5120), (223, 2304), (130, 17408)])
def test_quantize_d4_bit_exact(gpu, oracle, batch, cols):
    x = synth.normal(batch, cols, seed=7 + batch + cols)
    _, got = quantize_d4(x)
    rc, ref = oracle.quantize_q8_1_d4(x)
    assert rc == 0
    assert np.array_equal(got, ref), f"{(got != ref).sum()} differing bytes"


def test_quantize_d4_special_and_heavy_tail(gpu, oracle):
    x = special_rows(256)[:8]   # NaN/inf rows are covered by the Q8_1 test
    _, got = quantize_d4(x)
    rc, ref = oracle.quantize_q8_1_d4(x)
    assert np.array_equal(got, ref)
    t = synth.student_t3(64, 5120, seed=11)
    _, got = quantize_d4(t)
    rc, ref = oracle.quantize_q8_1_d4(t)
    assert np.array_equal(got, ref)
    _, got = quantize_q8_1(t)
    rc, ref = oracle.quantize_q8_1(t)
    assert np.array_equal(got, ref)
