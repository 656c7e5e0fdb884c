"""GPU parity at the model's own shapes: the decode GEMV set of one layer exactly as bench.py times
it (QKV fan-out 5120 -> 6144 + 1024 + 1024, O 6144 -> 5120 with residual, gate/up 5120 -> 17408 SwiGLU,
down 17408 -> 5120 with residual), at M = 1 (quantizer inside the fan-out and O launches), 2, 3, 4, 6 and
8, on three weight seeds, against the CPU oracle."""
import numpy as np
import pytest

import bench
from gpu_common import assert_close_fp32
import q8mi_support as synth
from q8mi import hip

pytestmark = pytest.mark.gpu

SHAPES = {"q": (bench.QDIM, bench.HIDDEN), "k": (bench.KVDIM, bench.HIDDEN), "v": (bench.KVDIM, bench.HIDDEN),
          "o": (bench.HIDDEN, bench.ATTN_OUT), "gate": (bench.FFN, bench.HIDDEN), "up": (bench.FFN, bench.HIDDEN),
          "down": (bench.HIDDEN, bench.FFN)}


# three weight seeds: the benchmark definition regenerates the layer's weights per seed
@pytest.fixture(scope="module", params=[3, 5, 11], ids=lambda s: f"seed{s}")
def layer(gpu, request):
    seed = request.param
    dev_layer = bench.Layer(synth, hip, seed=seed)
    host = {name: synth.q8_0_weight(r, c, seed=seed * 16 + i, sigma=0.02) for i, (name, (r, c)) in enumerate(SHAPES.items())}
    yield dev_layer, host
    for b in dev_layer.w.values():
        b.free()


@pytest.mark.parametrize("m", [1, 2, 3, 4, 6, 8])
def test_decode_layer_at_model_shapes(gpu, oracle, layer, m):
    dev_layer, host = layer
    step = bench.DecodeStep(gpu, hip, m, seed=40 + m)
    hip.synchronize()
    x = step.x.download(np.float32).reshape(m, bench.HIDDEN)
    x_ffn = step.x_ffn.download(np.float32).reshape(m, bench.HIDDEN)
    attn = step.attn.download(np.float32).reshape(m, bench.ATTN_OUT)
    h0 = step.h.download(np.float32).reshape(m, bench.HIDDEN)
    step.run(dev_layer)
    hip.synchronize()

    def linear(name, y):
        r, c = SHAPES[name]
        rc, ref = oracle.gemv(host[name], y, r, c, m, threads=8)
        rc, mag = oracle.gemv_abs(host[name], y, r, c, m)
        return ref, mag

    rc, yx = oracle.quantize_q8_1(x)
    for name, buf in (("q", step.q), ("k", step.k), ("v", step.v)):
        ref, mag = linear(name, yx)
        assert_close_fp32(buf.download(np.float32), ref, mag, f"{name} projection, M={m}")
    rc, yx_ffn = oracle.quantize_q8_1(x_ffn)
    g, gmag = linear("gate", yx_ffn)
    u, umag = linear("up", yx_ffn)
    rc, silu_ref = oracle.gemv_silu_mul(host["gate"], host["up"], yx_ffn, bench.FFN, bench.HIDDEN, m)
    ffn = step.ffn.download(np.float32).reshape(m, bench.FFN)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    sig = 1.0 / (1.0 + np.exp(-g64))
    lim = (1e-5 * np.abs(g64 * sig * u64) + np.abs(u64 * sig * (1.0 + g64 * (1.0 - sig))) * (1e-5 * np.abs(g64) + 1e-6 * gmag)
           + np.abs(g64 * sig) * (1e-5 * np.abs(u64) + 1e-6 * umag))
    assert np.all(np.abs(ffn - silu_ref) <= lim), f"SwiGLU, M={m}"
    # the down projection consumes the GPU's own SwiGLU output (as in the model)
    rc, ya = oracle.quantize_q8_1(attn)
    rc, yf = oracle.quantize_q8_1(ffn)
    o, omag = linear("o", ya)
    d, dmag = linear("down", yf)
    want = (h0 + o) + d
    assert_close_fp32(step.h.download(np.float32), want, np.abs(h0) + omag + dmag, f"residual stream, M={m}")


def test_decode_layer_with_norms_both_forms_agree(gpu, layer):
    """The M=1 layer with its two RMS norms, as bench.py times it: norm + quantizer inside the fan-out
    and SwiGLU launches (5 launches) against norm + quantizer kernels of their own in front of the
    Q8_1 GEMVs (7 launches).  Same bits in every output, at the model's shapes (17408 row pairs in
    one launch: workgroups of several rounds)."""
    dev_layer, _ = layer
    step = bench.DecodeStep(gpu, hip, 1, seed=77)
    hip.synchronize()
    h0 = step.h.download(np.float32)
    results = []
    for one_launch in (True, False):
        step.h.upload(h0)
        for buf in (step.q, step.k, step.v, step.ffn, step.x):
            buf.fill(0xee)
        step.run_with_norms(dev_layer, one_launch)
        hip.synchronize()
        results.append([b.download(np.uint32).copy() for b in (step.q, step.k, step.v, step.ffn, step.x, step.h)])
    for name, a, b in zip(("q", "k", "v", "ffn", "normalized x", "h"), *results):
        assert np.array_equal(a, b), name
    assert np.isfinite(results[0][3].view(np.float32)).all()
