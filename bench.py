#!/usr/bin/env python3
"""Bench of the Q8_0 quantized-linear hot path on one MI355X.

One "step" = one pass over the decode GEMV set of one 27B-style layer at M=1
(config 1 of the benchmark definition), through the C ABI, every operator reading its own fp32
input as in the model (the fan-out reads the attention norm's output, the SwiGLU the FFN norm's):

    qgemv_fanout4(x_attn[5120])   Q 5120x6144, K 5120x1024, V 5120x1024 (quantizer inside the GEMV)
    qgemv_add(a[6144])            O 6144x5120, residual add (quantizer inside the GEMV)
    quantize_q8_1(x_ffn[5120])
    gemv_silu_mul                 gate, up 5120x17408 each
    quantize_q8_1(f[17408])
    gemv_add                      down 17408x5120, residual add

(the faster of "quantizer inside" and "quantizer launch + GEMV" for each operator); for batch 2..8
every operator is quantize_q8_1 + GEMV (8 launches).

`value` is algorithmic bytes per step / time per step with all inputs resident
in HBM, cycling through several distinct copies of the layer's weights so that
no copy can be served from the 256 MB last-level cache ("streaming").  The same
loop on a single copy is reported as `resident_gbps`.

Prints ONE JSON line (see the keys at the bottom).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "kvmem-qw3_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))      # q8mi_support: input generators and ceiling probes

HBM_PEAK_GBPS = 8000.0        # MI355X published HBM3E bandwidth
INT8_PEAK_TOPS = 5000.0       # MI355X published dense int8 MFMA rate (TOP/s)

HIDDEN, QDIM, KVDIM, ATTN_OUT, FFN, VOCAB = 5120, 24 * 256, 4 * 256, 6144, 17408, 248320


def w_bytes(rows, cols):
    return rows * (cols // 32) * 34


def q81_bytes(m, cols):
    return m * (cols // 32) * 36


class Layer:
    """Device-resident Q8_0 weights of one layer (one seed)."""

    def __init__(self, synth, hip, seed):
        shapes = {"q": (QDIM, HIDDEN), "k": (KVDIM, HIDDEN), "v": (KVDIM, HIDDEN), "o": (HIDDEN, ATTN_OUT),
                  "gate": (FFN, HIDDEN), "up": (FFN, HIDDEN), "down": (HIDDEN, FFN)}
        self.w = {}
        for i, (name, (rows, cols)) in enumerate(shapes.items()):
            host = synth.q8_0_weight(rows, cols, seed=seed * 16 + i, sigma=0.02)
            self.w[name] = hip.to_device(host)
        self.bytes = sum(w_bytes(r, c) for r, c in shapes.values())


class DecodeStep:
    """Buffers + the launch sequence of one layer's decode GEMVs for batch m."""

    def __init__(self, q8mi, hip, m, seed=1):
        import q8mi_support as synth
        self.L = q8mi.lib()
        self.ok = q8mi.ok
        self.m = m
        f32 = lambda n: hip.DeviceBuffer(4 * n)
        self.x = hip.to_device(synth.normal(m, HIDDEN, seed=seed))          # attention norm's output
        self.x_ffn = hip.to_device(synth.normal(m, HIDDEN, seed=seed + 3))  # FFN norm's output
        self.attn = hip.to_device(synth.normal(m, ATTN_OUT, seed=seed + 1))  # attention output
        self.h = hip.to_device(synth.normal(m, HIDDEN, seed=seed + 2))       # residual stream
        self.q, self.k, self.v = f32(m * QDIM), f32(m * KVDIM), f32(m * KVDIM)
        self.ffn = f32(m * FFN)
        self.y5120 = hip.DeviceBuffer(q81_bytes(m, HIDDEN))
        self.y6144 = hip.DeviceBuffer(q81_bytes(m, ATTN_OUT))
        self.y17408 = hip.DeviceBuffer(q81_bytes(m, FFN))

    def algorithmic_bytes(self, layer_bytes):
        return decode_step_bytes(self.m, layer_bytes)

    @property
    def launches(self):
        return 6 if self.m == 1 else 8

    def run(self, layer, stream=None):
        """Every operator on its own fp32 input.  At M=1 the fan-out and the O projection quantize
        inside the GEMV (one launch instead of two); the SwiGLU and the down projection, and every
        operator at M >= 2, read Q8_1 blocks from a quantizer launch of their own."""
        L, m, w = self.L, self.m, layer.w
        ok = self.ok
        if m == 1:
            ok(L.q8mi_qgemv_fanout4(w["q"].ptr, w["k"].ptr, w["v"].ptr, None, self.x.ptr, HIDDEN,
                                    self.q.ptr, self.k.ptr, self.v.ptr, None, QDIM, KVDIM, KVDIM, 0,
                                    HIDDEN, m, QDIM, KVDIM, KVDIM, 0, stream), "qfanout4")
            ok(L.q8mi_qgemv_add(w["o"].ptr, self.attn.ptr, ATTN_OUT, self.h.ptr, 0, HIDDEN, ATTN_OUT, m, HIDDEN,
                                stream), "qo")
        else:
            ok(L.q8mi_quantize_q8_1(self.x.ptr, self.y5120.ptr, m, HIDDEN, HIDDEN, stream), "quantize x")
            ok(L.q8mi_gemv_fanout4(w["q"].ptr, w["k"].ptr, w["v"].ptr, None, self.y5120.ptr,
                                   self.q.ptr, self.k.ptr, self.v.ptr, None, QDIM, KVDIM, KVDIM, 0,
                                   HIDDEN, m, QDIM, KVDIM, KVDIM, 0, stream), "fanout4")
            ok(L.q8mi_quantize_q8_1(self.attn.ptr, self.y6144.ptr, m, ATTN_OUT, ATTN_OUT, stream), "quantize attn")
            ok(L.q8mi_gemv_add(w["o"].ptr, self.y6144.ptr, self.h.ptr, HIDDEN, ATTN_OUT, m, HIDDEN, stream), "o")
        ok(L.q8mi_quantize_q8_1(self.x_ffn.ptr, self.y5120.ptr, m, HIDDEN, HIDDEN, stream), "quantize x_ffn")
        self.run_silu(layer, stream)
        ok(L.q8mi_quantize_q8_1(self.ffn.ptr, self.y17408.ptr, m, FFN, FFN, stream), "quantize ffn")
        ok(L.q8mi_gemv_add(w["down"].ptr, self.y17408.ptr, self.h.ptr, HIDDEN, FFN, m, HIDDEN, stream), "down")

    def run_with_norms(self, layer, one_launch, stream=None):
        """The same GEMVs at M=1 preceded by the layer's two RMS norms: inside the fan-out and
        SwiGLU launches (5 launches), or as norm + quantizer kernels of their own in front of
        them (7)."""
        L, w, ok = self.L, layer.w, self.ok
        if not hasattr(self, "norm_w"):
            import numpy as np
            from q8mi import hip
            self.norm_w = hip.to_device(np.ones(HIDDEN, np.float32))
            self.h_in = hip.to_device(np.linspace(-2.0, 2.0, HIDDEN, dtype=np.float32))
        eps = 1e-6
        def fanout():
            if one_launch:
                ok(L.q8mi_nqgemv_fanout4(w["q"].ptr, w["k"].ptr, w["v"].ptr, None, self.h_in.ptr, self.norm_w.ptr, eps,
                                         self.x.ptr, self.q.ptr, self.k.ptr, self.v.ptr, None, QDIM, KVDIM, KVDIM, 0,
                                         HIDDEN, 1, stream), "nqfanout4")
                return
            ok(L.q8mi_rms_norm_quantize_q8_1(self.h_in.ptr, self.norm_w.ptr, self.x.ptr, self.y5120.ptr, 1, HIDDEN, HIDDEN,
                                             HIDDEN, eps, stream), "norm+quantize")
            ok(L.q8mi_gemv_fanout4(w["q"].ptr, w["k"].ptr, w["v"].ptr, None, self.y5120.ptr, self.q.ptr, self.k.ptr,
                                   self.v.ptr, None, QDIM, KVDIM, KVDIM, 0, HIDDEN, 1, QDIM, KVDIM, KVDIM, 0, stream), "fanout4")
        def silu():
            if one_launch:
                ok(L.q8mi_nqgemv_silu_mul(w["gate"].ptr, w["up"].ptr, self.h_in.ptr, self.norm_w.ptr, eps, self.x.ptr,
                                          self.ffn.ptr, FFN, HIDDEN, 1, stream), "nqsilu_mul")
                return
            ok(L.q8mi_rms_norm_quantize_q8_1(self.h_in.ptr, self.norm_w.ptr, self.x.ptr, self.y5120.ptr, 1, HIDDEN, HIDDEN,
                                             HIDDEN, eps, stream), "norm+quantize")
            ok(L.q8mi_gemv_silu_mul(w["gate"].ptr, w["up"].ptr, self.y5120.ptr, self.ffn.ptr, FFN, HIDDEN, 1, FFN, stream),
               "silu_mul")
        fanout()
        ok(L.q8mi_qgemv_add(w["o"].ptr, self.attn.ptr, ATTN_OUT, self.h.ptr, 0, HIDDEN, ATTN_OUT, 1, HIDDEN, stream), "qo")
        silu()
        ok(L.q8mi_quantize_q8_1(self.ffn.ptr, self.y17408.ptr, 1, FFN, FFN, stream), "quantize ffn")
        ok(L.q8mi_gemv_add(w["down"].ptr, self.y17408.ptr, self.h.ptr, HIDDEN, FFN, 1, HIDDEN, stream), "down")

    def run_silu(self, layer, stream=None):
        """gate/up SwiGLU on the Q8_1 blocks of x (quantized by run(), or by prepare_silu())."""
        self.ok(self.L.q8mi_gemv_silu_mul(layer.w["gate"].ptr, layer.w["up"].ptr, self.y5120.ptr, self.ffn.ptr,
                                          FFN, HIDDEN, self.m, FFN, stream), "silu_mul")

    def prepare_silu(self):
        self.ok(self.L.q8mi_quantize_q8_1(self.x.ptr, self.y5120.ptr, self.m, HIDDEN, HIDDEN, None), "quantize x")

    def silu_bytes(self):
        return 2 * w_bytes(FFN, HIDDEN) + q81_bytes(self.m, HIDDEN) + 4 * self.m * FFN


def time_loop(hip, fn, steps, warmup):
    """Device time of `steps` calls of fn(i), HIP events on the (default) stream."""
    for i in range(warmup):
        fn(i)
    hip.synchronize()
    e0, e1 = hip.Event(), hip.Event()
    e0.record()
    for i in range(steps):
        fn(warmup + i)
    e1.record()
    e1.synchronize()
    hip.synchronize()
    return e0.elapsed_ms(e1) / steps


def settle(hip, fn, ms=40.0, chunk=50):
    """Untimed calls of fn(i) until `ms` of device time have passed.  After host-side work (weight
    generation, uploads: the GPU idles for seconds) the first tens of milliseconds of device work
    run a few per cent slow, which a fixed handful of warm-up launches of a 10 us kernel does not
    cover (the fused LM head read 195 us as the first case timed and 193 us as a later one)."""
    done, total = 0, 0.0
    while total < ms:
        total += time_loop(hip, lambda i: fn(done + i), chunk, 0) * chunk
        done += chunk


def time_loop_settled(hip, fn, steps, warmup, settle_ms=40.0, min_ms=100.0):
    """The headline timing, robust against small --steps / --warmup: `warmup` untimed steps, then
    further untimed rounds until settle_ms of device time have passed since the host-side set-up
    (the first ~20 ms after it run a few per cent slow), then timed rounds of `steps` steps each
    until at least min_ms of device time has been timed.  Returns (ms per step, steps timed)."""
    done = 0
    for i in range(warmup):
        fn(done + i)
    done += warmup
    hip.synchronize()
    round_ms = time_loop(hip, lambda i: fn(done + i), steps, 0) * steps     # untimed in effect: sizes the rest
    done += steps
    settled = round_ms
    while settled < settle_ms:
        settled += time_loop(hip, lambda i: fn(done + i), steps, 0) * steps
        done += steps
    total_ms, timed = 0.0, 0
    while timed == 0 or total_ms < min_ms:
        total_ms += time_loop(hip, lambda i: fn(done + i), steps, 0) * steps
        done += steps
        timed += steps
    return total_ms / timed, timed


def time_graph_replays(hip, record, steps, warmup):
    """Device time per replay of the launches `record(stream)` makes, captured once as a HIP graph
    on a stream of its own (events recorded on that stream)."""
    stream = hip.Stream()
    record(stream.handle)            # eager once: first-use set-up of every kernel happens outside the capture
    stream.synchronize()
    g = hip.Graph(stream)
    with g:
        record(stream.handle)
    for _ in range(warmup):
        g.launch()
    stream.synchronize()
    e0, e1 = hip.Event(), hip.Event()
    e0.record(stream)
    for _ in range(steps):
        g.launch()
    e1.record(stream)
    e1.synchronize()
    return e0.elapsed_ms(e1) / steps


def time_each_launch(hip, fn, n, warmup=5):
    """Average duration of single launches, one event pair per launch."""
    for i in range(warmup):
        fn(i)
    hip.synchronize()
    pairs = [(hip.Event(), hip.Event()) for _ in range(n)]
    for i, (a, b) in enumerate(pairs):
        a.record()
        fn(warmup + i)
        b.record()
    hip.synchronize()
    ds = np.array([a.elapsed_ms(b) for a, b in pairs])
    return float(ds.mean()), float(np.median(ds)), float(ds.min())


def cpu_baseline(seconds=12.0):
    """The oracle's scalar GEMV (oracle/q8_oracle.c) on benchmark config 0
    (5120x5120, M=1), timed on this host: once on one core, once row-parallel."""
    sys.path.insert(0, ROOT)
    from oracle import q8_oracle as o
    import q8mi_support as synth
    rows = cols = HIDDEN
    w = synth.q8_0_weight(rows, cols, seed=12345)
    x = synth.normal(1, cols, seed=54321)
    rc, y = o.quantize_q8_1(x)
    nbytes = w_bytes(rows, cols) + q81_bytes(1, cols) + 4 * rows

    def run(threads, budget):
        o.gemv(w, y, rows, cols, 1, threads=threads)     # warm
        n, t0 = 0, time.perf_counter()
        while True:
            o.gemv(w, y, rows, cols, 1, threads=threads)
            n += 1
            dt = time.perf_counter() - t0
            if dt >= budget:
                return nbytes * n / dt / 1e9, n

    cores = min(16, os.cpu_count() or 1)
    one, n1 = run(1, seconds / 2)
    many, nm = run(cores, seconds / 2)
    return {"value": round(many, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "host_cpu_count": os.cpu_count(),
            "sample": f"oracle q8o_gemv, config 0 (5120x5120, M=1), {nm} calls row-parallel on {cores} threads "
                      f"of the {os.cpu_count()} the host reports (~{seconds / 2:.0f} s); single core: {one:.3f} GB/s "
                      f"over {n1} calls",
            "value_1core": round(one, 3)}


def cpu_gemm_sample(rows=2048, m=2048, cols=HIDDEN):
    """The oracle's scalar GEMM (D4 activations) on a row slice of the M=2048 gate/up shape,
    row-parallel on the host cores: a bounded sample of the prefill GEMM's CPU rate."""
    sys.path.insert(0, ROOT)
    from oracle import q8_oracle as o
    import q8mi_support as synth
    w = synth.q8_0_weight(rows, cols, seed=99)
    x = synth.normal(m, cols, seed=98)
    rc, y = o.quantize_q8_1_d4(x)
    cores = min(16, os.cpu_count() or 1)
    t0 = time.perf_counter()
    o.gemm_d4(w, y, rows, cols, m, threads=cores)
    dt = time.perf_counter() - t0
    return {"tops": round(2.0 * m * rows * cols / dt / 1e12, 4), "cores": cores, "seconds": round(dt, 2),
            "sample": f"oracle q8o_gemm_d4, {rows} of 17408 weight rows x M={m} x K={cols}"}


def bench_config0(q8mi, hip, synth, copies=48, reps=480):
    """Benchmark config 0: one 5120x5120 GEMV at M=1.  The GEMV proper reads Q8_1 activations
    (q8mi_gemv: what the bytes of this config count); also timed: the entry point that quantizes
    fp32 activations inside the GEMV, and quantizer + GEMV as two launches.
    Streaming: cycles through `copies` weight buffers (1.3 GB, no cache hits); resident: one buffer."""
    L, ok = q8mi.lib(), q8mi.ok
    host = synth.q8_0_weight(HIDDEN, HIDDEN, seed=31)
    ws = [hip.to_device(host) for _ in range(copies)]
    x = hip.to_device(synth.normal(1, HIDDEN, seed=32))
    y = hip.DeviceBuffer(q81_bytes(1, HIDDEN))
    dst = hip.DeviceBuffer(4 * HIDDEN)
    quant = lambda: ok(L.q8mi_quantize_q8_1(x.ptr, y.ptr, 1, HIDDEN, HIDDEN, None), "quantize")
    gemv = lambda w: ok(L.q8mi_gemv(w.ptr, y.ptr, dst.ptr, HIDDEN, HIDDEN, 1, HIDDEN, None), "gemv")
    qgemv = lambda w: ok(L.q8mi_qgemv(w.ptr, x.ptr, HIDDEN, dst.ptr, 0, HIDDEN, HIDDEN, 1, HIDDEN, None), "qgemv")
    quant()
    settle(hip, lambda i: gemv(ws[i % copies]))
    t_stream = time_loop(hip, lambda i: gemv(ws[i % copies]), reps, copies)
    t_res = time_loop(hip, lambda i: gemv(ws[0]), reps, 10)
    t_fused = time_loop(hip, lambda i: qgemv(ws[i % copies]), reps, copies)
    t_two = time_loop(hip, lambda i: (quant(), gemv(ws[i % copies])), reps, copies)
    nbytes = w_bytes(HIDDEN, HIDDEN) + q81_bytes(1, HIDDEN) + 4 * HIDDEN
    for b in ws + [x, y, dst]:
        b.free()
    gbps = lambda t: round(nbytes / (t * 1e-3) / 1e9, 1)
    return {"bytes": nbytes, "streaming_us": round(t_stream * 1e3, 3), "streaming_gbps": gbps(t_stream),
            "frac_of_hbm_peak": round(gbps(t_stream) / HBM_PEAK_GBPS, 4),
            "resident_us": round(t_res * 1e3, 3), "resident_gbps": gbps(t_res),
            "fp32_activations_one_launch_us": round(t_fused * 1e3, 3),
            "fp32_activations_quantizer_plus_gemv_us": round(t_two * 1e3, 3)}


def bench_launches_m1(q8mi, hip, synth, step, layers, reps=300):
    """Every launch of the M=1 step on its own, back to back over the rotating weight copies, beside
    a plain streaming read of the same number of bytes (windows of a 1 GiB buffer, so the
    memory-side cache cannot serve it): time, bytes, rate, and time / read time."""
    L, ok, m = q8mi.lib(), q8mi.ok, 1
    big, sink = hip.DeviceBuffer(1 << 30), hip.DeviceBuffer(64)
    nl = len(layers)

    def probe_us(nbytes):
        span = (nbytes + 4095) // 4096 * 4096
        windows = (1 << 30) // span
        fn = lambda i: synth.ok(synth.lib().q8sup_probe_read(big.at((i % windows) * span), nbytes, 2, sink.ptr, None),
                                "probe_read")
        return time_loop(hip, fn, reps, 20) * 1e3

    def fan(i):
        w = layers[i % nl].w
        ok(L.q8mi_qgemv_fanout4(w["q"].ptr, w["k"].ptr, w["v"].ptr, None, step.x.ptr, HIDDEN, step.q.ptr, step.k.ptr,
                                step.v.ptr, None, QDIM, KVDIM, KVDIM, 0, HIDDEN, m, QDIM, KVDIM, KVDIM, 0, None), "qfanout4")
    ops = [
        ("qgemv_fanout4 q/k/v 8192x5120 (fp32 in)", w_bytes(QDIM + 2 * KVDIM, HIDDEN), fan),
        ("qgemv_add o 5120x6144 (fp32 in)", w_bytes(HIDDEN, ATTN_OUT),
         lambda i: ok(L.q8mi_qgemv_add(layers[i % nl].w["o"].ptr, step.attn.ptr, ATTN_OUT, step.h.ptr, 0, HIDDEN,
                                       ATTN_OUT, m, HIDDEN, None), "qo")),
        ("quantize_q8_1 x_ffn (5120 floats)", 0,
         lambda i: ok(L.q8mi_quantize_q8_1(step.x_ffn.ptr, step.y5120.ptr, m, HIDDEN, HIDDEN, None), "quantize")),
        ("gemv_silu_mul gate/up 2x17408x5120", 2 * w_bytes(FFN, HIDDEN), lambda i: step.run_silu(layers[i % nl])),
        ("quantize_q8_1 ffn (17408 floats)", 0,
         lambda i: ok(L.q8mi_quantize_q8_1(step.ffn.ptr, step.y17408.ptr, m, FFN, FFN, None), "quantize")),
        ("gemv_add down 5120x17408", w_bytes(HIDDEN, FFN),
         lambda i: ok(L.q8mi_gemv_add(layers[i % nl].w["down"].ptr, step.y17408.ptr, step.h.ptr, HIDDEN, FFN, m,
                                      HIDDEN, None), "down")),
    ]
    step.prepare_silu()
    settle(hip, ops[0][2])
    out = []
    for name, nbytes, fn in ops:
        us = time_loop(hip, fn, reps, 20) * 1e3
        row = {"launch": name, "weight_bytes": nbytes, "us": round(us, 2)}
        if nbytes:
            pus = probe_us(nbytes)
            row.update({"gbps": round(nbytes / us / 1e3, 1), "plain_read_us": round(pus, 2), "ratio": round(us / pus, 3)})
        out.append(row)
    big.free()
    sink.free()
    return out


def bench_row_length_sweep(q8mi, hip, synth, rows=HIDDEN, reps=300):
    """q8mi_gemv at M=1 on `rows` weight rows of K columns, K = every whole number of KiB up to 17
    and a few lengths in between, beside a plain streaming read of the same bytes: what a row length
    without a kernel of its own costs.  Weights cycle through copies laid out in a 1 GiB buffer."""
    L, ok = q8mi.lib(), q8mi.ok
    big, sink = hip.DeviceBuffer(1 << 30), hip.DeviceBuffer(64)
    out = {}
    for cols in sorted(set(range(1024, 17408 + 1, 1024)) | {2560, 3584, 5632, 9728}):
        host = synth.q8_0_weight(rows, cols, seed=cols)
        nbytes = w_bytes(rows, cols)
        span = (nbytes + 4095) // 4096 * 4096
        copies = min((1 << 30) // span, 64)
        for c in range(copies):
            big.upload(host, c * span)
        x = hip.to_device(synth.normal(1, cols, seed=cols + 1))
        y = hip.DeviceBuffer(q81_bytes(1, cols))
        dst = hip.DeviceBuffer(4 * rows)
        ok(L.q8mi_quantize_q8_1(x.ptr, y.ptr, 1, cols, cols, None), "quantize")
        gemv = lambda i: ok(L.q8mi_gemv(big.at((i % copies) * span), y.ptr, dst.ptr, rows, cols, 1, rows, None), "gemv")
        settle(hip, gemv, ms=20.0)   # the host generated and uploaded this length's weights just now
        t = time_loop(hip, gemv, reps, copies)
        p = time_loop(hip, lambda i: synth.ok(synth.lib().q8sup_probe_read(big.at((i % copies) * span), nbytes, 2, sink.ptr,
                                                                           None), "probe_read"), reps, copies)
        out[f"k{cols}"] = {"us": round(t * 1e3, 2), "plain_read_us": round(p * 1e3, 2), "ratio": round(t / p, 3),
                           "gbps": round((nbytes + q81_bytes(1, cols) + 4 * rows) / (t * 1e-3) / 1e9, 1)}
        for b in (x, y, dst):
            b.free()
    big.free()
    sink.free()
    return out


def bench_read_probe(synth, hip, nbytes=1 << 30, reps=20):
    """Measured ceiling of a plain streaming read (every lane 16 bytes per load, grid-stride)."""
    buf, sink = hip.DeviceBuffer(nbytes), hip.DeviceBuffer(64)
    fn = lambda i: synth.ok(synth.lib().q8sup_probe_read(buf.ptr, nbytes, 2, sink.ptr, None), "probe_read")
    settle(hip, fn, chunk=10)
    t = time_loop(hip, fn, reps, 3)
    buf.free()
    sink.free()
    return round(nbytes / (t * 1e-3) / 1e9, 1)


def bench_mfma_ceilings(synth, hip, iters=5000):
    """Measured issue-rate ceilings of the matrix unit (register-only loops, two workgroups per CU):
    int8 MFMAs alone; with the 2 scalar fp32 FMAs per int32 sum that rescaling costs (packed fp32 math
    is not available), independent and fed by the MFMA results as in the kernel; and the arithmetic
    with 1 FMA per sum (block sums as fp32 from the fp16 matrix unit, scale products from the fp32
    matrix unit), in int8-equivalent TOP/s."""
    L = synth.lib()
    sink = hip.DeviceBuffer(L.q8sup_probe_mfma_sink_bytes())
    ops = C.c_uint64(0)
    out = {}
    for name, mode in (("mfma_only_tops", 0), ("mfma_with_rescale_tops", 1), ("mfma_with_dependent_rescale_tops", 3),
                       ("f16_mfma_one_fma_per_sum_tops", 2)):
        fn = lambda i: synth.ok(L.q8sup_probe_mfma(mode, iters, sink.ptr, C.byref(ops), None), "probe_mfma")
        t = time_loop(hip, fn, 3, 1)
        out[name] = round(ops.value / (t * 1e-3) / 1e12, 1)
    sink.free()
    return out


def bench_gemm(q8mi, hip, synth, reps=10):
    """Prefill GEMM (D4 quantize + MFMA GEMM): M=2048 on the two FFN shapes, M=8192 on gate/up."""
    L, ok = q8mi.lib(), q8mi.ok
    out = {}
    for name, rows, cols, m in (("m2048_k5120_n17408", FFN, HIDDEN, 2048), ("m2048_k17408_n5120", HIDDEN, FFN, 2048),
                                ("m8192_k5120_n17408", FFN, HIDDEN, 8192)):
        w = hip.to_device(synth.q8_0_weight(rows, cols, seed=rows + 7))
        x = hip.to_device(synth.normal(m, cols, seed=cols + 9))
        y = hip.DeviceBuffer(L.q8mi_q8_1_d4_scratch_bytes(m, cols))
        dst = hip.DeviceBuffer(4 * m * rows)
        ok(L.q8mi_quantize_q8_1_d4(x.ptr, y.ptr, m, cols, cols, None), "quantize_d4")
        gemm = lambda i: ok(L.q8mi_gemm(w.ptr, y.ptr, dst.ptr, rows, cols, m, rows, None), "gemm")
        quant = lambda i: ok(L.q8mi_quantize_q8_1_d4(x.ptr, y.ptr, m, cols, cols, None), "quantize_d4")
        t_gemm = time_loop(hip, gemm, reps, 3)
        t_quant = time_loop(hip, quant, reps, 3)
        ops = 2.0 * m * rows * cols
        out[name] = {"gemm_ms": round(t_gemm, 4), "quantize_ms": round(t_quant, 4),
                     "tops": round(ops / (t_gemm * 1e-3) / 1e12, 2),
                     "frac_of_int8_peak": round(ops / (t_gemm * 1e-3) / 1e12 / INT8_PEAK_TOPS, 4),
                     "tops_with_quantize": round(ops / ((t_gemm + t_quant) * 1e-3) / 1e12, 2)}
        for b in (w, x, y, dst):
            b.free()
    return out


def bench_gemm_medium(q8mi, hip, synth, reps=30):
    """Batches between the GEMV's and the prefill tile's (continuous-batching sizes) on the three
    layer shapes: D4 activations through q8mi_gemm, microseconds per call over rotating weight copies."""
    L, ok = q8mi.lib(), q8mi.ok
    out = {}
    for rows, cols in ((HIDDEN, HIDDEN), (FFN, HIDDEN), (HIDDEN, FFN)):
        ws = [hip.to_device(synth.q8_0_weight(rows, cols, seed=s + 31)) for s in range(3)]
        per = {}
        for m in (16, 32, 64, 128):
            x = hip.to_device(synth.normal(m, cols, seed=m))
            y = hip.DeviceBuffer(L.q8mi_q8_1_d4_scratch_bytes(m, cols))
            dst = hip.DeviceBuffer(4 * m * rows)
            ok(L.q8mi_quantize_q8_1_d4(x.ptr, y.ptr, m, cols, cols, None), "quantize_d4")
            gemm = lambda i: ok(L.q8mi_gemm(ws[i % 3].ptr, y.ptr, dst.ptr, rows, cols, m, rows, None), "gemm")
            settle(hip, gemm, ms=20.0)
            t = time_loop(hip, gemm, reps, 3)
            per[f"m{m}"] = round(t * 1e3, 1)
            for b in (x, y, dst):
                b.free()
        out[f"k{cols}_n{rows}_us"] = per
        for b in ws:
            b.free()
    return out


def split_to_gguf(split, rows, cols):
    """Split-plane rows ([fp16 d x nb][int8 x 32 nb]) back to interleaved 34-byte GGUF blocks:
    what DeviceBackend::weight_q8_0 takes."""
    nb = cols // 32
    rows_v = np.asarray(split, np.uint8).reshape(rows, nb * 34)
    d = rows_v[:, :2 * nb].reshape(rows, nb, 2)
    q = rows_v[:, 2 * nb:].reshape(rows, nb, 32)
    return np.ascontiguousarray(np.concatenate([d, q], axis=2)).reshape(-1)


class BackendSteps:
    """The layer's operators driven through qw3::HipQ8Backend (the C++ mirror of the reference's
    DeviceBackend) in the executors' call order: tests/cpp/backend_steps.cpp behind ctypes."""

    SHAPES = (("q", QDIM, HIDDEN), ("k", KVDIM, HIDDEN), ("v", KVDIM, HIDDEN), ("o", HIDDEN, ATTN_OUT),
              ("gate", FFN, HIDDEN), ("up", FFN, HIDDEN), ("down", HIDDEN, FFN))

    def __init__(self, synth, n_layers):
        path = os.path.join(ROOT, "tests", "cpp", "libbackend_steps.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: run __graft_entry__.build()")
        B = C.CDLL(path)
        B.bsteps_create.restype = C.c_void_p
        B.bsteps_create.argtypes = [C.c_uint32] * 5
        B.bsteps_destroy.argtypes = [C.c_void_p]
        B.bsteps_error.restype = C.c_char_p
        B.bsteps_error.argtypes = [C.c_void_p]
        B.bsteps_add_layer.argtypes = [C.c_void_p] * 8
        B.bsteps_set_head.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32]
        B.bsteps_prepare.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p]
        B.bsteps_time_layers.restype = C.c_double
        B.bsteps_time_layers.argtypes = [C.c_void_p, C.c_int, C.c_uint32, C.c_uint32]
        B.bsteps_time_head.restype = C.c_double
        B.bsteps_time_head.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
        self.B, self.synth = B, synth
        self.h = B.bsteps_create(HIDDEN, QDIM, KVDIM, ATTN_OUT, FFN)
        for s in range(n_layers):
            blocks = [split_to_gguf(synth.q8_0_weight(r, c, seed=(s + 1) * 16 + i, sigma=0.02), r, c)
                      for i, (_, r, c) in enumerate(self.SHAPES)]
            if B.bsteps_add_layer(self.h, *[b.ctypes.data_as(C.c_void_p) for b in blocks]) < 0:
                raise RuntimeError("backend steps: weight upload failed")

    def prepare(self, m):
        h, mid = self.synth.normal(m, HIDDEN, seed=71), self.synth.normal(m, ATTN_OUT, seed=72)
        if self.B.bsteps_prepare(self.h, m, h.ctypes.data_as(C.c_void_p), mid.ctypes.data_as(C.c_void_p)) != 0:
            raise RuntimeError("backend steps: tensor set-up failed")

    def time_layers(self, order, steps, warmup):
        ms = self.B.bsteps_time_layers(self.h, order, steps, warmup)
        if ms < 0:
            raise RuntimeError("backend steps: " + (self.B.bsteps_error(self.h) or b"").decode())
        return ms

    def set_head(self):
        blocks = split_to_gguf(self.synth.q8_0_weight(VOCAB, HIDDEN, seed=4242), VOCAB, HIDDEN)
        if self.B.bsteps_set_head(self.h, blocks.ctypes.data_as(C.c_void_p), VOCAB) != 0:
            raise RuntimeError("backend steps: LM head upload failed")

    def time_head(self, calls, warmup):
        ms = self.B.bsteps_time_head(self.h, calls, warmup, None, None)
        if ms < 0:
            raise RuntimeError("backend steps: " + (self.B.bsteps_error(self.h) or b"").decode())
        return ms

    def close(self):
        self.B.bsteps_destroy(self.h)


def bench_backend_layers(synth, n_layers, steps, layer_bytes, with_head=True):
    """Microseconds per layer step through HipQ8Backend: decode (M=1) in the executor's order, and
    M = 2, 4, 6, 8 in the executor's batched order (matmul + add_n) and the continuous-batching
    verifier's (matmul_add in place); the two RMS norms of the layer are part of each step.  Also the
    verify tail (final norm + fused LM head, host read of the accept result included)."""
    bs = BackendSteps(synth, n_layers)
    out = {}
    try:
        bs.prepare(1)
        t = bs.time_layers(-1, steps, 50)
        b1 = decode_step_bytes(1, layer_bytes)
        out["decode_m1"] = {"us_per_layer": round(t * 1e3, 2), "gbps": round(b1 / (t * 1e-3) / 1e9, 1)}
        for m in (2, 4, 6, 8):
            bs.prepare(m)
            row = {}
            for name, order in (("executor_order", 0), ("matmul_add_order", 1)):
                t = bs.time_layers(order, steps, 50)
                row[name] = {"us_per_layer": round(t * 1e3, 2),
                             "gbps": round(decode_step_bytes(m, layer_bytes) / (t * 1e-3) / 1e9, 1)}
            out[f"verify_m{m}"] = row
        if with_head:
            bs.set_head()
            head = {}
            for m in (1, 2, 4, 6, 8):
                bs.prepare(m)
                t = bs.time_head(60, 20)
                nbytes = w_bytes(VOCAB, HIDDEN) + q81_bytes(m, HIDDEN) + 8 * m
                head[f"m{m}"] = {"ms": round(t, 4), "gbps": round(nbytes / (t * 1e-3) / 1e9, 1)}
            out["norm_plus_lm_head_verify"] = head
    finally:
        bs.close()
    return out


def decode_step_bytes(m, layer_bytes):
    """Algorithmic bytes of one layer's GEMV set at batch m: the weights once, the Q8_1 blocks of the
    four activation rows, the fp32 outputs."""
    act = 2 * q81_bytes(m, HIDDEN) + q81_bytes(m, ATTN_OUT) + q81_bytes(m, FFN)
    outs = 4 * m * (QDIM + 2 * KVDIM + HIDDEN + FFN + HIDDEN)
    return layer_bytes + act + outs


def bench_prefill_ffn(q8mi, hip, synth, m=2048, reps=12):
    """The FFN block of a prefill chunk of m rows as a sequence, repeated back to back: D4 quantizer,
    gate/up SwiGLU, D4 quantizer, down projection + residual.  `separate`: the launches the
    reference's executor runs (two GEMMs + silu_mul, GEMM + add); `fused`: one tile launch per
    operator where the library has one (q8mi_gemm_silu_mul; q8mi_gemm_add unless it declines the shape)."""
    L, ok = q8mi.lib(), q8mi.ok
    wg = hip.to_device(synth.q8_0_weight(FFN, HIDDEN, seed=501))
    wu = hip.to_device(synth.q8_0_weight(FFN, HIDDEN, seed=502))
    wd = hip.to_device(synth.q8_0_weight(HIDDEN, FFN, seed=503))
    x = hip.to_device(synth.normal(m, HIDDEN, seed=504))
    h = hip.to_device(synth.normal(m, HIDDEN, seed=505))
    yx = hip.DeviceBuffer(L.q8mi_q8_1_d4_scratch_bytes(m, HIDDEN))
    yf = hip.DeviceBuffer(L.q8mi_q8_1_d4_scratch_bytes(m, FFN))
    gate, up, mid = (hip.DeviceBuffer(4 * m * FFN) for _ in range(3))
    tmp = hip.DeviceBuffer(4 * m * HIDDEN)
    add_fuses = L.q8mi_gemm_add(wd.ptr, yf.ptr, h.ptr, h.ptr, HIDDEN, FFN, m, HIDDEN, None) == q8mi.OK

    def down_separate():
        ok(L.q8mi_gemm(wd.ptr, yf.ptr, tmp.ptr, HIDDEN, FFN, m, HIDDEN, None), "gemm down")
        ok(L.q8mi_add(h.ptr, h.ptr, tmp.ptr, m * HIDDEN, 0, None), "add")

    def separate(i):
        ok(L.q8mi_quantize_q8_1_d4(x.ptr, yx.ptr, m, HIDDEN, HIDDEN, None), "quantize x")
        ok(L.q8mi_gemm(wg.ptr, yx.ptr, gate.ptr, FFN, HIDDEN, m, FFN, None), "gemm gate")
        ok(L.q8mi_gemm(wu.ptr, yx.ptr, up.ptr, FFN, HIDDEN, m, FFN, None), "gemm up")
        ok(L.q8mi_silu_mul(mid.ptr, gate.ptr, up.ptr, m * FFN, None), "silu_mul")
        ok(L.q8mi_quantize_q8_1_d4(mid.ptr, yf.ptr, m, FFN, FFN, None), "quantize mid")
        down_separate()

    def fused(i):
        ok(L.q8mi_quantize_q8_1_d4(x.ptr, yx.ptr, m, HIDDEN, HIDDEN, None), "quantize x")
        ok(L.q8mi_gemm_silu_mul(wg.ptr, wu.ptr, yx.ptr, mid.ptr, FFN, HIDDEN, m, FFN, None), "gemm_silu_mul")
        ok(L.q8mi_quantize_q8_1_d4(mid.ptr, yf.ptr, m, FFN, FFN, None), "quantize mid")
        if add_fuses:
            ok(L.q8mi_gemm_add(wd.ptr, yf.ptr, h.ptr, h.ptr, HIDDEN, FFN, m, HIDDEN, None), "gemm_add")
        else:
            down_separate()

    # alternate the two forms so that both see the same clocks: sustained matrix work runs the chip at its power limit
    t_sep, t_fus = [], []
    for _ in range(3):
        t_sep.append(time_loop(hip, separate, reps, 2))
        t_fus.append(time_loop(hip, fused, reps, 2))
    ops = 2.0 * m * FFN * HIDDEN * 3
    for b in (wg, wu, wd, x, h, yx, yf, gate, up, mid, tmp):
        b.free()
    t_s, t_f = min(t_sep), min(t_fus)
    return {"m": m, "separate_launches_ms": round(t_s, 4), "fused_stores_ms": round(t_f, 4),
            "separate_tops": round(ops / (t_s * 1e-3) / 1e12, 1), "fused_tops": round(ops / (t_f * 1e-3) / 1e12, 1),
            "down_plus_residual_in_one_launch": add_fuses, "all_rounds_ms": {"separate": [round(t, 4) for t in t_sep],
                                                                             "fused": [round(t, 4) for t in t_fus]}}


def bench_batch_sweep(q8mi, hip, step, layers, steps):
    """The layer's GEMV set at M = 1, 2, 3, 4, 6, 8 (quantizer launches included)."""
    sweep = {}
    for m in (1, 2, 3, 4, 6, 8):
        st = step if m == 1 else DecodeStep(q8mi, hip, m=m)
        b = st.algorithmic_bytes(layers[0].bytes)
        t = time_loop(hip, lambda i: st.run(layers[i % len(layers)]), steps, 50)
        sweep[f"m{m}"] = {"ms_per_step": round(t, 5), "gbps": round(b / (t * 1e-3) / 1e9, 1)}
    return sweep


def bench_small_launch_cost(q8mi, hip, synth, layers, reps=400):
    """What a small launch costs behind a large one on the same stream: the batch-8 down projection back to
    back on its own, followed by a 4 KB read, and followed by the batch-8 quantizer of 5120 columns
    (microseconds per repetition).  A kernel trace shows such a small dispatch open for 4 to 5 us, because it
    is open while the launch in front of it drains; what it adds to the sequence is the difference here."""
    L, ok = q8mi.lib(), q8mi.ok
    st = DecodeStep(q8mi, hip, m=8)
    ok(L.q8mi_quantize_q8_1(st.ffn.ptr, st.y17408.ptr, 8, FFN, FFN, None), "quantize ffn")
    sink, small = hip.DeviceBuffer(64), hip.DeviceBuffer(4096)
    down = lambda i: ok(L.q8mi_gemv_add(layers[i % len(layers)].w["down"].ptr, st.y17408.ptr, st.h.ptr, HIDDEN, FFN, 8,
                                        HIDDEN, None), "down")
    def with_read(i):
        down(i)
        synth.ok(synth.lib().q8sup_probe_read(small.ptr, 4096, 2, sink.ptr, None), "probe_read")
    def with_quantizer(i):
        down(i)
        ok(L.q8mi_quantize_q8_1(st.x.ptr, st.y5120.ptr, 8, HIDDEN, HIDDEN, None), "quantize x")
    out = {}
    for name, fn in (("down_m8_alone_us", down), ("followed_by_a_4kb_read_us", with_read),
                     ("followed_by_the_m8_quantizer_us", with_quantizer)):
        settle(hip, fn, ms=10.0)
        out[name] = round(time_loop(hip, fn, reps, 20) * 1e3, 2)
    return out


def bench_lm_head(q8mi, hip, synth, reps=100):
    """Fused LM head (5120 x 248320) + argmax + accept at M = 1, 2, 4, 6, 8."""
    L, ok = q8mi.lib(), q8mi.ok
    w = hip.to_device(synth.q8_0_weight(VOCAB, HIDDEN, seed=4242))
    out = {}
    for m in (1, 2, 4, 6, 8):
        x = hip.to_device(synth.normal(m, HIDDEN, seed=m))
        y = hip.DeviceBuffer(q81_bytes(m, HIDDEN))
        ok(L.q8mi_quantize_q8_1(x.ptr, y.ptr, m, HIDDEN, HIDDEN, None), "quantize")
        scratch = hip.DeviceBuffer(L.q8mi_lm_head_scratch_bytes(VOCAB, HIDDEN, m))
        rows_out, acc = hip.DeviceBuffer(8 * m), hip.DeviceBuffer(8)
        drafts = np.zeros(8, np.int32)
        fn = lambda i: ok(L.q8mi_lm_head_argmax_accept(w.ptr, y.ptr, VOCAB, HIDDEN, m,
                                                       drafts.ctypes.data_as(C.c_void_p), 0, 0, rows_out.ptr,
                                                       acc.ptr, None, VOCAB, scratch.ptr, None), "lm_head")
        # after the seconds of host-side weight generation above, untimed calls first (see settle)
        if not out:
            settle(hip, fn, chunk=20)
        t = time_loop(hip, fn, reps, 50)
        nbytes = w_bytes(VOCAB, HIDDEN) + q81_bytes(m, HIDDEN) + 8 * m
        out[f"m{m}"] = {"ms": round(t, 4), "gbps": round(nbytes / (t * 1e-3) / 1e9, 1)}
    w.free()
    return out


TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gemv_pairs_silu_m1_hbm_traffic.txt")
COPY_BYTES = 1 << 28


def measured_traffic():
    """HBM bytes per launch of the dominant kernel from hardware counters, as recorded in
    the committed counter summary (line `traffic_bytes_per_launch: N`); None if absent."""
    try:
        with open(TRAFFIC_FILE) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return int(float(line.split(":", 1)[1]))
    except OSError:
        pass
    return None


def counter_calibration(synth, hip, n=3):
    """A few launches of a plain copy kernel of known size (reads and writes COPY_BYTES
    each): the reference point that memory-traffic counters of a profiled run are scaled by."""
    src, dst = hip.DeviceBuffer(COPY_BYTES), hip.DeviceBuffer(COPY_BYTES)
    for _ in range(n):
        synth.ok(synth.lib().q8sup_probe_copy(src.ptr, dst.ptr, COPY_BYTES, None), "probe_copy")
    hip.synchronize()
    src.free()
    dst.free()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # a step is ~80 us; whatever --steps and --warmup say, at least 40 ms run untimed first and at
    # least 100 ms are timed (rounds of --steps steps), see time_loop_settled
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--copies", type=int, default=4, help="distinct weight copies cycled through (streaming)")
    ap.add_argument("--quick", action="store_true", help="headline number only: skip M sweep, GEMM, LM head, CPU")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", choices=["gemm", "lm_head", "ceilings", "sweep", "backend", "prefill_ffn", "row_lengths"], help="one secondary figure alone (for profiling runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU's throughput; run with --gpus 1 "
                 "(the path would shard by weight rows: each GPU keeps rows/N of every weight)")

    import q8mi
    from q8mi import hip
    import q8mi_support as synth
    if hip.device_count() < 1:
        sys.exit("bench.py: no HIP device visible")
    hip.set_device(0)
    q8mi.lib()

    if args.only == "gemm":
        print(json.dumps({"gemm_int8": bench_gemm(q8mi, hip, synth, reps=10),
                          "gemm_medium_batches": bench_gemm_medium(q8mi, hip, synth)}))
        return
    if args.only == "ceilings":
        print(json.dumps({"measured_ceilings": bench_mfma_ceilings(synth, hip)}))
        return
    if args.only == "lm_head":
        print(json.dumps({"lm_head_fused": bench_lm_head(q8mi, hip, synth)}))
        return
    if args.only == "backend":
        lb = sum(w_bytes(r, c) for _, r, c in BackendSteps.SHAPES)
        print(json.dumps({"through_hip_q8_backend": bench_backend_layers(synth, args.copies, max(args.steps // 2, 300), lb)}))
        return
    if args.only == "row_lengths":
        print(json.dumps({"gemv_m1_by_row_length_n5120": bench_row_length_sweep(q8mi, hip, synth)}))
        return
    if args.only == "prefill_ffn":
        print(json.dumps({"prefill_ffn_block": {f"m{m}": bench_prefill_ffn(q8mi, hip, synth, m=m, reps=r)
                                                for m, r in ((2048, 12), (8192, 4))}}))
        return
    if args.only == "sweep":
        layers = [Layer(synth, hip, seed=s + 1) for s in range(args.copies)]
        print(json.dumps({"gemv_layer_gbps_by_m": bench_batch_sweep(q8mi, hip, DecodeStep(q8mi, hip, m=1), layers,
                                                                     max(args.steps // 2, 300)),
                          "small_launch_behind_a_large_one": bench_small_launch_cost(q8mi, hip, synth, layers)}))
        return
    counter_calibration(synth, hip)
    layers = [Layer(synth, hip, seed=s + 1) for s in range(args.copies)]
    step = DecodeStep(q8mi, hip, m=1)
    step_bytes = step.algorithmic_bytes(layers[0].bytes)

    # headline: rounds of K timed steps over rotating weight copies, at least 100 ms of device time
    ms_stream, steps_timed = time_loop_settled(hip, lambda i: step.run(layers[i % len(layers)]), args.steps, args.warmup)
    value = step_bytes / (ms_stream * 1e-3) / 1e9
    ms_resident, _ = time_loop_settled(hip, lambda i: step.run(layers[0]), args.steps, 0, settle_ms=0.0, min_ms=50.0)

    # dominant kernel: the gate/up SwiGLU GEMV (52 % of the step's bytes)
    n_each = min(max(args.steps, 50), 400)
    step.prepare_silu()
    mean_ms, med_ms, min_ms = time_each_launch(hip, lambda i: step.run_silu(layers[i % len(layers)]), n_each)
    back_ms = time_loop(hip, lambda i: step.run_silu(layers[i % len(layers)]), n_each, 5)
    silu_bytes = step.silu_bytes()
    # average launch duration = HIP events around n_each back-to-back launches / n_each
    # (event pairs around single launches add ~1.5 us of their own; kept as launch_ms_*)
    achieved = silu_bytes / (back_ms * 1e-3) / 1e9
    result = {
        "metric": "Q8_0 GEMV HBM GB/s at M=1 (decode GEMV set of one 27B-style layer)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "steps_timed": steps_timed, "device": hip.device_name(),
        "ms_per_step": round(ms_stream, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 x int8 -> int32 dots, fp32 accumulate", "data": "synthetic",
        "config": {"workload": "BASELINE config 1: decode GEMV set of one layer, M=1 "
                               "(QKV 5120x8192 fan-out, O 6144x5120 +residual, gate/up 5120x17408 SwiGLU, "
                               "down 17408x5120 +residual), Q8_0 N(0,0.02) weights, Q8_1 N(0,1) activations",
                   "weight_copies_cycled": args.copies, "bytes_per_step": step_bytes,
                   "launches_per_step": step.launches},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "resident_gbps": round(step_bytes / (ms_resident * 1e-3) / 1e9, 1),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": measured_traffic(),
                     "kernel": "gemv_pairs_ksplit_kernel<1, 5, 5, true, false, false> (SwiGLU: gate+up 2 x 5120x17408, Q8_1 activations)",
                     "bytes_per_launch": silu_bytes, "launch_ms": round(back_ms, 5),
                     "launch_ms_mean": round(mean_ms, 5),
                     "launch_ms_median": round(med_ms, 5), "launch_ms_min": round(min_ms, 5),
                     "launches_timed": n_each},
    }

    if not args.quick:
        # the same step captured once as a HIP graph and replayed: 64 steps per graph (a decode graph of
        # the model holds 64 layers), cycling through the weight sets
        per_graph = 64
        def record(stream):
            for i in range(per_graph):
                step.run(layers[i % len(layers)], stream)
        ms_graph = time_graph_replays(hip, record, max(args.steps // per_graph, 10), 3) / per_graph
        result["graph_replay"] = {"ms_per_step": round(ms_graph, 5), "steps_per_graph": per_graph,
                                  "gbps": round(step_bytes / (ms_graph * 1e-3) / 1e9, 1)}
        result["gemv_layer_gbps_by_m"] = bench_batch_sweep(q8mi, hip, step, layers, max(args.steps // 2, 300))
        result["small_launch_behind_a_large_one"] = bench_small_launch_cost(q8mi, hip, synth, layers)
        # the layer's two RMS norms in front of the fan-out and the SwiGLU: inside those launches, or on their own
        norms = {}
        for name, one in (("norms_inside_the_gemv_5_launches", True), ("norm_quantizer_kernels_7_launches", False)):
            t = time_loop(hip, lambda i: step.run_with_norms(layers[i % len(layers)], one), max(args.steps // 2, 300), 50)
            norms[name] = {"ms_per_step": round(t, 5), "gbps": round(step_bytes / (t * 1e-3) / 1e9, 1)}
        result["layer_with_rms_norms_m1"] = norms
        result["launches_m1"] = bench_launches_m1(q8mi, hip, synth, step, layers)
        # the same layer through the C++ operator layer, in the executors' call order
        result["through_hip_q8_backend"] = bench_backend_layers(synth, len(layers), max(args.steps // 2, 300), layers[0].bytes)
    for l in layers[1:]:
        for b in l.w.values():
            b.free()
    if not args.quick:
        result["config0_gemv_m1"] = bench_config0(q8mi, hip, synth)
        result["hbm_read_probe_gbps"] = bench_read_probe(synth, hip)
        result["gemv_m1_by_row_length_n5120"] = bench_row_length_sweep(q8mi, hip, synth)
        result["gemm_int8"] = bench_gemm(q8mi, hip, synth)
        ceil = bench_mfma_ceilings(synth, hip)
        for v in result["gemm_int8"].values():
            v["frac_of_rescale_ceiling"] = round(v["tops"] / ceil["mfma_with_rescale_tops"], 4)
        result["gemm_int8"]["measured_ceilings"] = ceil
        # the second half of the dual metric in the shape of `roofline`: prefill GEMM at M=2048, gate/up shape
        g = result["gemm_int8"]["m2048_k5120_n17408"]
        result["roofline_gemm"] = {"bound": "mfma", "achieved": g["tops"], "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                                   "frac": g["frac_of_int8_peak"], "traffic": None,
                                   "kernel": "gemm_d4_dma_kernel<false, 4, false> (128 x 128 tiles, M=2048, K=5120, N=17408)",
                                   "ops_per_launch": 2 * 2048 * FFN * HIDDEN, "launch_ms": g["gemm_ms"],
                                   "frac_of_measured_rescale_ceiling": g["frac_of_rescale_ceiling"]}
        result["gemm_medium_batches"] = bench_gemm_medium(q8mi, hip, synth)
        result["prefill_ffn_block"] = {f"m{m}": bench_prefill_ffn(q8mi, hip, synth, m=m, reps=r) for m, r in ((2048, 12), (8192, 4))}
        result["lm_head_fused"] = bench_lm_head(q8mi, hip, synth)
    if not (args.quick or args.no_cpu):
        result["cpu_baseline"] = cpu_baseline()
        result["cpu_baseline"]["gemm_int8"] = cpu_gemm_sample()
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
