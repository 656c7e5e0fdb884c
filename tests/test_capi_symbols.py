"""The C-ABI library loads on a machine without a GPU and exports every function
that include/q8mi.h declares (no compute is called here)."""
import os
import re
import subprocess

import q8mi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "q8mi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(q8mi_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    names = declared_functions()
    assert len(names) >= 26
    assert sorted(q8mi.SIGNATURES) == names


def test_library_exports_every_declared_symbol():
    lib = q8mi.lib()
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in q8mi.h but not exported"
    out = subprocess.run(["nm", "-D", "--defined-only", q8mi.LIB_PATH], capture_output=True, text=True).stdout
    exported = set(re.findall(r" T (q8mi_[a-z0-9_]+)", out))
    assert exported == set(declared_functions())
    assert lib.q8mi_abi_version() == 1


def test_instruments_live_in_their_own_library():
    """Input generators, the block-dot checker and the ceiling probes are not part of the product:
    libq8mi.so exports none of them, libq8mi_support.so exports exactly what its header declares."""
    import q8mi_support
    out = subprocess.run(["nm", "-D", "--defined-only", q8mi.LIB_PATH], capture_output=True, text=True).stdout
    assert not re.findall(r" T \w*(?:probe|synth|block_dots)\w*", out)
    text = open(os.path.join(ROOT, "tests", "q8mi_support", "q8mi_support.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = sorted(set(re.findall(r"\b(q8sup_[a-z0-9_]+)\s*\(", text)))
    assert declared == sorted(q8mi_support.SIGNATURES)
    q8mi_support.lib()
    out = subprocess.run(["nm", "-D", "--defined-only", q8mi_support.LIB_PATH], capture_output=True, text=True).stdout
    assert set(re.findall(r" T (q8sup_[a-z0-9_]+)", out)) == set(declared)


def test_host_side_entry_points_without_gpu(oracle):
    """Size helpers, the host repack and the synthetic generator run on the CPU."""
    import ctypes as C
    import numpy as np
    import q8mi_support as synth
    L = q8mi.lib()
    assert L.q8mi_q8_1_scratch_bytes(8, 17408) == 8 * 544 * 36
    assert L.q8mi_q8_1_d4_scratch_bytes(2048, 5120) == 2048 * 40 * 144
    assert L.q8mi_argmax_rows_scratch_bytes(8, 248320) == 8 * 970 * 8
    rng = np.random.default_rng(0)
    wf = (rng.standard_normal((6, 96)) * 0.02).astype(np.float32)
    gguf = oracle.quantize_q8_0(wf)
    out = np.empty_like(gguf)
    assert L.q8mi_repack_q8_0_split_host(gguf.ctypes.data_as(C.c_void_p), 6, 96, out.ctypes.data_as(C.c_void_p)) == 0
    assert np.array_equal(out, oracle.repack_split_plane(gguf, 6, 96))
    assert L.q8mi_repack_q8_0_split_host(None, 1, 33, None) == q8mi.REJECTED
    assert "33" in q8mi.last_error()
    # the generator's weights equal oracle-quantized weights of the generator's floats
    assert np.array_equal(synth.q8_0_weight(16, 256, seed=5), oracle.make_weight(synth.normal(16, 256, 5, scale=0.02)))
    # thread count does not change the bytes
    assert np.array_equal(synth.q8_0_weight(64, 256, seed=6, threads=1), synth.q8_0_weight(64, 256, seed=6, threads=7))
    x = synth.normal(64, 4096, seed=8)
    assert abs(x.mean()) < 0.01 and abs(x.std() - 1) < 0.01
    t = synth.student_t3(256, 4096, seed=9, outlier_ppm=0)
    assert abs(np.median(np.abs(t)) - 0.7649 / np.sqrt(3)) < 0.01      # median |t3| = 0.7649
    t = synth.student_t3(16, 8192, seed=9, outlier_ppm=1000)
    cols = np.nonzero(np.abs(t).mean(axis=0) > 5)[0]
    assert 1 <= len(cols) <= 30                                          # about 0.1 % of the columns x 20
