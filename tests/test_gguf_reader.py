"""GGUF v3 reader of the host layer (kvmem-qw3_amd/host/gguf_q8.cpp), no GPU needed.

The files are written here, field by field, from the published container layout; the reader is
a separate C++ implementation, so agreement pins both.  Error behaviour follows the reference's
reader (src/gguf.cpp:217-277): wrong magic, version other than 3, truncation, a tensor that points
outside the file, rank above 8, quantized tensors that are not whole blocks."""
import os
import struct
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROBE = os.path.join(ROOT, "tests", "cpp", "gguf_probe")

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)


def gstr(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def gval(t, v):
    fmt = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q",
           I64: "<q", F64: "<d"}
    if t == STR:
        return gstr(v)
    if t == ARR:
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(gval(et, i) for i in items)
    return struct.pack(fmt[t], v)


def write_gguf(path, kvs, tensors, alignment=32, version=3, magic=b"GGUF", truncate=None, shift_last=0):
    """tensors: list of (name, dims, ggml_type, raw bytes)."""
    head = magic + struct.pack("<IQQ", version, len(tensors), len(kvs))
    for k, t, v in kvs:
        head += gstr(k) + struct.pack("<I", t) + gval(t, v)
    offs, data = [], b""
    for name, dims, typ, raw in tensors:
        pad = (-len(data)) % alignment
        data += b"\0" * pad
        offs.append(len(data))
        data += raw
    for i, ((name, dims, typ, raw), off) in enumerate(zip(tensors, offs)):
        if i == len(tensors) - 1:
            off += shift_last
        head += gstr(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", typ, off)
    blob = head + b"\0" * ((-len(head)) % alignment) + data
    if truncate is not None:
        blob = blob[:truncate]
    with open(path, "wb") as f:
        f.write(blob)
    return len(head) + ((-len(head)) % alignment), offs


def fnv1a64(b):
    h = 1469598103934665603
    for x in b:
        h = ((h ^ x) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


def probe(path):
    r = subprocess.run([PROBE, path], capture_output=True, text=True)
    return r.returncode, r.stdout.splitlines()


@pytest.fixture(scope="module")
def have_probe():
    if not os.path.exists(PROBE):
        pytest.fail("tests/cpp/gguf_probe is not built (run __graft_entry__.build())")


@pytest.mark.parametrize("alignment", [32, 64, 4096])
def test_reader_parses_what_was_written(tmp_path, have_probe, oracle, alignment):
    rng = np.random.default_rng(alignment)
    w = rng.standard_normal((48, 256)).astype(np.float32)
    q8 = oracle.quantize_q8_0(w).tobytes()                       # interleaved 34-byte blocks
    norm = rng.standard_normal(256).astype(np.float32).tobytes()
    exps = rng.standard_normal((3, 8, 64)).astype(np.float32)    # rank 3: rows = 3 * 8
    q8b = oracle.quantize_q8_0(exps.reshape(24, 64)).tobytes()
    kvs = [("general.architecture", STR, "qwen3"), ("general.alignment", U32, alignment),
           ("qwen3.block_count", U32, 64), ("qwen3.rope.freq_base", F32, 1000000.0),
           ("tokenizer.ggml.tokens", ARR, (STR, ["a", "bc", "", "d e"])),
           ("tokenizer.ggml.scores", ARR, (F32, [0.5, -1.0, 2.0])),
           ("general.file_type", I32, -7), ("flag", BOOL, 1), ("big", U64, 2 ** 40 + 3),
           ("nested", ARR, (ARR, [(U8, [1, 2]), (U16, [3])]))]
    tensors = [("token_embd.weight", [256, 48], 8, q8), ("output_norm.weight", [256], 0, norm),
               ("blk.0.ffn_gate_exps.weight", [64, 8, 3], 8, q8b)]
    if alignment == 32:
        kvs = [kv for kv in kvs if kv[0] != "general.alignment"]    # the default applies
    path = str(tmp_path / "m.gguf")
    data_off, offs = write_gguf(path, kvs, tensors, alignment)
    rc, lines = probe(path)
    assert rc == 0, lines
    assert lines[0].split() == ["header", "3", str(alignment), str(data_off), "3", str(len(kvs))]
    got_kv = {l.split(" ", 3)[1]: l.split(" ", 3)[2:] for l in lines if l.startswith("kv ")}
    assert got_kv["general.architecture"] == [str(STR), "qwen3"]
    assert got_kv["qwen3.block_count"] == [str(U32), "64"]
    assert got_kv["qwen3.rope.freq_base"] == [str(F32), "1000000"]
    assert got_kv["general.file_type"] == [str(I32), "-7"]
    assert got_kv["flag"] == [str(BOOL), "1"]
    assert got_kv["big"] == [str(U64), str(2 ** 40 + 3)]
    assert got_kv["tokenizer.ggml.tokens"] == [str(ARR), "4 a bc  d e"]
    assert got_kv["tokenizer.ggml.scores"] == [str(ARR), "3"]
    assert got_kv["nested"] == [str(ARR), "2"]
    got_t = [l.split() for l in lines if l.startswith("tensor ")]
    want = [("token_embd.weight", 8, "Q8_0", 48, 256, q8), ("output_norm.weight", 0, "F32", 1, 256, norm),
            ("blk.0.ffn_gate_exps.weight", 8, "Q8_0", 24, 64, q8b)]
    for g, (name, typ, tname, rows, cols, raw), off in zip(got_t, want, offs):
        assert g[1:6] == [name, str(typ), tname, str(rows), str(cols)]
        assert int(g[6]) == off and int(g[7]) == data_off + off and int(g[8]) == len(raw)
        assert off % alignment == 0
        assert int(g[9], 16) == fnv1a64(raw), name


def test_reader_rejections(tmp_path, have_probe):
    raw = bytes(34 * 4)
    t = [("w", [64, 2], 8, raw)]
    cases = {
        "magic": dict(magic=b"GGML"),
        "version": dict(version=2),
        "truncated": dict(truncate=40),
        "outside": dict(shift_last=1 << 20),
    }
    expect = {"magic": "does not start with the GGUF magic", "version": "version 2 is not supported",
              "truncated": "file ends inside", "outside": "lies outside the file"}
    for name, kw in cases.items():
        path = str(tmp_path / f"{name}.gguf")
        write_gguf(path, [("general.architecture", STR, "x")], t, **kw)
        rc, lines = probe(path)
        assert rc == 2 and lines and expect[name] in lines[-1], (name, lines)
    # rank above 8, quantized tensor that is not whole blocks, empty file, missing file
    path = str(tmp_path / "rank.gguf")
    write_gguf(path, [], [("w", [2] * 9, 0, bytes(4 * 512))])
    assert "has rank 9 (at most 8)" in probe(path)[1][-1]
    path = str(tmp_path / "blocks.gguf")
    write_gguf(path, [], [("w", [48], 8, bytes(51))])
    assert "do not fill whole blocks" in probe(path)[1][-1]
    path = str(tmp_path / "empty.gguf")
    open(path, "wb").close()
    assert "is empty" in probe(path)[1][-1]
    assert "cannot open" in probe(str(tmp_path / "absent.gguf"))[1][-1]
    # metadata of an unknown type
    path = str(tmp_path / "kvtype.gguf")
    with open(path, "wb") as f:
        f.write(b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + gstr("k") + struct.pack("<I", 99) + bytes(64))
    assert "metadata type 99 is not known" in probe(path)[1][-1]
