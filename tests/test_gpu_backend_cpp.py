"""Runs the C++ backend parity driver (tests/cpp/backend_parity.cpp): HipQ8Backend, the
host-side mirror of the reference's device operator interface, against the CPU oracle."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "tests", "cpp", "backend_parity")

CASES = ["closed_form", "matvec", "matmul", "matmul_add", "silu_mul", "norm_reuse", "argmax", "get_rows", "gguf", "lm_head", "rms_norm", "graph"]


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_backend_parity_driver(case):
    assert os.path.exists(DRIVER), "backend parity driver is not built (run __graft_entry__.build())"
    r = subprocess.run([DRIVER, case], capture_output=True, text=True, timeout=110)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert " 0 failed" in r.stdout


def test_host_library_exports_backend():
    """No GPU needed: the host library exists and carries the backend's entry points."""
    lib = os.path.join(ROOT, "kvmem-qw3_amd", "host", "libq8mi_host.so")
    assert os.path.exists(lib), "libq8mi_host.so is not built"
    out = subprocess.run(["nm", "-DC", "--defined-only", lib], capture_output=True, text=True, check=True).stdout
    for method in ("q8_0_matvec(", "q8_0_matvec_add(", "q8_0_matvec_silu_mul(", "q8_0_matvec_fanout(",
                   "q8_0_matmul(", "q8_0_matmul_fanout(", "q8_0_matmul_add(", "q8_0_matmul_silu_mul(", "silu_mul(", "silu_mul_n(",
                   "add(", "add_n(", "argmax(", "argmax_batch(",
                   "argmax_to_buffer(", "q8_0_get_row(", "q8_0_get_row_from_argmax(", "q8_0_get_rows_batch(",
                   "weight_q8_0(", "lm_head_verify(", "begin_capture(", "replay_graph("):
        assert f"qw3::HipQ8Backend::{method}" in out, method
