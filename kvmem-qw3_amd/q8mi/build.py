"""Builds libq8mi.so (the C-ABI library) with hipcc for gfx950, in-tree."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.normpath(os.path.join(PKG_DIR, "..", "csrc"))
LIB_PATH = os.path.join(PKG_DIR, "libq8mi.so")

SOURCES = [
    "q8mi_host.hip",
    "q8mi_quantize.hip",
    "q8mi_gemv.hip",
    "q8mi_gemv_pairs.hip",
    "q8mi_lm_head.hip",
    "q8mi_argmax.hip",
    "q8mi_get_rows.hip",
    "q8mi_rms_norm.hip",
    "q8mi_gemm.hip",
]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Packed-fp32 VALU forms are switched off for every device compile.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wextra",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose=False):
    """Compile every source and link the shared library.  Always recompiles."""

    def compile_one(src):
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True, cwd=CSRC)
        out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                        if "packed-fp32-ops" not in l and "is not a recognized feature" not in l
                        and "loop not unrolled" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and out.strip():
            print(out, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(6, os.cpu_count() or 1)) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    link = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs, "-lpthread"]
    r = subprocess.run(link, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
