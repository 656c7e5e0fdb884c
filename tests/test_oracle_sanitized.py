"""The CPU oracle under AddressSanitizer and UndefinedBehaviorSanitizer: a C driver
(oracle/sanitize_check.c) calls every oracle function on exactly-sized heap buffers; an
out-of-bounds access, a misaligned access or undefined arithmetic anywhere in the oracle
stops it with a non-zero exit status."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_oracle_runs_clean_under_sanitizers():
    r = subprocess.run(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "sanitize"], capture_output=True, text=True,
                       timeout=600)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-4000:]
    assert "sanitize_check: ok" in r.stdout
