import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "kvmem-qw3_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionfinish(session, exitstatus):
    """GPU runs leave what the fp32 comparisons measured (largest relative error per check family
    and how many outputs needed the sum|t_kb| term of the bound) beside the run's other output."""
    try:
        import gpu_common
    except Exception:
        return
    if not gpu_common.TOLERANCE_STATS:
        return
    import json
    out_dir = os.path.join(ROOT, "gpurun_out")
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "tolerance_stats.json"), "w") as f:
        json.dump(gpu_common.TOLERANCE_STATS, f, indent=1, sort_keys=True)


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (built on demand from oracle/q8_oracle.c)."""
    from oracle import q8_oracle
    q8_oracle.lib()
    return q8_oracle


@pytest.fixture(scope="session")
def gpu():
    """Loaded C-ABI library + HIP runtime on device 0.  Fails (not skips) when the
    library is not built: GPU tests must never pass without the native code."""
    import q8mi
    from q8mi import hip
    if hip.device_count() < 1:
        pytest.fail("GPU test selected but no HIP device is visible")
    hip.set_device(0)
    q8mi.lib()
    return q8mi
