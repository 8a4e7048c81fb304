"""The C ABI from a caller that has no Python and no torch: ``ditango_amd/csrc/capi_demo.cpp`` includes only
``include/ditango_hip.h`` and the HIP runtime, allocates with hipMalloc, runs two chunks of attention, their merge,
a round trip through a cache slot and a device-built schedule row, and checks each against host loops in double
precision (out 2e-2, lse 1e-3, bf16 slot and schedule exact).  ``python -m ditango_amd.build`` links it next to the
library; here it only runs."""
import subprocess

import pytest

from ditango_amd.build import DEMO_PATH

pytestmark = pytest.mark.gpu


def test_c_caller_without_torch():
    if not DEMO_PATH.exists():
        pytest.skip(f"{DEMO_PATH} is not built (python -m ditango_amd.build links it)")
    res = subprocess.run([str(DEMO_PATH)], capture_output=True, text=True, timeout=100)
    print(res.stdout, res.stderr, flush=True)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "capi demo ok" in res.stdout
