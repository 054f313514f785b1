import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950); run with -m gpu on the GPU box")


@pytest.fixture(scope="session")
def vectors():
    """Known-answer vectors transcribed from the reference (tests/golden/make_fixtures.py)."""
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def oracle():
    import oracle as O  # oracle/oracle.py: the CPU checker, test infrastructure only

    return O


@pytest.fixture(scope="session")
def hip():
    """The device tier of the product. GPU tests fail loudly if the library is not usable there."""
    from frankentorch_amd import device

    if not device.is_available():
        if os.path.exists("/dev/kfd"):
            pytest.fail("a GPU driver node exists but the HIP library reports no usable gfx950 device")
        pytest.skip("no MI355X in this container")
    return device


def rel_err(got, ref):
    """max|got - ref| / max|ref|, the tolerance form of the metric definition."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    denom = np.max(np.abs(ref)) if ref.size else 1.0
    if denom == 0.0:
        denom = 1.0
    return float(np.max(np.abs(got - ref)) / denom) if ref.size else 0.0


# Tolerances of the metric definition: fp32 row ops, fp32 GEMM / attention, fp64.
TOL_ROW_F32 = 1e-5
TOL_GEMM_F32 = 2e-5
TOL_F64 = 1e-12

# Column sums over the batch (dweight, dbias of the norm and linear backward): the reference adds the rows in one serial
# chain; the kernels add (rows of a workgroup) then (workgroups), and for long batches the re-associated fp32 sum of
# thousands of terms differs from the serial one by a few ulp of the largest partial sum. Enforced bar: 4x the row-op bar.
NORM_COLSUM_TOL_FACTOR = 4
