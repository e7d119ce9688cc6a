import pathlib
import sys

import numpy as np
import pytest

ROOT = pathlib.Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    """Arrays written by tests/golden/make_reference_vectors.py from the reference's torch code."""
    with np.load(ROOT / "tests" / "golden" / "reference_vectors.npz") as z:
        return {k: z[k] for k in z.files}


@pytest.fixture
def gemm_tuning():
    """Force a GEMM tile / in-workgroup K split for one test (flh_gemm_set_tuning); automatic again afterwards."""
    from flh_amd import _ops

    def force(tile=0, k_split=0):
        _ops.gemm_set_tuning(tile, k_split)
    yield force
    _ops.gemm_set_tuning(0, 0)
