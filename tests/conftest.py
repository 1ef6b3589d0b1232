import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    """Committed fixtures: seeded inputs and expectations computed with PyTorch CPU float64
    (tests/golden/make_golden.py)."""
    return np.load(os.path.join(GOLDEN_DIR, "hotpath_golden.npz"))


@pytest.fixture
def sdfg_name(request):
    # same naming rule as the reference's fixture (tests/conftest.py:53-56)
    return request.node.name.replace("[", "-").replace("]", "").replace("-", "_").replace(".", "_")


@pytest.fixture(scope="session")
def c_oracle():
    from oracle import c_oracle as c
    c.build()
    return c


def rel_err(expected, actual):
    """max |actual - expected| / max |expected|, in float64."""
    e = np.asarray(expected, dtype=np.float64)
    a = np.asarray(actual, dtype=np.float64)
    assert e.shape == a.shape, (e.shape, a.shape)
    if e.size == 0:
        return 0.0
    scale = np.abs(e).max()
    return float(np.abs(a - e).max() / (scale if scale > 0 else 1.0))


#: fp32 parity bar for every floating-point kernel: 1e-4 relative to the largest
#: magnitude of the expected tensor (integer kernels must be bit-exact)
FP32_REL_TOL = 1e-4


@pytest.fixture
def tuning():
    """Forces kernel variants through the library's ``MI355X_*`` variables: ``tuning(MI355X_GEMM_NT_BN="48")`` sets
    them (``None`` unsets one) and has the library read them again. Whatever happens in the test, the variables are
    taken back and the library re-reads its own choice before the next test runs (the library reads them once and
    caches what it found)."""
    from dace_onnx_amd import _lib
    lib = _lib.library()
    before = {}

    def force(**variables):
        for name, value in variables.items():
            assert name.startswith("MI355X_"), name
            before.setdefault(name, os.environ.get(name))
            if value is None:
                os.environ.pop(name, None)
            else:
                os.environ[name] = str(value)
        lib.mi355x_reload_tuning()

    try:
        yield force
    finally:
        for name, value in before.items():
            if value is None:
                os.environ.pop(name, None)
            else:
                os.environ[name] = value
        lib.mi355x_reload_tuning()
