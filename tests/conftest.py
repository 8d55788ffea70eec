import importlib.util
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "strix.rs_amd")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def _load_by_path(name, path, search=None):
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(name, path, submodule_search_locations=search)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def pkg():
    """The product package (directory name has a dot, so it is loaded by path)."""
    return _load_by_path("strix_rs_amd", os.path.join(PKG_DIR, "__init__.py"), [PKG_DIR])


@pytest.fixture(scope="session")
def synth():
    return _load_by_path("strix_rs_amd_synth", os.path.join(PKG_DIR, "synth.py"))


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (test infrastructure)."""
    return _load_by_path("strix_oracle", os.path.join(ROOT, "oracle", "strix_oracle.py"))


@pytest.fixture(scope="session")
def accel(pkg):
    """One context for the whole GPU session; fails loudly without the built library or a GPU."""
    a = pkg.Mi355WeightAccel(0)
    yield a
    a.close()


def rel_err(got, ref):
    """max|got-ref| / max|ref|: the reference's normalisation (strix-backend-rocm/src/lib.rs:217-222)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))


@pytest.fixture(scope="session")
def relerr():
    return rel_err


GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


@pytest.fixture(scope="session")
def golden():
    def load(name):
        return np.load(os.path.join(GOLDEN_DIR, name), allow_pickle=False)
    return load
