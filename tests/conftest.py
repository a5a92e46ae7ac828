import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")
REFVEC = os.path.join(GOLDEN, "refvec")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import binding
    binding.lib()
    return binding


@pytest.fixture(scope="session")
def hyb(oracle):
    return oracle.Codebook()


@pytest.fixture(scope="session")
def syn(oracle):
    return oracle.Codebook(oracle.synthetic_tlut(1))


def load_pkg():
    """The package directory name has a hyphen; load it under an importable alias."""
    import importlib.util
    name = "behemoth_qtip_amd"
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(name, os.path.join(ROOT, "behemoth-qtip_amd", "__init__.py"))
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def pkg():
    return load_pkg()


@pytest.fixture(scope="session")
def qz(pkg):
    """A quantizer context on cuda:0.  GPU tests only; fails loudly without the HIP library or a gfx950 GPU."""
    q = pkg.Quantizer(0)
    yield q
    q.close()
