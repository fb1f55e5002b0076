import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
PKG_NAME = "ascend-transformer-boost_amd"
# error-path tests would otherwise fill stderr with the library's ERROR lines
os.environ.setdefault("ASCEND_GLOBAL_LOG_LEVEL", "4")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _ensure_built():
    lib = os.path.join(ROOT, PKG_NAME, "lib")
    if not (os.path.exists(os.path.join(lib, "libatb.so")) and
            os.path.exists(os.path.join(lib, "libatbmi_kernels.so"))):
        build = importlib.import_module(PKG_NAME + ".build")
        build.build_all()


@pytest.fixture(scope="session")
def pkg():
    _ensure_built()
    return importlib.import_module(PKG_NAME)


@pytest.fixture(scope="session")
def binding(pkg):
    return pkg.binding


@pytest.fixture(scope="session")
def oracle():
    return importlib.import_module("oracle.atb_oracle")
