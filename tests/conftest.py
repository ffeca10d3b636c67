import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle_native():
    from oracle.native import OracleNative
    return OracleNative()


@pytest.fixture()
def orc(oracle_native):
    """API namespace (Tensor, Linear, Adam ...) bound to a freshly reset CPU oracle."""
    from framework_amd.api import bind
    oracle_native.resetEngine()
    return bind(oracle_native)


@pytest.fixture(scope="session")
def rocm_native():
    from framework_amd.native import Native, Rocm
    r = Rocm()
    r.init(0)
    return Native()


@pytest.fixture(scope="session")
def rocm():
    from framework_amd.native import Rocm
    r = Rocm()
    r.init(0)
    return r


@pytest.fixture()
def gpu(rocm_native):
    """API namespace bound to a freshly reset HIP engine."""
    from framework_amd.api import bind
    rocm_native.resetEngine()
    return bind(rocm_native)
