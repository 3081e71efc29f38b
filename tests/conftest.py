import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def checker():
    """The plain-C restatement of the reference's CPU path (oracle/liboracle.so)."""
    import oracle
    if not os.path.exists(oracle.ORACLE_PATH):
        pytest.fail("oracle/liboracle.so is not built (run __graft_entry__.build())")
    return oracle.Oracle()


@pytest.fixture(scope="session")
def reference():
    """The reference itself compiled for the CPU (oracle/_ref/libacro_ref.so); tests that need it are skipped
    where it has not been built."""
    import oracle
    if not oracle.have_reference():
        pytest.skip("oracle/_ref/libacro_ref.so not built (needs the reference sources)")
    return oracle.Reference()


@pytest.fixture(scope="session")
def at():
    import acrotensor_amd
    return acrotensor_amd


@pytest.fixture(scope="session")
def engine(at):
    """A TensorEngine on the HIP policy (GPU tests only)."""
    if not at.is_hip_ready():
        pytest.fail("GPU test selected but no HIP device is usable: the HIP path must not be skipped silently")
    return at.TensorEngine("HIP")
