import ctypes as C
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _oracle_lib():
    """The CPU oracle (oracle/): test infrastructure only -- never imported by the product."""
    from oracle.load import oracle_lib
    try:
        return oracle_lib()
    except RuntimeError as e:
        pytest.fail(str(e))


@pytest.fixture(scope="session")
def oracle():
    return _oracle_lib()


@pytest.fixture(scope="session")
def cpu(oracle):
    """ug::CpuDevice restatement, usable wherever a ug_amd.Device is."""
    from oracle.load import cpu_device
    return cpu_device()


@pytest.fixture(scope="session")
def cpu_ops(oracle):
    from oracle.load import cpu_llama_ops
    return cpu_llama_ops()


@pytest.fixture(scope="session")
def hip():
    """The HIP device; fails loudly when the GPU or the native library is missing."""
    import ug_amd
    return ug_amd.hip_device(0)


@pytest.fixture(scope="session")
def hip_ops():
    import ug_amd
    return ug_amd.LlamaOps.hip()
