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
    import ug_amd  # noqa: F401  (loads libug_host.so first; the oracle links against it)
    path = os.path.join(ROOT, "oracle", "_build", "libug_oracle.so")
    if not os.path.exists(path):
        pytest.fail(f"{path} missing: run `python -m ug_amd.build` first")
    lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
    lib.ugo_last_error.restype = C.c_char_p
    return lib


@pytest.fixture(scope="session")
def oracle():
    return _oracle_lib()


@pytest.fixture(scope="session")
def cpu(oracle):
    """ug::CpuDevice restatement, usable wherever a ug_amd.Device is."""
    import ug_amd
    out = C.c_void_p()
    assert oracle.ugo_cpu_device_new(C.byref(out)) == 0, oracle.ugo_last_error()
    return ug_amd.Device(out.value)


@pytest.fixture(scope="session")
def cpu_ops(oracle):
    import ug_amd
    out = C.c_void_p()
    assert oracle.ugo_llama_ops_cpu(C.byref(out)) == 0, oracle.ugo_last_error()
    return ug_amd.LlamaOps(out.value)


@pytest.fixture(scope="session")
def hip():
    """The HIP device; fails loudly when the GPU or the native library is missing."""
    import ug_amd
    return ug_amd.hip_device(0)


@pytest.fixture(scope="session")
def hip_ops():
    import ug_amd
    return ug_amd.LlamaOps.hip()
