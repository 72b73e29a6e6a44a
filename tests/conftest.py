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


class _Tune:
    """Tuning switches of the native libraries with monkeypatch's vocabulary: setenv / delenv on UGHIP_<NAME> go to
    ughip_set_tuning, on UG_LLAMA_<NAME> to the host library's switches (both tables are read from the environment only
    once per process, so changing os.environ would do nothing); everything set is cleared at teardown."""

    def __init__(self):
        self.touched = set()

    def setenv(self, name, value):
        import ug_amd
        self.touched.add(name)
        if name.startswith("UG_LLAMA_"):
            ug_amd.set_llama_switch(name, True)
        else:
            ug_amd.set_tuning(name, int(value))

    def delenv(self, name, raising=False):
        import ug_amd
        if name.startswith("UG_LLAMA_"):
            ug_amd.set_llama_switch(name, False)
        else:
            ug_amd.set_tuning(name, None)

    def undo(self):
        for name in self.touched:
            self.delenv(name)


@pytest.fixture
def tune():
    t = _Tune()
    yield t
    t.undo()
