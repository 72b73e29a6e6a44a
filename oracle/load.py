"""Loads the CPU oracle's shared library (oracle/_build/libug_oracle.so).  TEST INFRASTRUCTURE ONLY: used by tests/,
by __graft_entry__.smoke() and by bench.py's CPU-baseline legs as the checker / the baseline -- never by the product
(nothing under ug_amd/ imports this)."""
import ctypes as C
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_lib = None


def oracle_lib():
    global _lib
    if _lib is None:
        import ug_amd  # noqa: F401  (loads libug_host.so first; the oracle links against it)
        path = os.path.join(ROOT, "oracle", "_build", "libug_oracle.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} missing: run `python -m ug_amd.build` first")
        _lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
        _lib.ugo_last_error.restype = C.c_char_p
    return _lib


def cpu_device():
    """The restatement of ug::CpuDevice, usable wherever a ug_amd.Device is."""
    import ug_amd
    out = C.c_void_p()
    if oracle_lib().ugo_cpu_device_new(C.byref(out)) != 0:
        raise RuntimeError(oracle_lib().ugo_last_error().decode())
    return ug_amd.Device(out.value)


def cpu_llama_ops():
    """The restatement of ug-llama/src/cpu_ops.rs as a ug_amd.LlamaOps."""
    import ug_amd
    out = C.c_void_p()
    if oracle_lib().ugo_llama_ops_cpu(C.byref(out)) != 0:
        raise RuntimeError(oracle_lib().ugo_last_error().decode())
    return ug_amd.LlamaOps(out.value)
