import ctypes as C

from .. import api


def call(f):
    """Errors surface as ValueError, as in ug-pyo3 (ug-pyo3/src/lib.rs:6-8)."""
    try:
        return f()
    except api.UgError as e:
        raise ValueError(str(e)) from None


def text(fn, handle):
    """A string returned through (buf, len) by one of the host library's *_str functions."""
    lib = api.host_lib()
    f = getattr(lib, fn)
    f.restype = C.c_size_t
    n = f(api._p(handle), None, C.c_size_t(0))
    buf = C.create_string_buffer(n + 1)
    f(api._p(handle), buf, C.c_size_t(n + 1))
    return buf.value.decode()


def dims(shape):
    shape = tuple(int(d) for d in shape)
    return (C.c_size_t * len(shape))(*shape), len(shape)
