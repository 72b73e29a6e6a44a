"""`ug.op` (ug-pyo3/src/lib.rs:100-265): tensor-level expressions that lower to one SSA kernel
(ug-core/src/lang.rs:383-604, lower_op.rs)."""
import ctypes as C

from .. import api
from ._util import call, dims, text


class _Owned:
    _free = None

    def __init__(self, h):
        self._h = h

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            getattr(api.host_lib(), self._free)(api._p(h))


def _new(fn, *args):
    out = C.c_void_p()
    call(lambda: api._chk(getattr(api.host_lib(), fn)(*args, C.byref(out))))
    return out.value


class Arg(_Owned):
    """A kernel argument (lang.rs:138-178)."""
    _free = "ugh_op_arg_free"

    @staticmethod
    def _make(is_ptr, dtype):
        return Arg(_new("ugh_op_arg_new", int(is_ptr), dtype))

    @staticmethod
    def ptr_bf16():
        return Arg._make(True, api.BF16)

    @staticmethod
    def ptr_f16():
        return Arg._make(True, api.F16)

    @staticmethod
    def ptr_f32():
        return Arg._make(True, api.F32)

    @staticmethod
    def ptr_i32():
        return Arg._make(True, api.I32)

    @staticmethod
    def f32():
        return Arg._make(False, api.F32)

    @staticmethod
    def i32():
        return Arg._make(False, api.I32)

    def __str__(self):
        return text("ugh_op_arg_str", self._h)


class Ast(_Owned):
    """lib.rs:143-203."""
    _free = "ugh_op_ast_free"

    def _bin(self, op, rhs):
        if not isinstance(rhs, Ast):
            return NotImplemented
        return Ast(_new("ugh_op_binary", op, api._p(self._h), api._p(rhs._h)))

    def __add__(self, rhs):
        return self._bin(api.B_ADD, rhs)

    def __sub__(self, rhs):
        return self._bin(api.B_SUB, rhs)

    def __mul__(self, rhs):
        return self._bin(api.B_MUL, rhs)

    def __truediv__(self, rhs):
        return self._bin(api.B_DIV, rhs)

    def __neg__(self):
        return Ast(_new("ugh_op_unary", api._p(self._h), api.U_NEG))

    def exp(self):
        return Ast(_new("ugh_op_unary", api._p(self._h), api.U_EXP))

    def broadcast(self, shape):
        d, r = dims(shape)
        return Ast(_new("ugh_op_broadcast", api._p(self._h), d, C.c_size_t(r)))

    def _reduce(self, op, axis):
        return Ast(_new("ugh_op_reduce", op, api._p(self._h), C.c_size_t(int(axis))))

    def sum(self, axis):
        return self._reduce(api.R_SUM, axis)

    def min(self, axis):
        return self._reduce(api.R_MIN, axis)

    def max(self, axis):
        return self._reduce(api.R_MAX, axis)

    def shape(self):
        lib = api.host_lib()
        lib.ugh_op_ast_rank.restype = C.c_size_t
        r = lib.ugh_op_ast_rank(api._p(self._h))
        out = (C.c_size_t * max(r, 1))()
        lib.ugh_op_ast_dims(api._p(self._h), out)
        return tuple(out[i] for i in range(r))


def load(arg, shape):
    d, r = dims(shape)
    return Ast(_new("ugh_op_load", api._p(arg._h), d, C.c_size_t(r)))


def i32(v):
    return Ast(_new("ugh_op_cst_i32", C.c_int32(int(v))))


def f32(v):
    return Ast(_new("ugh_op_cst_f32", C.c_float(float(v))))


class Store(_Owned):
    """lib.rs:226-238."""
    _free = "ugh_op_store_free"

    def __init__(self, dst, shape, value):
        d, r = dims(shape)
        super().__init__(_new("ugh_op_store", api._p(dst._h), d, C.c_size_t(r), api._p(value._h)))


class Kernel(_Owned):
    """lib.rs:240-265."""
    _free = "ugh_op_kernel_free"

    def __init__(self, name, args, ops):
        a = (C.c_void_p * max(len(args), 1))(*[x._h for x in args])
        s = (C.c_void_p * max(len(ops), 1))(*[x._h for x in ops])
        super().__init__(_new("ugh_op_kernel_new", name.encode(), a, C.c_size_t(len(args)), s, C.c_size_t(len(ops))))

    def __str__(self):
        return text("ugh_op_kernel_str", self._h)

    def lower(self):
        from . import ssa
        return ssa.Kernel._wrap(api.SsaKernel(_new("ugh_op_kernel_lower", api._p(self._h))))
