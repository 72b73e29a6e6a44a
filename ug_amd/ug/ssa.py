"""`ug.ssa` (ug-pyo3/src/lib.rs:267-402): the flat SSA kernel of ug-core/src/lang.rs:611-753."""
import ctypes as C

from .. import api
from ._util import call, text

_UNARY = {"neg": api.U_NEG, "exp": api.U_EXP}
_BINARY = {"add": api.B_ADD, "mul": api.B_MUL, "sub": api.B_SUB, "div": api.B_DIV}


def _var(i):
    a = api.A()
    a.is_const, a.var = 0, int(i)
    return a


def _const(dtype, i=0, f=0.0):
    a = api.A()
    a.is_const, a.dtype, a.i, a.f = 1, dtype, int(i), float(f)
    return a


def _code(dtype):
    return dtype._code


class Instr:
    """One ssa::Instr; operands are line numbers of earlier instructions (lib.rs:269-275)."""

    def __init__(self, raw):
        self._raw = raw

    def __str__(self):
        return str(Kernel._from_raw([self._raw], check=False)).split(" ", 1)[1].rstrip("\n")

    @staticmethod
    def _make(op, dtype=0, sub=0, v=0, n=0, a=None, b=None):
        r = api.Instr()
        r.op, r.dtype, r.sub, r.v, r.n = op, dtype, sub, int(v), int(n)
        if a is not None:
            r.a = a
        if b is not None:
            r.b = b
        return Instr(r)

    @staticmethod
    def const_i32(v):
        return Instr._make(api.I_CONST, api.I32, a=_const(api.I32, i=v))

    @staticmethod
    def const_f32(v):
        if v != v:
            raise ValueError("cannot use nan in const")
        return Instr._make(api.I_CONST, api.F32, a=_const(api.F32, f=v))

    @staticmethod
    def define_acc_i32(v):
        return Instr._make(api.I_DEFINE_ACC, api.I32, a=_const(api.I32, i=v))

    @staticmethod
    def define_acc_f32(v):
        if v != v:
            raise ValueError("cannot use nan in const")
        return Instr._make(api.I_DEFINE_ACC, api.F32, a=_const(api.F32, f=v))

    @staticmethod
    def end_range(start_idx):
        return Instr._make(api.I_END_RANGE, v=start_idx)

    @staticmethod
    def range(lo, up, end_idx):
        return Instr._make(api.I_RANGE, v=end_idx, n=1, a=_var(lo), b=_var(up))

    @staticmethod
    def load(src, offset, dtype):
        return Instr._make(api.I_LOAD, _code(dtype), v=src, a=_var(offset))

    @staticmethod
    def store(dst, offset, value, dtype):
        return Instr._make(api.I_STORE, _code(dtype), v=dst, a=_var(offset), b=_var(value))

    @staticmethod
    def define_global(index, dtype):
        return Instr._make(api.I_DEFINE_GLOBAL, _code(dtype), n=index)

    @staticmethod
    def special_ti():
        return Instr._make(api.I_SPECIAL, sub=api.SPECIAL_THREAD_IDX)

    @staticmethod
    def special_bi():
        return Instr._make(api.I_SPECIAL, sub=api.SPECIAL_BLOCK_IDX)

    @staticmethod
    def unary(op, arg, dtype):
        if op not in _UNARY:
            raise ValueError(f"unknown unary op '{op}'")
        return Instr._make(api.I_UNARY, _code(dtype), sub=_UNARY[op], a=_var(arg))

    @staticmethod
    def binary(op, lhs, rhs, dtype):
        if op not in _BINARY:
            raise ValueError(f"unknown binary op '{op}'")
        return Instr._make(api.I_BINARY, _code(dtype), sub=_BINARY[op], a=_var(lhs), b=_var(rhs))


class Kernel:
    """ssa::Kernel::from_instrs (lang.rs:739-753): arguments are the DefineGlobal lines, launch 1 x 1."""

    def __init__(self, instrs):
        self._k = call(lambda: api.SsaKernel.from_instrs([i._raw for i in instrs]))

    @classmethod
    def _wrap(cls, inner):
        self = cls.__new__(cls)
        self._k = inner
        return self

    @classmethod
    def _from_raw(cls, raws, check=True):
        return cls._wrap(api.SsaKernel.from_instrs(list(raws)))

    def __str__(self):
        return text("ugh_ssa_str", self._k.h)

    def flops_and_mem(self):
        fl, mem = C.c_size_t(), C.c_size_t()
        call(lambda: api._chk(api.host_lib().ugh_ssa_flops_mem(api._p(self._k.h), C.byref(fl), C.byref(mem))))
        return fl.value, mem.value

    def to_list(self):
        out = []
        for r in self._k.instrs():
            c = api.Instr()
            C.memmove(C.byref(c), C.byref(r), C.sizeof(api.Instr))
            out.append(Instr(c))
        return out

    def cuda_code(self, name):
        raise ValueError("this build generates HIP for gfx950: use hip_code(name)")

    def hip_code(self, name):
        """`cuda_code` (lib.rs:396-401) for HIP: `extern "C" __global__ void <name>(...)`, one pointer per
        kernel argument, translated statement by statement for the kernel's own launch configuration."""
        w = self._k.wire()
        lib = api.ughip_lib()
        n = C.c_size_t()
        if lib.ughip_codegen_as_written(C.byref(w), name.encode(), None, C.c_size_t(0), C.byref(n)):
            raise ValueError(lib.ughip_last_error().decode())
        buf = C.create_string_buffer(n.value + 1)
        lib.ughip_codegen_as_written(C.byref(w), name.encode(), buf, C.c_size_t(n.value + 1), None)
        return buf.value.decode()
