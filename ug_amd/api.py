"""ctypes bindings: the same names and argument meaning as ug's Rust API for this path
(`LazyBuffer` builders of ug-core/src/lazy_buffer.rs, `Schedule`, `Device`/`Slice`), so tests
read like the reference's own (ug-core/tests/lb_tests.rs, ug-core/src/common_tests.rs)."""
import contextlib
import ctypes as C
import os

import numpy as np

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")

BF16, F16, F32, I32, I64 = 0, 1, 2, 3, 4
_NP = {F32: np.float32, I32: np.int32, I64: np.int64, BF16: np.uint16, F16: np.float16}

UNARY = {"id": 0, "exp": 1, "sin": 2, "cos": 3, "neg": 4, "sqrt": 5}
BINARY = {"add": 0, "sub": 1, "mul": 2, "div": 3, "mod": 4, "min": 5, "max": 6}
REDUCE = {"sum": 0, "max": 1, "min": 2}
STRATEGY = {0: "literal", 1: "elementwise", 2: "row_block", 3: "row_thread", 4: "grid_reduce"}
# ssa::Instr discriminants and selectors on the wire (include/ughip.h, order of ug-core/src/lang.rs:690-709)
(I_DEFINE_ACC, I_DEFINE_GLOBAL, I_DEFINE_LOCAL, I_SPECIAL, I_CONST, I_UNARY, I_BINARY, I_RANGE, I_LOAD, I_ASSIGN, I_END_RANGE, I_IF, I_END_IF,
 I_STORE, I_BARRIER, I_REDUCE_LOCAL) = range(16)
SPECIAL_THREAD_IDX, SPECIAL_BLOCK_IDX = 0, 1
R_SUM, R_MAX, R_MIN = 0, 1, 2
U_ID, U_EXP, U_SIN, U_COS, U_NEG, U_SQRT, U_CAST = range(7)
B_ADD, B_SUB, B_MUL, B_DIV, B_MOD, B_MIN, B_MAX = range(7)


class UgError(RuntimeError):
    """ug::Error: every failure on the path carries a message."""


def np_dtype(dtype):
    return _NP[dtype]


def _load(name):
    path = os.path.join(_LIB_DIR, name)
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build the native libraries first (python -m ug_amd.build); "
                          "there is no CPU fallback for the HIP path")
    return C.CDLL(path, mode=C.RTLD_GLOBAL)


_ughip = None
_host = None


def ughip_lib():
    """libughip.so: the C ABI of include/ughip.h."""
    global _ughip
    if _ughip is None:
        lib = _load("libughip.so")
        lib.ughip_last_error.restype = C.c_char_p
        lib.ughip_last_kernel.restype = C.c_char_p
        lib.ughip_slice_len.restype = C.c_size_t
        lib.ughip_slice_ptr.restype = C.c_void_p
        lib.ughip_func_source.restype = C.c_size_t
        _ughip = lib
    return _ughip


class FuncInfo(C.Structure):
    _fields_ = [("strategy", C.c_int32), ("grid_dim", C.c_uint32), ("block_dim", C.c_uint32), ("lds_bytes", C.c_uint32),
                ("scratch_bytes", C.c_uint64)]


class A(C.Structure):
    _fields_ = [("is_const", C.c_uint8), ("dtype", C.c_uint8), ("pad_", C.c_uint16), ("var", C.c_uint32), ("i", C.c_int64), ("f", C.c_float),
                ("pad2_", C.c_uint32)]


class Instr(C.Structure):
    _fields_ = [("op", C.c_int32), ("dtype", C.c_int32), ("sub", C.c_int32), ("v", C.c_uint32), ("n", C.c_uint64), ("a", A), ("b", A)]


class KernelArg(C.Structure):
    _fields_ = [("arg_id", C.c_uint64), ("is_ptr", C.c_uint8), ("dtype", C.c_uint8), ("pad_", C.c_uint16), ("var", C.c_uint32)]


class SsaWire(C.Structure):
    _fields_ = [("instrs", C.POINTER(Instr)), ("n_instrs", C.c_size_t), ("args", C.POINTER(KernelArg)), ("n_args", C.c_size_t),
                ("grid_dim", C.c_uint32), ("block_dim", C.c_uint32), ("shared_mem", C.c_uint32), ("pad_", C.c_uint32)]


class LlamaConfig(C.Structure):
    """ug-llama/src/model.rs:10-24; defaults are the TinyLlama-1.1B shape."""
    _fields_ = [("hidden_size", C.c_size_t), ("intermediate_size", C.c_size_t), ("max_position_embeddings", C.c_size_t),
                ("num_attention_heads", C.c_size_t), ("num_key_value_heads", C.c_size_t), ("num_hidden_layers", C.c_size_t),
                ("rms_norm_eps", C.c_double), ("rope_interleaved", C.c_int), ("rope_theta", C.c_float), ("vocab_size", C.c_size_t)]

    def __init__(self, hidden_size=2048, intermediate_size=5632, max_position_embeddings=2048, num_attention_heads=32,
                 num_key_value_heads=4, num_hidden_layers=22, rms_norm_eps=1e-5, rope_interleaved=False, rope_theta=10000.0,
                 vocab_size=32000):
        super().__init__(hidden_size, intermediate_size, max_position_embeddings, num_attention_heads, num_key_value_heads,
                         num_hidden_layers, rms_norm_eps, int(rope_interleaved), rope_theta, vocab_size)

    @property
    def head_dim(self):
        return self.hidden_size // self.num_attention_heads


CUSTOM_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_void_p), C.c_size_t)


def host_lib():
    """libug_host.so: lazy-buffer front-end + HipDevice (flat C API of csrc/host/capi.cpp)."""
    global _host
    if _host is None:
        ughip_lib()
        lib = _load("libug_host.so")
        lib.ugh_last_error.restype = C.c_char_p
        lib.ugh_device_name.restype = C.c_char_p
        for f in ("ugh_slice_len", "ugh_lb_rank", "ugh_lb_elem_count", "ugh_schedule_n_items", "ugh_schedule_item_n_args",
                  "ugh_compiled_n_funcs", "ugh_cache_size"):
            getattr(lib, f).restype = C.c_size_t
        for f in ("ugh_cache_new", "ugh_device_raw_hip", "ugh_func_raw_hip", "ugh_compiled_func_raw_hip", "ugh_slice_raw_hip"):
            getattr(lib, f).restype = C.c_void_p
        for f in ("ugh_device_free", "ugh_slice_free", "ugh_func_free", "ugh_ssa_free", "ugh_lb_free", "ugh_schedule_free", "ugh_cache_free",
                  "ugh_compiled_free", "ugh_llama_ops_free", "ugh_llama_model_free", "ugh_lb_dims", "ugh_ssa_set_launch"):
            getattr(lib, f).restype = None
        _host = lib
    return _host


def _chk(rc):
    if rc:
        raise UgError(host_lib().ugh_last_error().decode(errors="replace"))


def _p(h):
    return C.c_void_p(h)


def _dims(shape):
    if isinstance(shape, int):
        shape = (shape,)
    shape = tuple(int(s) for s in shape)
    return (C.c_size_t * max(1, len(shape)))(*shape), len(shape)


class _Handle:
    _free = None

    def __init__(self, h):
        self.h = h

    def __del__(self):
        h, self.h = getattr(self, "h", None), None
        if h and self._free and _host is not None:
            getattr(_host, self._free)(_p(h))


class Slice(_Handle):
    """trait Slice (ug-core/src/lib.rs:29-47)."""
    _free = "ugh_slice_free"

    def __len__(self):
        return host_lib().ugh_slice_len(_p(self.h))

    @property
    def dtype(self):
        return host_lib().ugh_slice_dtype(_p(self.h))

    def raw(self):
        """The ughip_slice* of a HIP slice, for direct calls into libughip.so (0 on other devices)."""
        return host_lib().ugh_slice_raw_hip(_p(self.h)) or 0

    def copy_host_to_device(self, src, dtype=None):
        src = np.ascontiguousarray(src)
        dtype = _np_to_dtype(src.dtype) if dtype is None else dtype
        _chk(host_lib().ugh_slice_h2d(_p(self.h), src.ctypes.data_as(C.c_void_p), dtype, C.c_size_t(src.size)))

    def to_vec(self, dtype=None):
        dtype = self.dtype if dtype is None else dtype
        out = np.empty(len(self), dtype=_NP[dtype])
        _chk(host_lib().ugh_slice_d2h(_p(self.h), out.ctypes.data_as(C.c_void_p), dtype, C.c_size_t(out.size)))
        return out


def _np_to_dtype(dt):
    dt = np.dtype(dt)
    for k, v in _NP.items():
        if np.dtype(v) == dt and k != F16:
            return k
    if dt == np.float16:
        return F16
    raise UgError(f"unsupported numpy dtype {dt}")


class Func(_Handle):
    _free = "ugh_func_free"

    def _raw(self):
        return host_lib().ugh_func_raw_hip(_p(self.h))

    def source(self):
        return _func_source(self._raw())

    def info(self):
        return _func_info(self._raw())


def _func_source(raw):
    if not raw:
        return None
    lib = ughip_lib()
    n = lib.ughip_func_source(C.c_void_p(raw), None, C.c_size_t(0))
    buf = C.create_string_buffer(n + 1)
    lib.ughip_func_source(C.c_void_p(raw), buf, C.c_size_t(n + 1))
    return buf.value.decode()


def _func_info(raw):
    if not raw:
        return None
    info = FuncInfo()
    if ughip_lib().ughip_func_get_info(C.c_void_p(raw), C.byref(info)):
        raise UgError(ughip_lib().ughip_last_error().decode())
    return {"strategy": STRATEGY[info.strategy], "grid_dim": info.grid_dim, "block_dim": info.block_dim, "lds_bytes": info.lds_bytes,
            "scratch_bytes": info.scratch_bytes}


class SsaKernel(_Handle):
    """ssa::Kernel (ug-core/src/lang.rs:711-753)."""
    _free = "ugh_ssa_free"

    @staticmethod
    def sample(name, p0=0, p1=0, p2=0):
        """ug::samples::ssa::* (ug-core/src/samples.rs:10-232)."""
        out = C.c_void_p()
        _chk(host_lib().ugh_sample_ssa(name.encode(), C.c_size_t(p0), C.c_size_t(p1), C.c_size_t(p2), C.byref(out)))
        return SsaKernel(out.value)

    @staticmethod
    def sample_op(name, p0=0, p1=0, block_axis=-1, thread_dim=-1, thread_block_dim=0):
        """ug::samples::op::softmax(..).lower(&opts) and the `affine` kernel of basic_tests.rs:118-136."""
        out = C.c_void_p()
        _chk(host_lib().ugh_sample_op_ssa(name.encode(), C.c_size_t(p0), C.c_size_t(p1), C.c_long(block_axis), C.c_long(thread_dim),
                                          C.c_size_t(thread_block_dim), C.byref(out)))
        return SsaKernel(out.value)

    @staticmethod
    def from_instrs(instrs, grid=1, block=1, shared=0):
        arr = (Instr * len(instrs))(*instrs)
        out = C.c_void_p()
        _chk(host_lib().ugh_ssa_from_raw(arr, C.c_size_t(len(instrs)), C.c_uint32(grid), C.c_uint32(block), C.c_uint32(shared), C.byref(out)))
        return SsaKernel(out.value)

    def set_launch(self, grid, block, shared=0):
        host_lib().ugh_ssa_set_launch(_p(self.h), C.c_uint32(grid), C.c_uint32(block), C.c_uint32(shared))

    def wire(self):
        w = SsaWire()
        _chk(host_lib().ugh_ssa_wire(_p(self.h), C.byref(w)))
        return w

    def instrs(self):
        w = self.wire()
        return [w.instrs[i] for i in range(w.n_instrs)]

    def min_lens(self):
        """Per kernel argument, the slice length ughip_run asks for (-1: not bounded statically); needs no device."""
        w = self.wire()
        out = (C.c_int64 * w.n_args)()
        lib = ughip_lib()
        if lib.ughip_codegen_min_len(C.byref(w), out, C.c_size_t(w.n_args)):
            raise UgError(lib.ughip_last_error().decode())
        return list(out)

    def hip_code(self, name=None):
        """Counterpart of `Kernel.cuda_code()` (ug-pyo3/src/lib.rs:396-401); needs no device."""
        w = self.wire()
        n = C.c_size_t()
        info = FuncInfo()
        lib = ughip_lib()
        nm = name.encode() if name else None
        if lib.ughip_codegen(C.byref(w), nm, None, C.c_size_t(0), C.byref(n), C.byref(info)):
            raise UgError(lib.ughip_last_error().decode())
        buf = C.create_string_buffer(n.value + 1)
        lib.ughip_codegen(C.byref(w), nm, buf, C.c_size_t(n.value + 1), None, None)
        return buf.value.decode(), {"strategy": STRATEGY[info.strategy], "grid_dim": info.grid_dim, "block_dim": info.block_dim,
                                    "scratch_bytes": info.scratch_bytes}


class Device(_Handle):
    """trait Device (ug-core/src/lib.rs:49-73)."""
    _free = "ugh_device_free"

    @property
    def name(self):
        return host_lib().ugh_device_name(_p(self.h)).decode()

    def use_grid(self):
        return bool(host_lib().ugh_device_use_grid(_p(self.h)))

    def synchronize(self):
        _chk(host_lib().ugh_device_synchronize(_p(self.h)))

    def allocate_uninit(self, dtype, length):
        out = C.c_void_p()
        _chk(host_lib().ugh_device_alloc(_p(self.h), dtype, C.c_size_t(length), C.byref(out)))
        return Slice(out.value)

    def slice_from(self, arr):
        arr = np.ascontiguousarray(arr)
        s = self.allocate_uninit(_np_to_dtype(arr.dtype), arr.size)
        s.copy_host_to_device(arr)
        return s

    def compile(self, kernel, name=None):
        out = C.c_void_p()
        _chk(host_lib().ugh_device_compile(_p(self.h), _p(kernel.h), name.encode() if name else None, C.byref(out)))
        return Func(out.value)

    def run(self, func, slices):
        arr = (C.c_void_p * max(1, len(slices)))(*[s.h for s in slices])
        _chk(host_lib().ugh_device_run(_p(self.h), _p(func.h), arr, C.c_size_t(len(slices))))

    def matmul(self, dst, lhs, rhs, bmnk, lhs_l, rhs_l):
        """lhs_l / rhs_l: (dims, strides, offset) as in ug::Layout."""
        b, m, n, k = bmnk
        rank = len(lhs_l[0])
        sz = C.c_size_t * rank
        _chk(host_lib().ugh_device_matmul(_p(self.h), _p(dst.h), _p(lhs.h), _p(rhs.h), C.c_size_t(b), C.c_size_t(m), C.c_size_t(n),
                                          C.c_size_t(k), C.c_size_t(rank), sz(*lhs_l[0]), sz(*lhs_l[1]), C.c_size_t(lhs_l[2]),
                                          sz(*rhs_l[0]), sz(*rhs_l[1]), C.c_size_t(rhs_l[2])))

    def convert(self, dst, src):
        """Element type conversion between two slices in device memory; False if the device has none."""
        done = C.c_int()
        _chk(host_lib().ugh_device_convert(_p(self.h), _p(dst.h), _p(src.h), C.byref(done)))
        return bool(done.value)

    def set_zero_fill(self, on):
        """HIP device only: zero-fill fresh allocations (default, like ug's CpuDevice) or not (like ug-cuda)."""
        _chk(host_lib().ugh_hip_device_set_zero_fill(_p(self.h), int(on)))

    def raw_hip(self):
        return host_lib().ugh_device_raw_hip(_p(self.h))


def last_kernel():
    """The hand-written kernel this thread's last Device.matmul launched (ughip_last_kernel)."""
    return ughip_lib().ughip_last_kernel().decode()


def set_tuning(name, value=None):
    """One tuning switch of the backend (ughip_set_tuning): value None clears it.  The table is read from the environment
    (UGHIP_<NAME>) once per process; later changes of the environment are not seen, this call is."""
    lib = ughip_lib()
    if lib.ughip_set_tuning(name.encode(), 0 if value is None else 1, C.c_int64(0 if value is None else int(value))):
        raise UgError(lib.ughip_last_error().decode())


@contextlib.contextmanager
def tuning(**switches):
    """with tuning(GEMM_SHAPE=0, GEMM_SPLIT=4): ...  -- sets the switches, clears them again on the way out."""
    for k, v in switches.items():
        set_tuning(k, v)
    try:
        yield
    finally:
        for k in switches:
            set_tuning(k, None)


def set_llama_switch(name, on=True):
    """A switch of the host-side llama loops and hooks (NO_FOLD_EPILOGUES, NO_APPEND_PAIR, VERBOSE, NO_LAYER_STEPS,
    HOST_ARGMAX, NO_OVERLAP); like the backend's table, read from the environment (UG_LLAMA_<NAME>) once per process."""
    _chk(host_lib().ugh_llama_set_switch(name.encode(), int(bool(on))))


@contextlib.contextmanager
def llama_switches(*names):
    for n in names:
        set_llama_switch(n, True)
    try:
        yield
    finally:
        for n in names:
            set_llama_switch(n, False)


def hip_device(ordinal=0):
    """ug_hip::Device::new(ordinal).  Raises when no GPU is present."""
    out = C.c_void_p()
    _chk(host_lib().ugh_hip_device_new(ordinal, C.byref(out)))
    return Device(out.value)


class LazyBuffer(_Handle):
    """ug::LazyBuffer (ug-core/src/lazy_buffer.rs)."""
    _free = "ugh_lb_free"

    def __init__(self, h, device):
        super().__init__(h)
        self.device = device
        self._keep = []

    def _new(self, fn, *args):
        out = C.c_void_p()
        _chk(getattr(host_lib(), fn)(*args, C.byref(out)))
        lb = LazyBuffer(out.value, self.device)
        lb._keep = [self]
        return lb

    # -- constructors
    @staticmethod
    def cst(value, shape, device, dtype=F32):
        d, r = _dims(shape)
        out = C.c_void_p()
        _chk(host_lib().ugh_lb_cst(_p(device.h), dtype, C.c_double(value), d, C.c_size_t(r), C.byref(out)))
        return LazyBuffer(out.value, device)

    @staticmethod
    def copy(data, shape, device):
        data = np.ascontiguousarray(data)
        d, r = _dims(shape)
        out = C.c_void_p()
        _chk(host_lib().ugh_lb_copy(_p(device.h), _np_to_dtype(data.dtype), data.ctypes.data_as(C.c_void_p), C.c_size_t(data.size), d,
                                    C.c_size_t(r), C.byref(out)))
        return LazyBuffer(out.value, device)

    @staticmethod
    def alloc_uninit(dtype, shape, device):
        d, r = _dims(shape)
        out = C.c_void_p()
        _chk(host_lib().ugh_lb_alloc_uninit(_p(device.h), dtype, d, C.c_size_t(r), C.byref(out)))
        return LazyBuffer(out.value, device)

    @staticmethod
    def custom(f, args, shape, dtype, device):
        """f(list_of_Slice) with inputs first and the destination last (lazy_buffer.rs:292-310)."""
        cb = _wrap_custom(f)
        arr = (C.c_void_p * max(1, len(args)))(*[a.h for a in args])
        d, r = _dims(shape)
        out = C.c_void_p()
        _chk(host_lib().ugh_lb_custom(_p(device.h), cb, None, arr, C.c_size_t(len(args)), d, C.c_size_t(r), dtype, C.byref(out)))
        lb = LazyBuffer(out.value, device)
        lb._keep = [cb] + list(args)
        return lb

    def custom_ip(self, f, args=()):
        cb = _wrap_custom(f)
        arr = (C.c_void_p * max(1, len(args)))(*[a.h for a in args])
        lb = self._new("ugh_lb_custom_ip", _p(self.h), cb, None, arr, C.c_size_t(len(args)))
        lb._keep += [cb] + list(args)
        return lb

    @staticmethod
    def ssa(kernel, args, shape, dtype, device):
        arr = (C.c_void_p * max(1, len(args)))(*[a.h for a in args])
        d, r = _dims(shape)
        out = C.c_void_p()
        _chk(host_lib().ugh_lb_ssa(_p(device.h), _p(kernel.h), arr, C.c_size_t(len(args)), d, C.c_size_t(r), dtype, C.byref(out)))
        lb = LazyBuffer(out.value, device)
        lb._keep = list(args)
        return lb

    @staticmethod
    def cat(args, dim):
        arr = (C.c_void_p * len(args))(*[a.h for a in args])
        out = C.c_void_p()
        _chk(host_lib().ugh_lb_cat(arr, C.c_size_t(len(args)), C.c_long(dim), C.byref(out)))
        lb = LazyBuffer(out.value, args[0].device)
        lb._keep = list(args)
        return lb

    # -- ops
    def unary(self, op):
        return self._new("ugh_lb_unary", _p(self.h), UNARY[op])

    def cast(self, dtype):
        return self._new("ugh_lb_cast", _p(self.h), dtype)

    def binary(self, op, rhs):
        lb = self._new("ugh_lb_binary", _p(self.h), BINARY[op], _p(rhs.h))
        lb._keep.append(rhs)
        return lb

    def reduce(self, op, dim):
        return self._new("ugh_lb_reduce", _p(self.h), REDUCE[op], C.c_long(dim))

    def matmul(self, rhs):
        lb = self._new("ugh_lb_matmul", _p(self.h), _p(rhs.h), 0)
        lb._keep.append(rhs)
        return lb

    def matmul_t(self, rhs):
        lb = self._new("ugh_lb_matmul", _p(self.h), _p(rhs.h), 1)
        lb._keep.append(rhs)
        return lb

    def split_dim(self, dim, s1, s2):
        return self._new("ugh_lb_split_dim", _p(self.h), C.c_long(dim), C.c_size_t(s1), C.c_size_t(s2))

    def merge_dims(self, dim):
        return self._new("ugh_lb_merge_dims", _p(self.h), C.c_long(dim))

    def squeeze(self, dim):
        return self._new("ugh_lb_squeeze", _p(self.h), C.c_long(dim))

    def unsqueeze(self, dim):
        return self._new("ugh_lb_unsqueeze", _p(self.h), C.c_long(dim))

    def get_on_dim(self, dim, index):
        return self._new("ugh_lb_get_on_dim", _p(self.h), C.c_long(dim), C.c_size_t(index))

    def get(self, index):
        return self.get_on_dim(0, index)

    def reshape(self, shape):
        d, r = _dims(shape)
        return self._new("ugh_lb_reshape", _p(self.h), d, C.c_size_t(r))

    def narrow(self, dim, offset, length):
        return self._new("ugh_lb_narrow", _p(self.h), C.c_long(dim), C.c_size_t(offset), C.c_size_t(length))

    def broadcast(self, shape):
        d, r = _dims(shape)
        return self._new("ugh_lb_broadcast", _p(self.h), d, C.c_size_t(r))

    def transpose(self, d1, d2):
        return self._new("ugh_lb_transpose", _p(self.h), C.c_long(d1), C.c_long(d2))

    def set(self, values):
        lb = self._new("ugh_lb_set", _p(self.h), _p(values.h))
        lb._keep.append(values)
        return lb

    def set_l(self, values, dims, strides=None, offset=0):
        """dst_layout as (dims, strides, offset); strides default to contiguous (Layout::from_shape)."""
        dims = (dims,) if isinstance(dims, int) else tuple(dims)
        if strides is None:
            strides, st = [], 1
            for d in reversed(dims):
                strides.insert(0, st)
                st *= d
        sz = C.c_size_t * max(1, len(dims))
        lb = self._new("ugh_lb_set_l", _p(self.h), _p(values.h), sz(*dims), sz(*strides), C.c_size_t(len(dims)), C.c_size_t(offset))
        lb._keep.append(values)
        return lb

    # -- access
    def dims(self):
        r = host_lib().ugh_lb_rank(_p(self.h))
        out = (C.c_size_t * max(1, r))()
        host_lib().ugh_lb_dims(_p(self.h), out)
        return list(out[:r])

    @property
    def dtype(self):
        return host_lib().ugh_lb_dtype(_p(self.h))

    def elem_count(self):
        return host_lib().ugh_lb_elem_count(_p(self.h))

    def realized(self):
        return bool(host_lib().ugh_lb_realized(_p(self.h)))

    def realize(self):
        _chk(host_lib().ugh_lb_realize(_p(self.h)))

    def data_vec(self, dtype=None):
        dtype = self.dtype if dtype is None else dtype
        out = np.empty(self.elem_count(), dtype=_NP[dtype])
        _chk(host_lib().ugh_lb_data_vec(_p(self.h), dtype, out.ctypes.data_as(C.c_void_p), C.c_size_t(out.size)))
        return out

    def write(self, data):
        """Overwrite the realised storage (what lb_tests.rs:82-94 does through `lb.data()`)."""
        data = np.ascontiguousarray(data)
        _chk(host_lib().ugh_lb_write(_p(self.h), data.ctypes.data_as(C.c_void_p), _np_to_dtype(data.dtype), C.c_size_t(data.size)))


class _BorrowedSlice(Slice):
    _free = None


def _wrap_custom(f):
    def cb(_user, slices, n):
        try:
            f([_BorrowedSlice(slices[i]) for i in range(n)])
            return 0
        except Exception:  # surfaced as "custom op callback failed"
            import traceback
            traceback.print_exc()
            return 1
    return CUSTOM_FN(cb)


class CompilationCache(_Handle):
    """ug::cache::CompilationCache (ug-core/src/cache.rs:74-101)."""
    _free = "ugh_cache_free"

    def __init__(self):
        super().__init__(host_lib().ugh_cache_new())

    def __len__(self):
        return host_lib().ugh_cache_size(_p(self.h))


class CompiledSchedule(_Handle):
    _free = "ugh_compiled_free"
    KINDS = {0: "kernel", 1: "matmul", 2: "custom"}

    def run(self):
        _chk(host_lib().ugh_compiled_run(_p(self.h)))

    def funcs(self):
        lib = host_lib()
        out = []
        for i in range(lib.ugh_compiled_n_funcs(_p(self.h))):
            kind = self.KINDS[lib.ugh_compiled_func_kind(_p(self.h), C.c_size_t(i))]
            raw = lib.ugh_compiled_func_raw_hip(_p(self.h), C.c_size_t(i))
            out.append({"kind": kind, "info": _func_info(raw), "source": _func_source(raw)})
        return out


class Schedule(_Handle):
    """ug::Schedule (ug-core/src/schedule.rs:61-208)."""
    _free = "ugh_schedule_free"
    KINDS = {0: "kernel", 1: "matmul", 2: "custom", 3: "ssa"}

    @staticmethod
    def create(buffers):
        arr = (C.c_void_p * len(buffers))(*[b.h for b in buffers])
        out = C.c_void_p()
        _chk(host_lib().ugh_schedule_create(arr, C.c_size_t(len(buffers)), C.byref(out)))
        s = Schedule(out.value)
        s._keep = list(buffers)
        return s

    @staticmethod
    def create_one(buffer):
        return Schedule.create([buffer])

    def items(self):
        lib = host_lib()
        out = []
        for i in range(lib.ugh_schedule_n_items(_p(self.h))):
            kind = self.KINDS[lib.ugh_schedule_item_kind(_p(self.h), C.c_size_t(i))]
            item = {"kind": kind, "n_args": lib.ugh_schedule_item_n_args(_p(self.h), C.c_size_t(i))}
            if kind == "kernel":
                buf = C.create_string_buffer(64)
                _chk(lib.ugh_schedule_item_name(_p(self.h), C.c_size_t(i), buf, C.c_size_t(64)))
                item["name"] = buf.value.decode()
            out.append(item)
        return out

    def item_ssa(self, i, optimize=True):
        """`item.kernel()?.optimize()?.lower(&Opts::default())` (schedule.rs:145-189, serial nest)."""
        out = C.c_void_p()
        _chk(host_lib().ugh_schedule_item_ssa(_p(self.h), C.c_size_t(i), int(optimize), C.byref(out)))
        return SsaKernel(out.value)

    def compile(self, cache=None):
        out = C.c_void_p()
        _chk(host_lib().ugh_schedule_compile(_p(self.h), _p(cache.h) if cache is not None else None, C.byref(out)))
        cs = CompiledSchedule(out.value)
        cs._keep = [self, cache]
        return cs


class LlamaOps(_Handle):
    """`trait Device` of ug-llama/src/main.rs:22-28."""
    _free = "ugh_llama_ops_free"

    @staticmethod
    def hip(bf16x3=False):
        """bf16x3: two or more f32 rows against a BF16 matrix are split into three bf16 terms each and multiplied on the
        bf16 matrix pipe (UGHIP_PRODUCT_BF16X3) instead of widening the matrix for the f32 pipe."""
        out = C.c_void_p()
        _chk(host_lib().ugh_llama_ops_hip_ex(1 if bf16x3 else 0, C.byref(out)))
        return LlamaOps(out.value)

    def _op(self, fn, first, *rest):
        out = C.c_void_p()
        _chk(getattr(host_lib(), fn)(_p(self.h), _p(first.h), *rest, C.byref(out)))
        lb = LazyBuffer(out.value, first.device)
        lb._keep = [first, self] + [r for r in rest if isinstance(r, LazyBuffer)]
        return lb

    def rope(self, src, cos, sin, pos):
        lb = self._op("ugh_llama_rope", src, _p(cos.h), _p(sin.h), _p(pos.h), 0)
        lb._keep += [cos, sin, pos]
        return lb

    def rope_i(self, src, cos, sin, pos):
        lb = self._op("ugh_llama_rope", src, _p(cos.h), _p(sin.h), _p(pos.h), 1)
        lb._keep += [cos, sin, pos]
        return lb

    def cat(self, lhs, rhs, axis):
        lb = self._op("ugh_llama_cat", lhs, _p(rhs.h), C.c_size_t(axis))
        lb._keep.append(rhs)
        return lb

    def custom_softmax(self, src):
        return self._op("ugh_llama_custom_softmax", src)

    def causal_mask(self, src):
        return self._op("ugh_llama_causal_mask", src)

    def causal_softmax(self, src):
        """softmax(causal_mask(src)); one kernel on the HIP device, op by op elsewhere."""
        return self._op("ugh_llama_causal_softmax", src)

    def attention_decode(self, q, k, v, scale):
        """One query position: q [b, nh, 1, d], k and v [b, nkv, s, d] -> [b, nh, 1, d]."""
        lb = self._op("ugh_llama_attention_decode", q, _p(k.h), _p(v.h), C.c_float(scale))
        lb._keep += [k, v]
        return lb


    def rope_append(self, cache, x, cos=None, sin=None, pos=None, interleaved=False):
        """cache [b, n, s, d] grown by the row(s) of x [b, 1, n * d], rotated when a table is given."""
        rope = cos is not None
        lb = self._op("ugh_llama_rope_append", cache, _p(x.h), _p(cos.h) if rope else None, _p(sin.h) if rope else None,
                      _p(pos.h) if rope else None, int(interleaved))
        lb._keep += [x] + ([cos, sin, pos] if rope else [])
        return lb

    def attention_decode_flat(self, q, k, v, scale, cos=None, sin=None, pos=None, interleaved=False):
        """q [b, 1, nh * d] (rotated first when a table is given), k and v [b, nkv, s, d] -> [b, 1, nh * d]."""
        rope = cos is not None
        lb = self._op("ugh_llama_attention_decode_flat", q, _p(k.h), _p(v.h), C.c_float(scale), _p(cos.h) if rope else None,
                      _p(sin.h) if rope else None, _p(pos.h) if rope else None, int(interleaved))
        lb._keep += [k, v] + ([cos, sin, pos] if rope else [])
        return lb

    def kv_cache_capacity(self, max_positions, head_dim=64):
        """Rows this device preallocates per cache head (0: caches grow by concatenation)."""
        out = C.c_size_t()
        _chk(host_lib().ugh_llama_kv_cache_capacity(_p(self.h), C.c_size_t(max_positions), C.c_size_t(head_dim), C.byref(out)))
        return out.value

    def kv_append(self, cache, length, x, cos=None, sin=None, pos=None, interleaved=False, x_offset=0, x_row_stride=0):
        """cache [b, n, cap, d] holding `length` rows receives x [b, t, n * d] as rows length .. length + t - 1
        (rotated when a table is given): in place when cap > length, by concatenation when cap == length.
        x_offset / x_row_stride: x as a column range of wider rows (a packed q|k|v projection)."""
        rope = cos is not None
        lb = self._op("ugh_llama_kv_append", cache, C.c_size_t(length), _p(x.h), _p(cos.h) if rope else None, _p(sin.h) if rope else None,
                      _p(pos.h) if rope else None, int(interleaved), C.c_size_t(x_offset), C.c_size_t(x_row_stride))
        lb._keep += [x] + ([cos, sin, pos] if rope else [])
        return lb

    def attention_cached(self, q, k, v, s, scale, cos=None, sin=None, pos=None, interleaved=False, q_offset=0, q_row_stride=0, n_heads=0):
        """Causal attention of q [b, t, nh * d] over the first s rows of k, v [b, nkv, cap, d] -> [b, t, nh * d].
        q_offset / q_row_stride / n_heads: q as a column range of wider rows (a packed q|k|v projection)."""
        rope = cos is not None
        lb = self._op("ugh_llama_attention_cached", q, _p(k.h), _p(v.h), C.c_size_t(s), C.c_float(scale), _p(cos.h) if rope else None,
                      _p(sin.h) if rope else None, _p(pos.h) if rope else None, int(interleaved), C.c_size_t(q_offset), C.c_size_t(q_row_stride), C.c_size_t(n_heads))
        lb._keep += [k, v] + ([cos, sin, pos] if rope else [])
        return lb

    def attention_step(self, qkv, kcache, vcache, length, n_heads, scale, cos=None, sin=None, pos=None, interleaved=False):
        """One decode position: the k | v parts of the packed row go into row `length` of the caches (which are
        written), the q part attends to rows 0 .. length -> [b, 1, n_heads * d]."""
        rope = cos is not None
        lb = self._op("ugh_llama_attention_step", qkv, _p(kcache.h), _p(vcache.h), C.c_size_t(length), C.c_size_t(n_heads), C.c_float(scale),
                      _p(cos.h) if rope else None, _p(sin.h) if rope else None, _p(pos.h) if rope else None, int(interleaved))
        lb._keep += [kcache, vcache] + ([cos, sin, pos] if rope else [])
        return lb


    def attention_steps(self, qkv, kcache, vcache, length, n_heads, scale, cos=None, sin=None, pos=None, interleaved=False):
        """t positions: the k | v parts of the packed rows go into rows length .. length + t - 1 of the caches (which
        are written), query i attends to rows 0 .. length + i -> [b, t, n_heads * d]."""
        rope = cos is not None
        lb = self._op("ugh_llama_attention_steps", qkv, _p(kcache.h), _p(vcache.h), C.c_size_t(length), C.c_size_t(n_heads), C.c_float(scale),
                      _p(cos.h) if rope else None, _p(sin.h) if rope else None, _p(pos.h) if rope else None, int(interleaved))
        lb._keep += [kcache, vcache] + ([cos, sin, pos] if rope else [])
        return lb

    def attention_steps_add(self, qkv, kcache, vcache, length, n_heads, scale, w_o, residual, cos=None, sin=None, pos=None, interleaved=False):
        """attention_steps followed by the output projection and its residual -> [b, t, n]."""
        rope = cos is not None
        lb = self._op("ugh_llama_attention_steps_add", qkv, _p(kcache.h), _p(vcache.h), C.c_size_t(length), C.c_size_t(n_heads), C.c_float(scale),
                      _p(cos.h) if rope else None, _p(sin.h) if rope else None, _p(pos.h) if rope else None, int(interleaved), _p(w_o.h), _p(residual.h))
        lb._keep += [kcache, vcache, w_o, residual] + ([cos, sin, pos] if rope else [])
        return lb

    def linear_norm(self, x, alpha, eps, w):
        """rms_norm(x, alpha, eps) w^T."""
        lb = self._op("ugh_llama_linear_norm", x, _p(alpha.h), C.c_float(eps), _p(w.h))
        lb._keep += [alpha, w]
        return lb

    def mlp_stacked(self, x, w_gate_up, w_down, residual, alpha=None, eps=0.0):
        """(silu(y gate^T) * (y up^T)) w_down^T + residual with y = x, or rms_norm(x, alpha, eps) when alpha is given."""
        lb = self._op("ugh_llama_mlp_stacked", x, _p(alpha.h) if alpha is not None else None, C.c_float(eps), _p(w_gate_up.h), _p(w_down.h), _p(residual.h))
        lb._keep += [w_gate_up, w_down, residual] + ([alpha] if alpha is not None else [])
        return lb

    def device_argmax(self):
        return bool(host_lib().ugh_llama_device_argmax(_p(self.h)))

    def argmax_into(self, token, logits, row, ids, vals, slot):
        """Index of the largest value of row `row` of logits -> token (in place), ids[slot]; the two largest values -> vals[2 slot ..]."""
        lb = self._op("ugh_llama_argmax_into", token, _p(logits.h), C.c_size_t(row), _p(ids.h), _p(vals.h), C.c_size_t(slot))
        lb._keep += [logits, ids, vals]
        return lb

    def packed_projections(self):
        return bool(host_lib().ugh_llama_packed_projections(_p(self.h)))

    def linear_packed(self, x, ws, alpha=None, eps=0.0):
        """x [b, t, k] against up to three [n_i, k] matrices -> [b, t, sum n_i], results side by side;
        on rms_norm(x, alpha, eps) when alpha is given."""
        arr = (C.c_void_p * len(ws))(*[w.h for w in ws])
        lb = self._op("ugh_llama_linear_packed", x, C.c_size_t(len(ws)), arr, _p(alpha.h) if alpha is not None else None, C.c_float(eps))
        lb._keep += list(ws) + ([alpha] if alpha is not None else [])
        return lb

    def gate_up(self, x, w_gate, w_up, alpha=None, eps=0.0):
        """silu(x gate^T) * (x up^T); on rms_norm(x, alpha, eps) when alpha is given."""
        lb = self._op("ugh_llama_gate_up", x, _p(w_gate.h), _p(w_up.h), _p(alpha.h) if alpha is not None else None, C.c_float(eps))
        lb._keep += [w_gate, w_up] + ([alpha] if alpha is not None else [])
        return lb

    def gate_up_stacked(self, x, w_gate_up):
        """silu(x gate^T) * (x up^T) against one [2n, k] matrix holding the gate rows, then the up rows."""
        lb = self._op("ugh_llama_gate_up_stacked", x, _p(w_gate_up.h))
        lb._keep += [w_gate_up]
        return lb

    def linear(self, x, w):
        """x w^T for a matrix that may be stored as bf16 under f32 rows."""
        lb = self._op("ugh_llama_linear", x, _p(w.h))
        lb._keep += [w]
        return lb

    def linear_add(self, x, w, residual):
        """x w^T + residual"""
        lb = self._op("ugh_llama_linear_add", x, _p(w.h), _p(residual.h))
        lb._keep += [w, residual]
        return lb


class _Llama:
    """Graph builders of ug-llama/src/model.rs:32-109."""

    @staticmethod
    def _un(fn, src, *rest, keep=()):
        out = C.c_void_p()
        _chk(getattr(host_lib(), fn)(_p(src.h), *rest, C.byref(out)))
        lb = LazyBuffer(out.value, src.device)
        lb._keep = [src] + list(keep)
        return lb

    def rms_norm(self, src, alpha, eps):
        return self._un("ugh_llama_rms_norm", src, _p(alpha.h), C.c_float(eps), keep=[alpha])

    def softmax(self, src):
        return self._un("ugh_llama_softmax", src)

    def silu(self, src):
        return self._un("ugh_llama_silu", src)

    def repeat(self, src, axis, n_rep):
        return self._un("ugh_llama_repeat", src, C.c_size_t(axis), C.c_size_t(n_rep))

    def index_select(self, src, ids):
        return self._un("ugh_llama_index_select", src, _p(ids.h), keep=[ids])

    def rope_tables(self, device, cfg):
        cos, sin = C.c_void_p(), C.c_void_p()
        _chk(host_lib().ugh_llama_rope_tables(_p(device.h), C.byref(cfg), C.byref(cos), C.byref(sin)))
        return LazyBuffer(cos.value, device), LazyBuffer(sin.value, device)


llama = _Llama()


class Safetensors(_Handle):
    """Memory-mapped safetensors file(s): ug-core/src/safetensors.rs (MmapedSafetensors)."""
    _free = "ugh_safetensors_free"

    def __init__(self, paths):
        if isinstance(paths, (str, bytes, os.PathLike)):
            paths = [paths]
        arr = (C.c_char_p * len(paths))(*[os.fsencode(p) for p in paths])
        out = C.c_void_p()
        _chk(host_lib().ugh_safetensors_open(arr, C.c_size_t(len(paths)), C.byref(out)))
        super().__init__(out.value)
        self.last_cast_on_device = False

    def tensors(self):
        """[(name, dtype string, shape, nbytes)] in file order."""
        lib = host_lib()
        lib.ugh_safetensors_count.restype = C.c_size_t
        out = []
        for i in range(lib.ugh_safetensors_count(_p(self.h))):
            name, dt = C.create_string_buffer(1024), C.create_string_buffer(32)
            rank, nbytes, dims = C.c_size_t(), C.c_size_t(), (C.c_size_t * 8)()
            _chk(lib.ugh_safetensors_entry(_p(self.h), C.c_size_t(i), name, C.c_size_t(1024), dt, C.c_size_t(32), C.byref(rank), dims, C.byref(nbytes)))
            out.append((name.value.decode(), dt.value.decode(), tuple(dims[: rank.value]), nbytes.value))
        return out

    def load(self, name, device, dtype=None):
        """`load` (stored dtype) or, with dtype, `load_with_cast`."""
        out, on_dev = C.c_void_p(), C.c_int()
        _chk(host_lib().ugh_safetensors_load(_p(self.h), name.encode(), _p(device.h), -1 if dtype is None else int(dtype), C.byref(out), C.byref(on_dev)))
        self.last_cast_on_device = bool(on_dev.value)
        lb = LazyBuffer(out.value, device)
        lb._keep = [self]
        return lb


class LlamaModel(_Handle):
    """ug_llama::Model with random-init weights N(0, std) from the seeded generator."""
    _free = "ugh_llama_model_free"

    def __init__(self, device, ops, cfg, custom_softmax=False, seed=9, std=0.02, round_bf16=False, fused_attention=False, bf16_matrices=False,
                 norm_mean=0.0, embed_std=0.0):
        """norm_mean: the norm vectors are norm_mean + N(0, std); embed_std > 0: the embedding table (= the tied head) is N(0, embed_std)."""
        out = C.c_void_p()
        _chk(host_lib().ugh_llama_model_new_ex(_p(device.h), _p(ops.h), C.byref(cfg), int(custom_softmax), C.c_uint64(seed), C.c_float(std),
                                               int(round_bf16), C.c_float(norm_mean), C.c_float(embed_std), C.byref(out)))
        super().__init__(out.value)
        if fused_attention:
            _chk(host_lib().ugh_llama_model_set_fused_attention(_p(self.h), int(fused_attention)))
        if bf16_matrices:
            _chk(host_lib().ugh_llama_model_store_matrices_bf16(_p(self.h)))
        self._keep = [device, ops]
        self.cfg = cfg

    @classmethod
    def from_safetensors(cls, device, ops, cfg, paths, custom_softmax=False, fused_attention=False, bf16_matrices=False):
        """Weights by their HF names from safetensors file(s), cast to f32 (model.rs:299-346)."""
        if isinstance(paths, (str, bytes, os.PathLike)):
            paths = [paths]
        arr = (C.c_char_p * len(paths))(*[os.fsencode(p) for p in paths])
        out = C.c_void_p()
        _chk(host_lib().ugh_llama_model_from_safetensors(_p(device.h), _p(ops.h), C.byref(cfg), int(custom_softmax), arr, C.c_size_t(len(paths)), C.byref(out)))
        self = cls.__new__(cls)
        _Handle.__init__(self, out.value)
        self._keep = [device, ops]
        self.cfg = cfg
        if fused_attention:
            _chk(host_lib().ugh_llama_model_set_fused_attention(_p(self.h), int(fused_attention)))
        if bf16_matrices:
            _chk(host_lib().ugh_llama_model_store_matrices_bf16(_p(self.h)))
        return self

    def generate(self, prompt, n_steps, forced=None):
        """Prefill over `prompt`, then n_steps greedy single-token steps.  Returns
        (n_steps + 1 token ids, {"prefill_ms", "decode_ms", "margins", "top1"}).
        forced (n_steps ids): decode step i is fed forced[i - 1] instead of the id picked one step earlier."""
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        toks = np.zeros(n_steps + 1, dtype=np.int32)
        margins = np.zeros(n_steps + 1, dtype=np.float32)
        top1 = np.zeros(n_steps + 1, dtype=np.float32)
        pre, dec = C.c_double(), C.c_double()
        fp = None
        if forced is not None:
            forced = np.ascontiguousarray(forced, dtype=np.int32)
            if forced.size != n_steps:
                raise ValueError(f"forced: expected {n_steps} ids, got {forced.size}")
            fp = forced.ctypes.data_as(C.c_void_p)
        _chk(host_lib().ugh_llama_generate_ex(_p(self.h), prompt.ctypes.data_as(C.c_void_p), C.c_size_t(prompt.size), C.c_size_t(n_steps), fp,
                                              toks.ctypes.data_as(C.c_void_p), C.byref(pre), C.byref(dec), margins.ctypes.data_as(C.c_void_p),
                                              top1.ctypes.data_as(C.c_void_p)))
        items = host_lib().ugh_llama_last_decode_items
        items.restype = C.c_size_t
        return toks, {"prefill_ms": pre.value, "decode_ms": dec.value, "margins": margins, "top1": top1, "decode_items": int(items())}
