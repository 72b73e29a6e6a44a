"""The Python module of ug-pyo3 (`import ug`, ug-pyo3/src/lib.rs:600-636) over the HIP backend.

Same classes, method names, argument meaning and error type (ValueError, lib.rs:6-8) as the
reference's extension module, so its examples read the same with `from ug_amd import ug`:

    ug.Device, ug.DType, ug.Func, ug.Slice          lib.rs:23-98, 405-473
    ug.ssa.Instr, ug.ssa.Kernel                      lib.rs:267-402
    ug.op.Arg / Ast / Store / Kernel / load / i32 / f32   lib.rs:100-265

What differs, because the device is not a CUDA one:
  * `ssa.Kernel.hip_code(name)` takes the place of `cuda_code(name)` and `Device.compile_hip` that
    of `compile_cu`; `cuda_code` and `compile_ptx` raise ValueError saying so.
  * `Device.compile(kernel, name=None)` and `Func.launch(*slices)` are additions: the SSA kernel
    goes to the backend as ug-core's `Device::compile` sends it and is re-parallelised there, where
    the text from `hip_code` is the statement-by-statement translation for the launch
    configuration given to `compile_hip` (1 x 1 by default, like the reference's flow).
  * `ssa.Instr.define_acc_f32` builds a DefineAcc; the reference's builds a Const (lib.rs:303-305).
  * `ug.lang`, the block-level front-end of ug-core/src/lower.rs, is not provided.
"""
import ctypes as _C

import numpy as _np

from .. import api as _api
from . import op, ssa  # noqa: F401  (submodules, as in the reference)
from ._util import call as _call

__all__ = ["Device", "DType", "Func", "Slice", "op", "ssa"]


class DType:
    """lib.rs:69-98: the element types, as class attributes."""

    def __init__(self, code, name):
        self._code, self._name = code, name

    def __repr__(self):
        return f"DType.{self._name}"


DType.f32 = DType(_api.F32, "f32")
DType.i64 = DType(_api.I64, "i64")
DType.i32 = DType(_api.I32, "i32")
DType.bf16 = DType(_api.BF16, "bf16")
DType.f16 = DType(_api.F16, "f16")


class Slice:
    """lib.rs:53-67: device memory holding f32 values."""

    def __init__(self, inner):
        self._s = inner

    def to_vec(self):
        return _call(lambda: self._s.to_vec(_api.F32)).tolist()

    def len(self):
        return len(self._s)

    def __len__(self):
        return len(self._s)


class Func:
    """lib.rs:23-51: a compiled kernel with its launch configuration."""

    def __init__(self, device, inner, n_args):
        self._device, self._f, self._n_args = device, inner, n_args

    def launch3(self, s1, s2, s3):
        length, len1, len2 = s3.len(), s1.len(), s2.len()
        if len1 != length:
            raise ValueError(f"length mismatch {len1} <> {length}")
        if len2 != length:
            raise ValueError(f"length mismatch {len2} <> {length}")
        self.launch(s1, s2, s3)

    def launch(self, *slices):
        """Any number of slices, in kernel-argument order (not in the reference)."""
        if self._n_args is not None and len(slices) != self._n_args:
            raise ValueError(f"kernel takes {self._n_args} arguments, got {len(slices)}")
        _call(lambda: self._device._d.run(self._f, [s._s for s in slices]))


class Device:
    """lib.rs:405-473, on GPU `device_id` of this machine."""

    def __init__(self, device_id):
        self._d = _call(lambda: _api.hip_device(int(device_id)))

    def compile_ptx(self, ptx_code, func_name, block_dim=1, grid_dim=1, shared_mem_bytes=0):
        raise ValueError("PTX is CUDA's intermediate language: this device takes HIP source (compile_hip) or an ssa.Kernel (compile)")

    def compile_cu(self, cu_code, func_name, block_dim=1, grid_dim=1, shared_mem_bytes=0):
        raise ValueError("this device compiles HIP source: use Kernel.hip_code() with compile_hip()")

    def compile_hip(self, hip_code, func_name, block_dim=1, grid_dim=1, shared_mem_bytes=0):
        """`compile_cu` (lib.rs:438-456) for HIP source: kernel `func_name` of `hip_code`, launched as
        grid_dim x block_dim with three f32 pointers (what `launch3` passes)."""
        lib = _api.host_lib()
        out = _C.c_void_p()
        dts = (_C.c_int * 3)(_api.F32, _api.F32, _api.F32)

        def go():
            _api._chk(lib.ugh_hip_compile_source(_api._p(self._d.h), hip_code.encode(), func_name.encode(), _C.c_size_t(3), dts, _C.c_uint32(grid_dim),
                                                 _C.c_uint32(block_dim), _C.c_uint32(shared_mem_bytes), _C.byref(out)))
        _call(go)
        return Func(self, _api.Func(out.value), 3)

    def compile(self, kernel, name=None):
        """ug::Device::compile (ug-core/src/lib.rs:56-60) on an `ssa.Kernel` (not in the reference's module)."""
        f = _call(lambda: self._d.compile(kernel._k, name))
        return Func(self, f, int(kernel._k.wire().n_args))

    def zeros(self, len):  # noqa: A002  (the reference's argument name)
        return Slice(_call(lambda: self._d.slice_from(_np.zeros(int(len), _np.float32))))

    def slice(self, vs):
        return Slice(_call(lambda: self._d.slice_from(_np.asarray(list(vs), dtype=_np.float32))))

    def synchronize(self):
        _call(self._d.synchronize)
