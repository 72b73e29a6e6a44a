"""ug_amd: MI355X (gfx950) backend for ug, behind the C ABI of include/ughip.h.

Python only binds the native libraries with ctypes; all compute is HIP.  Importing this package
loads `lib/libughip.so` (backend) and `lib/libug_host.so` (host-side lazy-buffer front-end) and
raises if they have not been built -- there is no CPU fallback.
"""
from .api import (  # noqa: F401
    BF16, F16, F32, I32, I64,
    CompilationCache, Device, Func, LazyBuffer, LlamaConfig, LlamaModel, LlamaOps, Safetensors, Schedule, Slice, SsaKernel, UgError,
    hip_device, host_lib, last_kernel, ughip_lib, llama, np_dtype, set_tuning, tuning, set_llama_switch, llama_switches,
)
from . import rng  # noqa: F401
