"""`ug_amd.ug`: the Python module of ug-pyo3 (ug-pyo3/src/lib.rs) over the HIP backend, driven the way
the reference's py-examples/softmax.py and py-examples/dotprod.py drive theirs."""
import ctypes as C

import numpy as np
import pytest

import ug_amd
from ug_amd import rng, ug
from ug_amd.ug.ssa import Instr, Kernel


def softmax_kernel(dim1, dim2, dst_first=True):
    # py-examples/softmax.py:3-12 (broadcast takes the target shape, lib.rs:174-177)
    src_ptr = ug.op.Arg.ptr_f32()
    dst_ptr = ug.op.Arg.ptr_f32()
    src = ug.op.load(src_ptr, (dim1, dim2))
    exps = (src - src.max(1).broadcast((dim1, dim2))).exp()
    sm = exps / exps.sum(1).broadcast((dim1, dim2))
    st = ug.op.Store(dst_ptr, (dim1, dim2), sm)
    return ug.op.Kernel("softmax", [dst_ptr, src_ptr] if dst_first else [src_ptr, dst_ptr], [st])


def add_kernel(vec_len):
    # py-examples/dotprod.py:6-18 (DefineGlobal carries the element type, lib.rs:334-337)
    return Kernel([
        Instr.define_global(0, ug.DType.f32),
        Instr.define_global(1, ug.DType.f32),
        Instr.define_global(2, ug.DType.f32),
        Instr.const_i32(0),
        Instr.const_i32(vec_len),
        Instr.range(3, 4, 10),
        Instr.load(1, 5, ug.DType.f32),
        Instr.load(2, 5, ug.DType.f32),
        Instr.binary("add", 6, 7, ug.DType.f32),
        Instr.store(0, 5, 8, ug.DType.f32),
        Instr.end_range(5),
    ])


def raw_instrs(kernel):
    return [bytes(i) for i in kernel._k.instrs()]


def test_op_kernel_lowers_to_the_sample_softmax():
    """The kernel py-examples/softmax.py builds is ug::samples::op::softmax (samples.rs:236-249), which lists
    the source before the destination: with the arguments in that order the SSA is the same, line for line."""
    k = softmax_kernel(512, 128)
    sample = ug_amd.SsaKernel.sample_op("softmax", 512, 128)
    assert k.lower().flops_and_mem() == ug_amd_flops(sample)
    assert raw_instrs(softmax_kernel(512, 128, dst_first=False).lower()) == [bytes(i) for i in sample.instrs()]
    text = str(k)
    assert text.startswith('Kernel { name: "softmax"') and "ReduceMax" in text and "ReduceSum" in text
    listing = str(k.lower()).splitlines()
    assert listing[0] == "000 DefineGlobal { index: 0, dtype: F32 }"
    assert listing[2] == "002 Range { lo: Const(I32(0)), up: Const(I32(512)), step: 1, end_idx: 41 }"
    assert sum("DefineAcc" in line for line in listing) == 3      # max, max again inside the sum, sum (the reference recomputes)
    assert listing[-1].startswith("041 EndRange")


def ug_amd_flops(ssa_kernel):
    return Kernel._wrap(ssa_kernel).flops_and_mem()


def test_ast_shapes_and_errors():
    a = ug.op.Arg.ptr_f32()
    x = ug.op.load(a, (4, 6))
    assert x.shape() == (4, 6)
    assert x.sum(1).shape() == (4, 1) and x.max(0).shape() == (1, 6)
    assert x.sum(1).broadcast((4, 6)).shape() == (4, 6)
    assert (-x).shape() == (4, 6) and ug.op.f32(2.0).shape() == ()
    assert "Ptr(F32)" in str(a) and "Value(I32)" in str(ug.op.Arg.i32())
    with pytest.raises(ValueError, match="cannot broadcast"):
        x.broadcast((4, 7))
    with pytest.raises(ValueError, match="less dimensions"):
        x.broadcast((6,))
    with pytest.raises(ValueError, match="unexpected dtype for load"):
        ug.op.load(ug.op.Arg.f32(), (2,))
    with pytest.raises(ValueError, match="dtype mismatch"):
        x + ug.op.load(ug.op.Arg.ptr_i32(), (4, 6))
    with pytest.raises(ValueError, match="no dim"):
        x.sum(2)


def test_ssa_instrs_listing_flops_and_text():
    k = add_kernel(128)
    lines = str(k).splitlines()
    assert lines[5] == "005 Range { lo: Var(3), up: Var(4), step: 1, end_idx: 10 }"
    assert lines[8] == "008 Binary { op: Add, lhs: Var(6), rhs: Var(7), dtype: F32 }"
    assert str(k.to_list()[9]) == "Store { dst: 0, offset: Var(5), value: Var(8), dtype: F32 }"
    assert len(k.to_list()) == 11
    assert k.flops_and_mem() == (128, 3 * 128 * 4)          # lang.rs:755-811: per thread, loop trips multiplied in
    assert str(Instr.define_acc_f32(0.5)) == "DefineAcc(Const(F32(0.5)))"
    assert str(Instr.special_ti()) == "Special(ThreadIdx)" and str(Instr.special_bi()) == "Special(BlockIdx)"
    with pytest.raises(ValueError, match="unknown binary op 'pow'"):
        Instr.binary("pow", 0, 1, ug.DType.f32)
    with pytest.raises(ValueError, match="unknown unary op 'sqrt'"):
        Instr.unary("sqrt", 0, ug.DType.f32)
    with pytest.raises(ValueError, match="unexpected order for arguments"):
        Kernel([Instr.define_global(1, ug.DType.f32)])
    with pytest.raises(ValueError, match="HIP"):
        k.cuda_code("sum")


def test_hip_code_is_the_kernel_as_written_and_builds_for_gfx950():
    k = add_kernel(128)
    code = k.hip_code("sum")
    assert 'extern "C" __global__ void __launch_bounds__(1) sum(float* __restrict__ v0, const float* __restrict__ v1, const float* __restrict__ v2)' in code
    assert "for (int v5 = v3; v5 < v4; v5 += 1)" in code
    n = C.c_size_t()
    lib = ug_amd.ughip_lib()
    assert lib.ughip_rtc_check(code.encode(), b"gfx950", C.byref(n)) == 0, lib.ughip_last_error().decode()
    assert n.value > 0
    sm = softmax_kernel(8, 16).lower().hip_code("softmax")
    body = sm[sm.index('extern "C" __global__'):]
    assert body.count("for (int ") == 5 and 'void __launch_bounds__(1) softmax(' in body      # rows, columns, max, max, sum
    assert lib.ughip_rtc_check(sm.encode(), b"gfx950", C.byref(n)) == 0, lib.ughip_last_error().decode()
    with pytest.raises(ValueError, match="not a valid kernel name"):
        k.hip_code("no spaces")


@pytest.mark.gpu
def test_dotprod_example_runs_on_the_gpu():
    """py-examples/dotprod.py:1-31 with hip_code / compile_hip in place of cuda_code / compile_cu."""
    print("ug module: dotprod example", flush=True)
    device = ug.Device(0)
    kernel = add_kernel(128)
    func = device.compile_hip(kernel.hip_code("sum"), "sum")
    s1 = device.slice([1.0, 2.0, 3.0, 4.0] * 32)
    s2 = device.slice(range(128))
    s_dst = device.zeros(128)
    assert s_dst.to_vec() == [0.0] * 128 and s_dst.len() == 128
    func.launch3(s_dst, s1, s2)
    device.synchronize()
    assert s_dst.to_vec() == [float([1, 2, 3, 4][i % 4] + i) for i in range(128)]
    # the same kernel through ug::Device::compile (re-parallelised by the backend)
    fast = device.compile(kernel)
    again = device.zeros(128)
    fast.launch3(again, s1, s2)
    assert again.to_vec() == s_dst.to_vec()
    with pytest.raises(ValueError, match="length mismatch 64 <> 128"):
        func.launch3(s_dst, device.zeros(64), s2)
    with pytest.raises(ValueError, match="length mismatch 128 <> 5"):      # lengths are compared with the third slice's (lib.rs:30-39)
        func.launch3(s_dst, s1, device.zeros(5))
    with pytest.raises(ValueError, match="already borrowed"):
        func.launch3(s_dst, s1, s_dst)
    with pytest.raises(ValueError, match="PTX"):
        device.compile_ptx("", "sum")
    with pytest.raises(ValueError, match="no kernel 'other'"):
        device.compile_hip(kernel.hip_code("sum"), "other")
    with pytest.raises(ValueError, match="compilation failed"):
        device.compile_hip("this is not HIP", "sum")


@pytest.mark.gpu
def test_softmax_example_runs_on_the_gpu():
    """py-examples/softmax.py's kernel, lowered, on the device both ways: as written (one thread, like the
    reference's flow with its default 1 x 1 launch) and through the backend's own mapping."""
    print("ug module: softmax example", flush=True)
    dim1, dim2 = 64, 96
    device = ug.Device(0)
    ssa = softmax_kernel(dim1, dim2).lower()
    x = rng.normal(141, dim1 * dim2, 2.0)
    e = np.exp(x.reshape(dim1, dim2).astype(np.float64) - x.reshape(dim1, dim2).max(1, keepdims=True))
    truth = (e / e.sum(1, keepdims=True)).ravel()
    src = device.slice(x.tolist())
    outs = []
    for func in (device.compile_hip(ssa.hip_code("softmax"), "softmax"), device.compile(ssa, "softmax")):
        dst = device.zeros(dim1 * dim2)
        func.launch(dst, src) if func._n_args == 2 else func.launch(dst, src, device.zeros(1))
        device.synchronize()
        outs.append(np.array(dst.to_vec(), np.float32))
        np.testing.assert_allclose(outs[-1], truth, rtol=2e-6, atol=1e-9)
    np.testing.assert_allclose(outs[0], outs[1], rtol=1e-6, atol=1e-9)
