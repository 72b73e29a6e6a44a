"""Pins the oracle (oracle/): every golden vector the reference's tests hold for this path, run
through the restated interpreter and the restated CPU backend (C emission + gcc)."""
import ctypes as C

import numpy as np
import pytest

import ref_suite
from ref_suite import GOLD, f32
import ug_amd
from ug_amd import F32, I32, LazyBuffer as LB, Schedule, SsaKernel, rng


def eval_ssa(oracle, kernel, buffers, n_lanes, grid_idx=0):
    """ug::interpreter::eval_ssa::<N>(&kernel, buffers, &[], grid_idx)"""
    n = len(buffers)
    datas = (C.c_void_p * n)(*[b.ctypes.data for b in buffers])
    dts = (C.c_int * n)(*[F32 if b.dtype == np.float32 else I32 for b in buffers])
    lens = (C.c_size_t * n)(*[b.size for b in buffers])
    rc = oracle.ugo_eval_ssa(C.c_void_p(kernel.h), datas, dts, lens, C.c_size_t(n), C.c_size_t(n_lanes), C.c_size_t(grid_idx))
    if rc:
        raise RuntimeError(oracle.ugo_last_error().decode())


# ---- ug-core/tests/basic_tests.rs ----------------------------------------------------------------------
def test_eval_add(oracle):
    g = GOLD["eval_add"]
    a = np.zeros(2, np.int32)
    eval_ssa(oracle, SsaKernel.sample("simple_add", 2), [a, np.array(g["b"], np.int32), np.array(g["c"], np.int32)], 1)
    assert a.tolist() == g["expect"]


def test_eval_dotprod(oracle):
    g = GOLD["eval_dotprod"]
    a = np.zeros(1, np.float32)
    eval_ssa(oracle, SsaKernel.sample("simple_dotprod", 2), [a, f32(g["b"]), f32(g["c"])], 1)
    assert a.tolist() == g["expect"]


def test_softmax_op_lowered(oracle):
    g = GOLD["softmax"]
    k = SsaKernel.sample_op("softmax", g["rows"], g["cols"])
    a, b = f32(g["input"]), np.zeros(8, np.float32)
    eval_ssa(oracle, k, [a, b], 1)
    np.testing.assert_array_equal(b, f32(g["expect"]))


@pytest.mark.parametrize("name", ["softmax_barrier", "softmax_reduce"])
def test_ssa_softmax(oracle, name):
    g = GOLD["softmax"]
    k = SsaKernel.sample(name, g["rows"], g["cols"])
    a, b = f32(g["input"]), np.zeros(8, np.float32)
    for group in range(g["rows"]):
        eval_ssa(oracle, k, [a, b], g["cols"], group)
    np.testing.assert_array_equal(b, f32(g["expect"]))


def test_affine(oracle):
    g = GOLD["affine"]
    a = f32(g["input"])
    eval_ssa(oracle, SsaKernel.sample_op("affine", 4), [a], 4)
    assert a.tolist() == g["expect"]


def test_interpreter_rejects_divergence(oracle):
    # exp_block steps threads over a row; with a mismatched lane count the Range diverges
    k = SsaKernel.sample_op("softmax", 2, 4, block_axis=0, thread_dim=1, thread_block_dim=3)
    with pytest.raises(RuntimeError, match="diverging"):
        eval_ssa(oracle, k, [f32(GOLD["softmax"]["input"]), np.zeros(8, np.float32)], 3, 0)


# ---- ug-core/tests/cpu_tests.rs -------------------------------------------------------------------------
def test_cpu_run_add(oracle, cpu):
    g = GOLD["cpu_run_add"]
    k = SsaKernel.sample("simple_add", 6)
    n = C.c_size_t()
    assert oracle.ugo_gen_c(C.c_void_p(k.h), b"foo", None, C.c_size_t(0), C.byref(n)) == 0
    buf = C.create_string_buffer(n.value + 1)
    oracle.ugo_gen_c(C.c_void_p(k.h), b"foo", buf, C.c_size_t(n.value + 1), None)
    code = buf.value.decode()
    assert code.startswith("#include<math.h>\nvoid foo(\n  int* __var0,\n  int* __var1,\n  int* __var2\n) {\n")
    assert "  for (int __var3 = 0; __var3 < 6; __var3+=1) {\n    int __var4 = __var1[__var3];\n" in code
    func = cpu.compile(k, "foo")
    v1 = cpu.slice_from(np.zeros(6, np.int32))
    cpu.run(func, [v1, cpu.slice_from(np.array(g["v2"], np.int32)), cpu.slice_from(np.array(g["v3"], np.int32))])
    assert v1.to_vec().tolist() == g["expect"]


def test_c_text_of_softmax_exp_kernel(oracle, cpu):
    """The exact C of the first softmax kernel on [32,1024] (hand-traced from lower_op.rs and
    cpu_code_gen.rs): names the kernel, hoists nothing, fmax for the fold, -inf as `-1. / 0.`."""
    src = LB.copy(np.zeros(32 * 1024, np.float32), (32, 1024), cpu)
    s = Schedule.create_one(ref_suite.softmax_graph(src))
    items = s.items()
    assert [i["kind"] for i in items] == ["kernel", "kernel"]
    assert [i["name"] for i in items] == ["Ue_Bs_O_Lb_Rx_O", "Bd_O_Lb_Rs_O"]
    assert [i["n_args"] for i in items] == [2, 2]
    k = s.item_ssa(0)
    n = C.c_size_t()
    oracle.ugo_gen_c(C.c_void_p(k.h), b"k", None, C.c_size_t(0), C.byref(n))
    buf = C.create_string_buffer(n.value + 1)
    oracle.ugo_gen_c(C.c_void_p(k.h), b"k", buf, C.c_size_t(n.value + 1), None)
    expect = """#include<math.h>
void k(
  float* __var0,
  float* __var1
) {
  for (int __var2 = 0; __var2 < 32; __var2+=1) {
    for (int __var3 = 0; __var3 < 1024; __var3+=1) {
      int __var4 = __var2 * 1024;
      int __var5 = __var3 + __var4;
      int __var6 = __var2 * 1024;
      int __var7 = __var3 + __var6;
      float __var8 = __var0[__var7];
      float __var9 = -1. / 0.;
      for (int __var10 = 0; __var10 < 1024; __var10+=1) {
        int __var11 = __var2 * 1024;
        int __var12 = __var10 + __var11;
        float __var13 = __var0[__var12];
        float __var14 = fmax(__var9, __var13);
        __var9 = __var14;
      }
      float __var17 = __var8 - __var9;
      float __var18 = expf(__var17);
      __var1[__var5] = __var18;
    }
  }
}
"""
    assert buf.value.decode() == expect


# ---- ug-core/tests/lb_tests.rs + common_tests.rs on the restated CPU backend ------------------------------
@pytest.mark.parametrize("case", ref_suite.ALL, ids=lambda f: f.__name__)
def test_lb_reference_cases(cpu, case):
    case(cpu)


def test_schedule_interpret_and_cpu_agree(oracle, cpu):
    # lb_tests.rs:5-49
    s = ref_suite.schedule_one_item(cpu)
    k = s.item_ssa(0, optimize=False)
    buf = np.zeros(10, np.float32)
    eval_ssa(oracle, k, [buf], 1)
    assert buf.tolist() == GOLD["lb_add"]["expect"]
    func = cpu.compile(k)
    out = cpu.allocate_uninit(F32, 10)
    cpu.run(func, [out])
    assert out.to_vec().tolist() == GOLD["lb_add"]["expect"]


def test_more_than_five_args_is_an_error(cpu):
    # cpu_runtime.rs:331
    xs = [LB.copy(f32([i, i]), (2,), cpu) for i in range(6)]
    acc = xs[0]
    for x in xs[1:]:
        acc = acc.binary("add", x)
    with pytest.raises(Exception, match="unsupported number of args"):
        acc.data_vec()


def test_copy_checks(cpu):
    # cpu_runtime.rs:376-412
    s = cpu.allocate_uninit(F32, 4)
    assert s.to_vec().tolist() == [0, 0, 0, 0]  # zero-filled (cpu_runtime.rs:255-264)
    with pytest.raises(Exception, match="len mismatch"):
        s.copy_host_to_device(np.zeros(3, np.float32))
    with pytest.raises(Exception, match="dtype mismatch"):
        s.copy_host_to_device(np.zeros(4, np.int32))


def test_cpu_matmul_f16(cpu):
    """cpu_runtime.rs:345-356 accepts F16 as well as F32; f32 accumulation, one rounding at the end."""
    a = np.floor(rng.uniform_pm1(40, 2 * 5 * 7) * 8).astype(np.float16).reshape(2, 5, 7)
    w = np.floor(rng.uniform_pm1(41, 2 * 7 * 3) * 8).astype(np.float16).reshape(2, 7, 3)
    got = LB.copy(a, a.shape, cpu).matmul(LB.copy(w, w.shape, cpu))
    assert got.dtype == ug_amd.F16
    np.testing.assert_array_equal(got.data_vec().reshape(2, 5, 3), (a.astype(np.float32) @ w.astype(np.float32)).astype(np.float16))
    x = rng.uniform_pm1(42, 4 * 64).astype(np.float16).reshape(4, 64)
    y = rng.uniform_pm1(43, 64 * 6).astype(np.float16).reshape(64, 6)
    got = LB.copy(x, x.shape, cpu).matmul(LB.copy(y, y.shape, cpu)).data_vec().astype(np.float64).reshape(4, 6)
    exact = x.astype(np.float64) @ y.astype(np.float64)
    assert np.all(np.abs(got - exact) <= 2.0 ** -11 * np.abs(exact) + 64 * np.finfo(np.float32).eps * (np.abs(x).astype(np.float64) @ np.abs(y).astype(np.float64)))
    with pytest.raises(ug_amd.UgError, match="incorrect dtypes"):
        LB.copy(rng.to_bf16_bits(x.astype(np.float32)), x.shape, cpu).matmul(LB.copy(rng.to_bf16_bits(y.astype(np.float32)), y.shape, cpu)).data_vec()
