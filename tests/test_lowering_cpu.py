"""CPU-side checks of the HIP backend: the C ABI exports what include/ughip.h declares, and every
kernel the lazy-graph cases produce lowers to HIP source that hiprtc accepts for gfx950 (no GPU is
needed to compile).  No compute call is made here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import cases
import ref_suite
import ug_amd
from ug_amd import LazyBuffer as LB, Schedule, SsaKernel

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_c_abi_exports_every_declared_symbol():
    text = open(os.path.join(ROOT, "include", "ughip.h")).read()
    names = sorted(set(re.findall(r"\b(ughip_[a-z0-9_]+)\s*\(", text)))
    assert len(names) >= 25
    lib = ug_amd.ughip_lib()
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    assert lib.ughip_use_grid() == 0


def test_entry_points_refuse_a_null_device_without_touching_the_gpu():
    """Argument checks come before any HIP call: every data entry point answers a null device (or null
    slices) with an error code and a message, on a box without a GPU too."""
    lib = ug_amd.ughip_lib()
    z, n3 = C.c_size_t(0), (C.c_size_t * 3)(4, 4, 4)
    f = C.c_float(1.0)
    calls = {
        "ughip_softmax_rows": (None, None, None, z, z),
        "ughip_causal_mask": (None, None, None, z, z, z),
        "ughip_rope": (None, None, None, None, None, None, z, z, z, 0),
        "ughip_cat": (None, None, None, None, z, z, z),
        "ughip_causal_softmax_rows": (None, None, None, z, z, z),
        "ughip_attention_decode": (None, None, None, None, None, z, z, z, z, z, f),
        "ughip_rope_append": (None, None, None, None, z, z, z, None, None, None, 0),
        "ughip_kv_append": (None, None, None, z, z, z, z, z, z, z, z, None, None, None, 0),
        "ughip_kv_append_pair": (None, None, None, None, z, z, z, z, z, z, z, z, z, None, None, None, 0),
        "ughip_attention_cached": (None, None, z, z, None, None, None, z, z, z, C.c_size_t(2), z, z, C.c_size_t(64), f, None, None, None, 0),
        "ughip_attention_cached_linear_add_rows": (None, None, z, z, None, None, z, z, C.c_size_t(2), C.c_size_t(2), z, z, C.c_size_t(64), f, None, None, None, 0, None, None, None, z, C.c_int(0)),
        "ughip_attention_step": (None, None, z, z, z, z, None, None, None, z, z, z, z, z, z, f, None, None, None, 0),
        "ughip_gemv_multi": (None, None, C.c_size_t(1), None, n3, C.c_size_t(4), None),
        "ughip_rms_gemv_multi": (None, None, None, f, C.c_size_t(1), None, n3, C.c_size_t(4), None),
        "ughip_gemv_gate_up": (None, None, None, None, None, z, C.c_size_t(4)),
        "ughip_rms_gemv_gate_up": (None, None, None, f, None, None, None, z, C.c_size_t(4)),
        "ughip_gemv_add": (None, None, None, None, None, z, C.c_size_t(4)),
        "ughip_linear_rows": (None, None, None, None, C.c_size_t(16), z, C.c_size_t(32), C.c_int(0)),
        "ughip_linear_add_rows": (None, None, None, None, None, C.c_size_t(16), z, C.c_size_t(32), C.c_int(0)),
        "ughip_linear_swiglu_rows": (None, None, None, None, C.c_size_t(16), z, C.c_size_t(32), C.c_int(0)),
        "ughip_rms_linear_rows": (None, None, None, f, None, None, C.c_size_t(16), z, C.c_size_t(32), C.c_int(0)),
        "ughip_rms_mlp_rows": (None, None, None, f, None, None, None, None, C.c_size_t(16), z, C.c_size_t(32), C.c_size_t(32), C.c_int(0)),
        "ughip_argmax_row": (None, None, C.c_size_t(4), z, None, None, None, z),
        "ughip_convert": (None, None, None),
        "ughip_matmul": (None, None, None, None, z, z, z, z, z, None, None, z, None, None, z),
    }
    for name, args in calls.items():
        rc = getattr(lib, name)(*args)
        assert rc != 0, name
        assert lib.ughip_last_error(), name


def test_no_gpu_is_a_loud_error_not_a_fallback():
    lib = ug_amd.ughip_lib()
    dev = C.c_void_p()
    rc = lib.ughip_device_create(0, C.byref(dev))
    if rc == 0:  # running on a GPU box: nothing to check here
        lib.ughip_device_release(dev)
        return
    assert b"HIP" in lib.ughip_last_error() or b"device" in lib.ughip_last_error()
    with pytest.raises(ug_amd.UgError):
        ug_amd.hip_device(0)


def rtc_ok(source):
    lib = ug_amd.ughip_lib()
    n = C.c_size_t()
    rc = lib.ughip_rtc_check(source.encode(), b"gfx950", C.byref(n))
    assert rc == 0, lib.ughip_last_error().decode()
    assert n.value > 0


def kernels_of(build, cpu):
    s = Schedule.create_one(build(cpu))
    out = []
    for i, item in enumerate(s.items()):
        if item["kind"] in ("kernel", "ssa"):
            out.append((item.get("name", "ssa"), s.item_ssa(i)))
    return out


@pytest.mark.parametrize("name,build,tol", cases.ELEMENTWISE_AND_REDUCE, ids=[c[0] for c in cases.ELEMENTWISE_AND_REDUCE])
def test_case_kernels_lower_and_compile(cpu, name, build, tol):
    ks = kernels_of(build, cpu)
    assert ks
    for kname, k in ks:
        src, info = k.hip_code(kname)
        assert 'extern "C" __global__' in src
        assert info["grid_dim"] >= 1 and 1 <= info["block_dim"] <= 1024
        rtc_ok(src)


def strategies(build, cpu):
    return [k.hip_code(n)[1]["strategy"] for n, k in kernels_of(build, cpu)]


def test_strategy_selection(cpu):
    assert strategies(cases.softmax((32, 1024)), cpu) == ["row_block", "row_block"]
    assert strategies(cases.softmax((4096, 128)), cpu) == ["row_block", "row_block"]
    assert strategies(cases.residual_add((1, 3, 2048)), cpu) == ["elementwise"]
    assert strategies(cases.rms_norm((1, 5, 2048)), cpu) == ["row_block"]
    # a reduce over the strided dim walks memory along the rows: one thread per column
    assert strategies(cases.reduce_dim((300, 70), "sum", 0), cpu) == ["row_thread"]
    assert strategies(cases.reduce_dim((70, 300), "sum", 1), cpu) == ["row_block"]
    # config 2: one output, 2^24-long reduction -> whole-device reduction
    (k,) = kernels_of(cases.fused_reduce(1 << 24), cpu)
    src, info = k[1].hip_code(k[0])
    assert info["strategy"] == "grid_reduce" and info["grid_dim"] >= 256 and info["scratch_bytes"] > 0
    rtc_ok(src)
    # its first stage streams the operands once, with loads that do not claim cache lines; nothing else does
    first, fin = src.split('extern "C" __global__')[1:]
    assert first.count("__builtin_nontemporal_load(") == 3 and "__builtin_nontemporal_load" not in fin
    for n, kk in kernels_of(cases.softmax((4096, 1024)), cpu):
        assert "__builtin_nontemporal_load" not in kk.hip_code(n)[0]


@pytest.mark.parametrize("dtype", [ug_amd.F32, ug_amd.I32, ug_amd.I64])
def test_grid_reduce_compiles_for_every_accumulator_type(cpu, dtype):
    """Cooperative reductions exist for 32- and 64-bit accumulators (a 16-bit sum depends on its order too much to
    be split; those kernels keep one thread per output)."""
    def build(dev):
        # only scheduled and lowered here; narrow as in config 2: a reduce keeps its dim at full length (lazy_buffer.rs:453-467)
        return LB.copy(np.zeros(1 << 22, np.float32), (1 << 22,), dev).cast(dtype).reduce("max", 0).narrow(0, 0, 1)
    ks = kernels_of(build, cpu)
    src, info = ks[-1][1].hip_code("wide_max")
    assert info["strategy"] == "grid_reduce" and "__builtin_nontemporal_load(" in src
    rtc_ok(src)


def test_gpu_style_ssa_is_translated_literally():
    for name, args, launch in [("exp", (64,), (4, 64)), ("exp_block", (256, 64), (4, 64)), ("softmax_barrier", (2, 64), (2, 64)),
                               ("softmax_reduce", (2, 64), (2, 64)), ("softmax_block", (2, 256, 64), (2, 64))]:
        k = SsaKernel.sample(name, *args)
        k.set_launch(*launch)
        src, info = k.hip_code(name)
        assert info["strategy"] == "literal" and (info["grid_dim"], info["block_dim"]) == launch
        rtc_ok(src)


def test_scheduler_grid_ssa_with_reduce_local_compiles():
    # what a `use_grid() == true` device would receive (schedule.rs:162-188)
    k = SsaKernel.sample_op("softmax", 32, 1024, block_axis=0, thread_dim=1, thread_block_dim=32)
    src, info = k.hip_code("softmax_grid")
    assert info["strategy"] == "literal" and "ug_block_reduce_dyn" in src
    rtc_ok(src)


def test_malformed_ssa_is_rejected():
    from ug_amd.api import Instr
    bad = Instr()
    bad.op = 8  # Load from an undefined pointer var
    bad.v = 5
    k = SsaKernel.from_instrs([bad])
    with pytest.raises(ug_amd.UgError, match="ssa lowering"):
        k.hip_code()


def test_zero_sized_nest_is_an_empty_launch(cpu):
    # the initial KV cache: cst(0) of shape [1,4,0,64] (ug-llama/src/model.rs:192)
    lb = LB.cst(0.0, (1, 4, 0, 64), cpu)
    s = Schedule.create_one(lb)
    k = s.item_ssa(0)
    src, info = k.hip_code("empty")
    assert "extern" in src
    assert lb.data_vec().size == 0


def test_rng_matches_native_generator():
    lib = ug_amd.host_lib()
    out = np.zeros(1001, np.float32)
    assert lib.ugh_synthetic_weights(C.c_uint64(9), C.c_float(0.02), 0, b"model.norm.weight", C.c_size_t(1001), out.ctypes.data_as(C.c_void_p)) == 0
    # python restatement of tensor_seed (FNV-1a folded into the seed)
    h = 0xcbf29ce484222325
    for c in b"model.norm.weight":
        h = ((h ^ c) * 0x100000001b3) & 0xFFFFFFFFFFFFFFFF
    from ug_amd.rng import _mix, normal
    with np.errstate(over="ignore"):
        ts = int(_mix(np.uint64(9 ^ h)))
    ref = normal(ts, 1001, 0.02)
    np.testing.assert_allclose(out, ref, rtol=1e-6, atol=1e-9)
    assert abs(float(out.std()) - 0.02) < 0.002
    # bf16 rounding helper agrees with the native one
    out16 = np.zeros(1001, np.float32)
    lib.ugh_synthetic_weights(C.c_uint64(9), C.c_float(0.02), 1, b"model.norm.weight", C.c_size_t(1001), out16.ctypes.data_as(C.c_void_p))
    np.testing.assert_array_equal(out16, ug_amd.rng.bf16_round(out))


def test_ref_suite_graph_shapes(cpu):
    a = LB.copy(np.ones(8, np.float32), (8,), cpu)
    b = LB.copy(np.ones(8, np.float32), (8,), cpu)
    r = ref_suite.fused_reduce_graph(a, b, cpu)
    assert r.dims() == [1]
    assert r.data_vec().tolist() == [12.0]


def _guard_prog(store_offset_var, extra=()):
    """A GPU-style kernel over 2 x 64 threads: i = bi * 64 + ti, then `extra` instructions, then a store of 3.0 at
    variable `store_offset_var` under If(var 6) where var 6 = max(100 - i, 0)."""
    from ug_amd.api import A, Instr
    I32_, F32_ = int(ug_amd.I32), int(ug_amd.F32)

    def var(i):
        return A(0, I32_, 0, i, 0, 0.0, 0)

    def ci(v):
        return A(1, I32_, 0, 0, v, 0.0, 0)

    def ins(op, dtype=0, sub=0, v=0, n=0, a=None, b=None):
        return Instr(op, dtype, sub, v, n, a or A(), b or A())

    extra = [ins(6, I32_, sub=sub, a=(var(a) if va else ci(a)), b=(var(b) if vb else ci(b))) for sub, va, a, vb, b in extra]
    n_if = 7 + len(extra)
    prog = [
        ins(1, F32_, n=0),                              # 0 DefineGlobal{0, F32}
        ins(3, I32_, sub=0),                            # 1 ThreadIdx
        ins(3, I32_, sub=1),                            # 2 BlockIdx
        ins(6, I32_, sub=2, a=var(2), b=ci(64)),        # 3 bi * 64
        ins(6, I32_, sub=0, a=var(3), b=var(1)),        # 4 i = bi * 64 + ti
        ins(6, I32_, sub=1, a=ci(100), b=var(4)),       # 5 100 - i
        ins(6, I32_, sub=6, a=var(5), b=ci(0)),         # 6 max(100 - i, 0): non-zero iff i < 100
    ] + extra + [
        ins(11, v=n_if + 2, a=var(6)),                  # If
        ins(13, F32_, v=0, a=var(store_offset_var), b=A(1, F32_, 0, 0, 0, 3.0, 0)),
        ins(12),                                        # EndIf
    ]
    return SsaKernel.from_instrs(prog, grid=2, block=64)


def test_a_guard_that_bounds_the_offset_narrows_the_length_a_slice_must_have():
    """`If(max(100 - i, 0))` around `dst[i]` with i up to 127: the body runs for i <= 99 only, so 100 elements are asked
    for; `dst[2 i + 1]` under the same guard: 200 (integers computed from the narrowed one narrow with it)."""
    assert _guard_prog(4).min_lens() == [100]
    two_i_plus_1 = [(2, True, 4, False, 2), (0, True, 7, False, 1)]   # 7 = i * 2, 8 = (i * 2) + 1
    assert _guard_prog(8, two_i_plus_1).min_lens() == [200]


def test_a_guard_that_says_nothing_about_the_offset_leaves_the_full_requirement():
    """The store's offset is a second copy of bi * 64 + ti that the guard's expression does not go through (an unrelated
    condition as far as the analysis can prove): all 128 offsets the grid can form count, and a 100-element slice
    would be refused by ughip_run."""
    other_i = [(2, True, 2, False, 64), (0, True, 7, True, 1)]        # 7 = bi * 64, 8 = 7 + ti
    assert _guard_prog(8, other_i).min_lens() == [128]
    # a guard on the thread index alone (ti < 50) bounds ti, not the block: 64 + 49 + 1
    from ug_amd.api import A, Instr
    k = _guard_prog(4)
    prog = list(k.instrs())
    I32_ = int(ug_amd.I32)
    prog[5] = Instr(6, I32_, 1, 0, 0, A(1, I32_, 0, 0, 50, 0.0, 0), A(0, I32_, 0, 1, 0, 0.0, 0))   # 5 = 50 - ti
    assert SsaKernel.from_instrs(prog, grid=2, block=64).min_lens() == [114]


def _plan(dtype, rhs_dtype, b, m, n, k, rhs_nk):
    lib = ug_amd.ughip_lib()
    buf = C.create_string_buffer(200)
    rc = lib.ughip_matmul_plan(int(dtype), int(rhs_dtype), C.c_size_t(b), C.c_size_t(m), C.c_size_t(n), C.c_size_t(k), int(rhs_nk), buf, C.c_size_t(200))
    if rc:
        raise ug_amd.UgError(lib.ughip_last_error().decode())
    return buf.value.decode()


def _rows_plan(w_dtype, product, form, m, n, k):
    lib = ug_amd.ughip_lib()
    buf = C.create_string_buffer(200)
    rc = lib.ughip_linear_rows_plan(int(w_dtype), int(product), int(form), C.c_size_t(m), C.c_size_t(n), C.c_size_t(k), buf, C.c_size_t(200))
    if rc:
        raise ug_amd.UgError(lib.ughip_last_error().decode())
    return buf.value.decode()


def test_kernel_choice_for_the_rows_of_a_prompt_is_pinned():
    """The projections of a llama layer (TinyLlama-1.1B shapes) for prompts of several lengths, f32 rows against bf16 matrices
    as three bf16 terms: 33 .. 128 rows take rows_x3 with the units per workgroup its cost rule picks (every CU busy in one
    round, then as few slabs as the units' time allows); fewer rows and more take the kernels that read planes.  Written down
    so that a changed rule shows here (the GPU suite checks that the launch reports the planned name:
    test_rows_plan_names_what_is_launched)."""
    B, F = ug_amd.BF16, ug_amd.F32
    X3, F32P = 1, 0
    want = {
        # (w dtype, product, form, m, n, k)
        (B, X3, 0, 128, 2560, 2048): "rows_x3<128x128,3 terms split in the kernel,4 units x 160 workgroups,8 slabs,fold>",
        (B, X3, 1, 128, 2048, 2048): "rows_x3<128x128,3 terms split in the kernel,4 units x 128 workgroups,8 slabs,+residual in the fold>",
        (B, X3, 2, 128, 5632, 2048): "rows_x3<128x128,3 terms split in the kernel,12 units x 235 workgroups,4 slabs,swiglu fold>",
        (B, X3, 1, 128, 2048, 5632): "rows_x3<128x128,3 terms split in the kernel,8 units x 176 workgroups,11 slabs,+residual in the fold>",
        (B, X3, 0, 128, 32000, 2048): "rows_x3<128x128,3 terms split in the kernel,32 units x 250 workgroups,1 slabs,no fold>",
        (B, X3, 0, 33, 2560, 2048): "rows_x3<128x128,3 terms split in the kernel,4 units x 160 workgroups,8 slabs,fold>",
        (B, X3, 0, 77, 8, 64): "rows_x3<128x128,3 terms split in the kernel,1 units x 1 workgroups,1 slabs,no fold>",
    }
    got = {key: _rows_plan(*key) for key in want}
    assert got == want
    # outside 33 .. 128 rows: planes through the register-staged kernel, and from a few hundred rows the one-wave-per-SIMD kernel
    assert _rows_plan(B, X3, 0, 32, 2560, 2048).startswith("gemm_tiled<bf16,NT,")
    assert _rows_plan(B, X3, 0, 200, 2560, 2048).startswith("gemm_tiled<bf16,NT,")
    assert _rows_plan(B, X3, 0, 1900, 2560, 2048).startswith("gemm_dma4<bf16,NT,") and "3 planes" in _rows_plan(B, X3, 0, 1900, 2560, 2048)
    assert _rows_plan(B, F32P, 0, 128, 2560, 2048) == "gemm_tiled<f32xbf16,NT,128x64,256t,splitK=6>"
    assert _rows_plan(F, F32P, 1, 128, 2048, 2048).startswith("gemm_tiled<f32,NT,")
    with pytest.raises(ug_amd.UgError):
        _rows_plan(F, X3, 0, 128, 2560, 2048)      # three terms need a bf16 matrix
    with pytest.raises(ug_amd.UgError):
        _rows_plan(B, X3, 0, 128, 2560, 2000)      # k % 64


def test_kernel_choice_for_the_baseline_shapes_is_pinned():
    """Which kernel, tile and K split a product gets follows from shapes and from cost models whose constants were fitted to
    measurements (gemm_dma_cost_us, gemm_tiled's pick_shape / pick_split).  The plans for BASELINE's products are written
    down here, so that a changed constant shows as a changed plan in a test that needs no GPU (the GPU suite then checks that
    ughip_matmul launches what the plan names: test_plan_names_what_is_launched)."""
    F, B = ug_amd.F32, ug_amd.BF16
    want = {
        # config 3: 8 x 1024^3, both rhs layouts
        (F, F, 8, 1024, 1024, 1024, 0): "gemm_dma_f32<f32,NN,256x128,320t>",
        (F, F, 8, 1024, 1024, 1024, 1): "gemm_tiled<f32,NT,256x128,512t>",
        (B, B, 8, 1024, 1024, 1024, 0): "gemm_dma4<bf16,NN,256x128,256t>",
        (B, B, 8, 1024, 1024, 1024, 1): "gemm_dma4<bf16,NT,256x128,256t>",
        # the large products the bench line carries
        (B, B, 1, 4096, 4096, 4096, 1): "gemm_dma4<bf16,NT,256x256,256t>",
        (B, B, 1, 4096, 4096, 4096, 0): "gemm_dma4<bf16,NN,256x256,256t>",
        (B, B, 1, 8192, 8192, 8192, 1): "gemm_dma4<bf16,NT,256x256,256t>",
        (B, B, 1, 3000, 4096, 4096, 1): "gemm_dma4<bf16,NT,256x256,256t>",
        # config 4: q k^T and att v at T = 512
        (F, F, 32, 512, 512, 64, 1): "gemm_tiled<f32,NT,256x128,512t>",
        (F, F, 32, 512, 64, 512, 0): "gemm_tiled<f32,NN,128x64,256t,splitK=2>",
        # config 5: decode projections (one row), single-query attention output, a 128-token prompt against bf16 matrices
        (F, F, 1, 1, 2048, 2048, 1): "gemv_nt<f32>",
        (F, F, 1, 1, 32000, 2048, 1): "gemv_nt<f32>",
        (F, F, 32, 1, 64, 1900, 0): "gemv_nn<f32>",
        (F, B, 1, 128, 2560, 2048, 1): "gemm_tiled<f32xbf16,NT,128x64,256t,splitK=6>",
        (F, B, 1, 128, 2048, 5632, 1): "gemm_tiled<f32xbf16,NT,128x64,256t,splitK=8>",
        (F, B, 1, 128, 32000, 2048, 1): "gemm_tiled<f32xbf16,NT,128x128,256t>",
        # mid-size 16-bit products where the two kernels are close
        (B, B, 1, 2048, 2048, 2048, 1): "gemm_tiled<bf16,NT,128x128,256t>",
        (B, B, 1, 2304, 2304, 2304, 1): "gemm_dma4<bf16,NT,128x128,256t>",
        (B, B, 1, 3072, 4096, 4096, 1): "gemm_dma4<bf16,NT,256x256,256t>",
        (F, F, 1, 100, 100, 100, 0): "gemm_any<f32>",
        # large f32 products: row-major rhs in whole rounds of tiles on the one-wave-per-SIMD kernel, the rest register-staged
        (F, F, 1, 4096, 4096, 4096, 0): "gemm_dma_f32<f32,NN,256x128,320t>",
        (F, F, 1, 4096, 4096, 4096, 1): "gemm_tiled<f32,NT,256x128,512t>",
        (F, F, 4, 2048, 2048, 2048, 0): "gemm_dma_f32<f32,NN,256x128,320t>",
    }
    got = {key: _plan(*key) for key in want}
    assert got == want
    with pytest.raises(ug_amd.UgError, match=r"\[n, k\]-major"):
        _plan(F, B, 1, 128, 2560, 2048, 0)
    with pytest.raises(ug_amd.UgError):
        _plan(ug_amd.I32, ug_amd.I32, 1, 8, 8, 8, 0)
    # f32 products as six bf16 terms: only with the switch, only where k % 64 == 0 and n % 8 == 0
    with ug_amd.tuning(MATMUL_X6=1):
        assert _plan(F, F, 8, 1024, 1024, 1024, 0) == "gemm_dma4<bf16,NN,256x128,256t,6 terms of 3 x 3 planes,f32 out>"
        assert _plan(F, F, 1, 4096, 4096, 4096, 1) == "gemm_dma4<bf16,NT,256x256,256t,6 terms of 3 x 3 planes,f32 out>"
        assert _plan(F, F, 1, 1024, 1020, 1024, 0) == "gemm_tiled<f32,NN,128x128,256t,ragged>" or "6 terms" not in _plan(F, F, 1, 1024, 1020, 1024, 0)
        assert "6 terms" not in _plan(F, F, 1, 1024, 1024, 1000, 1)
        assert "6 terms" not in _plan(B, B, 1, 4096, 4096, 4096, 1)
    assert "6 terms" not in _plan(F, F, 8, 1024, 1024, 1024, 0)
