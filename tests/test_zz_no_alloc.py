"""ughip_matmul_noalloc -- ughip_matmul for callers that cannot allocate: same kernels, the split-K partial tiles in a
static device array instead of a block grown with hipMalloc.  Called straight through the C ABI and held bit for bit
to ughip_matmul on the same operands, two calls in a row with the second one smaller (the array keeps the first
call's partial tiles), then on the other kernel families, which use no scratch at all."""
import ctypes as C
import os

import numpy as np
import pytest

import ug_amd
from ug_amd import rng

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 64 << 20      # UGHIP_MATMUL_NOALLOC_SCRATCH_BYTES of include/ughip.h


def _sizes(v):
    return (C.c_size_t * len(v))(*v)


def _call(entry, hip, dst, sa, sw, b, m, n, k, rhs_nk):
    lib = ug_amd.ughip_lib()
    fn = getattr(lib, entry)
    fn.restype = C.c_int
    raw = lambda s: C.c_void_p(s.raw())  # noqa: E731
    lhs_d, lhs_s = _sizes((b, m, k)), _sizes((m * k, k, 1))
    rhs_d, rhs_s = _sizes((b, k, n)), _sizes((k * n, 1, k) if rhs_nk else (k * n, n, 1))
    rc = fn(C.c_void_p(hip.raw_hip()), raw(dst), raw(sa), raw(sw), C.c_size_t(b), C.c_size_t(m), C.c_size_t(n), C.c_size_t(k), C.c_size_t(3),
            lhs_d, lhs_s, C.c_size_t(0), rhs_d, rhs_s, C.c_size_t(0))
    return rc, lib.ughip_last_error().decode(), ug_amd.last_kernel()


def _both(hip, dtype, bmnk, rhs_nk, seed):
    """The product through ughip_matmul and through ughip_matmul_noalloc; returns (reference result, no-alloc result, kernel)."""
    b, m, n, k = bmnk
    a = rng.uniform_pm1(seed, b * m * k)
    w = rng.uniform_pm1(seed + 1, b * k * n)
    enc = rng.to_bf16_bits if dtype == ug_amd.BF16 else (lambda v: v)
    sa, sw = hip.slice_from(enc(a)), hip.slice_from(enc(w))
    outs = []
    for entry in ("ughip_matmul", "ughip_matmul_noalloc"):
        dst = hip.slice_from(enc(np.full(b * m * n, 7.0, np.float32)))
        rc, err, kernel = _call(entry, hip, dst, sa, sw, b, m, n, k, rhs_nk)
        assert rc == 0, err
        outs.append((dst.to_vec(), kernel))
    assert outs[0][1] == outs[1][1]
    # and the product is right, not merely the same twice
    got = rng.from_bf16_bits(outs[1][0]) if dtype == ug_amd.BF16 else outs[1][0]
    a64 = (rng.bf16_round(a) if dtype == ug_amd.BF16 else a).astype(np.float64).reshape(b, m, k)
    w64 = (rng.bf16_round(w) if dtype == ug_amd.BF16 else w).astype(np.float64)
    w64 = np.swapaxes(w64.reshape(b, n, k), 1, 2) if rhs_nk else w64.reshape(b, k, n)
    exact = a64 @ w64
    bound = k * float(np.finfo(np.float32).eps) * (np.abs(a64) @ np.abs(w64)) + (2.0 ** -8 * np.abs(exact) if dtype == ug_amd.BF16 else 0.0)
    assert np.all(np.abs(got.reshape(b, m, n) - exact) <= bound * 1.001 + 1e-12)
    return outs[0][0], outs[1][0], outs[1][1]


def test_noalloc_split_k_twice_the_second_call_smaller(hip):
    """128-token prefill projections: K split over 12-16 workgroups per tile, partial tiles in the static array.  The
    second product is smaller and runs over what the first one left there."""
    for dtype, name in ((ug_amd.F32, "f32"), (ug_amd.BF16, "bf16")):
        for rhs_nk in (True, False):
            big = _both(hip, dtype, (1, 128, 2048, 2048), rhs_nk, 81)
            small = _both(hip, dtype, (1, 128, 256, 2048), rhs_nk, 83)
            print("noalloc", name, "NT" if rhs_nk else "NN", big[2], "then", small[2], flush=True)
            assert "splitK=" in big[2] and "splitK=" in small[2]
            np.testing.assert_array_equal(big[1], big[0])
            np.testing.assert_array_equal(small[1], small[0])
            # once more the large one: nothing the small call left behind shows
            again = _both(hip, dtype, (1, 128, 2048, 2048), rhs_nk, 81)
            np.testing.assert_array_equal(again[1], big[0])


@pytest.mark.parametrize("bmnk,rhs_nk", [((2, 100, 2048, 2048), True), ((1, 128, 11264, 2048), True), ((1, 37, 5632, 256), True), ((8, 256, 256, 64), False),
                                         ((1, 1, 2048, 2048), True), ((32, 1, 64, 129), False), ((2, 130, 70, 50), False)])
def test_noalloc_other_shapes_match(hip, bmnk, rhs_nk):
    """Ragged split-K tiles, the stacked gate|up product of a prefill (the largest partial-tile block of config 5:
    29 MB), unsplit tiles, both GEMV families and the any-stride kernel."""
    ref, got, kernel = _both(hip, ug_amd.F32, bmnk, rhs_nk, 85)
    print("noalloc", bmnk, kernel, flush=True)
    np.testing.assert_array_equal(got, ref)


def test_noalloc_refuses_what_does_not_fit(hip, tune):
    """A forced 32-way split of a 1024 x 1024 result needs 128 MiB of partial tiles: refused with both sizes in the
    message and nothing launched; ughip_matmul takes the same call."""
    b, m, n, k = 1, 1024, 1024, 4096
    tune.setenv("UGHIP_GEMM_SHAPE", "1")
    tune.setenv("UGHIP_GEMM_SPLIT", "32")
    sa, sw = hip.slice_from(np.ones(m * k, np.float32)), hip.slice_from(np.ones(k * n, np.float32))
    dst = hip.slice_from(np.full(m * n, 7.0, np.float32))
    rc, err, _ = _call("ughip_matmul_noalloc", hip, dst, sa, sw, b, m, n, k, True)
    assert rc != 0
    assert str(32 * m * n * 4) in err and str(SCRATCH_BYTES) in err and "ughip_matmul" in err, err
    assert np.all(dst.to_vec() == 7.0)
    rc, err, kernel = _call("ughip_matmul", hip, dst, sa, sw, b, m, n, k, True)
    assert rc == 0, err
    assert "splitK=32" in kernel
    assert np.all(dst.to_vec() == float(k))
    # errors of the shared argument checks come through unchanged
    rc, err, _ = _call("ughip_matmul_noalloc", hip, dst, sa, sw, b, m, n, 2 * k, True)
    assert rc != 0 and "too short" in err
