"""Pins the oracle's five ug-llama ops (oracle/cpu_ops.cpp, the restatement of ug-llama/src/cpu_ops.rs:6-167) on
the CPU alone, each against an independent float64 numpy statement of the formula and against what the
mathematics fixes: rotations keep pair norms, position 0 is the identity, the two rope layouts are one
permutation apart, the mask is idempotent and lower-triangular, softmax rows sum to one and do not move under a
shift, cat is a pure gather.  A dropped term, a wrong sign, a swapped pair index or a wrong table row fails
one of them."""
import numpy as np
import pytest

import ug_amd
from ug_amd import LazyBuffer as LB, rng

EPS32 = float(np.finfo(np.float32).eps)


def _tables(max_pos, d, seed=3):
    """Arbitrary (not cos/sin of anything) tables: the op must use exactly the entries the formula names."""
    c = rng.uniform_pm1(seed, max_pos * (d // 2)).reshape(max_pos, d // 2)
    s = rng.uniform_pm1(seed + 1, max_pos * (d // 2)).reshape(max_pos, d // 2)
    return c, s


def _rope(cpu, cpu_ops, x, c, s, pos0, interleaved):
    b, h, t, d = x.shape
    f = cpu_ops.rope_i if interleaved else cpu_ops.rope
    out = f(LB.copy(x, x.shape, cpu), LB.copy(c, c.shape, cpu), LB.copy(s, s.shape, cpu), LB.copy(np.array([pos0], np.int32), (1,), cpu))
    return out.data_vec().reshape(x.shape)


@pytest.mark.parametrize("b,h,t,d,pos0", [(1, 4, 1, 64, 0), (1, 4, 1, 64, 17), (2, 3, 7, 6, 2), (1, 2, 5, 10, 11), (1, 32, 3, 64, 40)])
def test_rope_pairs_i_and_i_plus_half(cpu, cpu_ops, b, h, t, d, pos0):
    """cpu_ops.rs:91-126: x1 = x[i], x2 = x[i + d/2], table row pos[0] + i_t, column i."""
    x = rng.normal(5, b * h * t * d).reshape(b, h, t, d)
    c, s = _tables(pos0 + t + 3, d)
    got = _rope(cpu, cpu_ops, x, c, s, pos0, False)
    x64, c64, s64 = x.astype(np.float64), c[pos0:pos0 + t].astype(np.float64), s[pos0:pos0 + t].astype(np.float64)
    x1, x2 = x64[..., :d // 2], x64[..., d // 2:]
    want = np.concatenate([x1 * c64 - x2 * s64, x1 * s64 + x2 * c64], -1)
    np.testing.assert_allclose(got, want, rtol=0, atol=4 * EPS32 * float(np.abs(x).max()))


@pytest.mark.parametrize("b,h,t,d,pos0", [(1, 4, 1, 64, 0), (1, 4, 1, 64, 17), (2, 3, 7, 6, 2), (1, 2, 5, 10, 11)])
def test_rope_i_pairs_2i_and_2i_plus_1(cpu, cpu_ops, b, h, t, d, pos0):
    """cpu_ops.rs:58-89: x1 = x[2i], x2 = x[2i + 1]; the table index is the flat pair index inside the t*d chunk
    offset by pos[0]*d/2 -- i.e. row pos[0] + i_t, column i, as for rope."""
    x = rng.normal(6, b * h * t * d).reshape(b, h, t, d)
    c, s = _tables(pos0 + t + 3, d)
    got = _rope(cpu, cpu_ops, x, c, s, pos0, True)
    x64, c64, s64 = x.astype(np.float64), c[pos0:pos0 + t].astype(np.float64), s[pos0:pos0 + t].astype(np.float64)
    x1, x2 = x64[..., 0::2], x64[..., 1::2]
    want = np.empty_like(x64)
    want[..., 0::2] = x1 * c64 - x2 * s64
    want[..., 1::2] = x1 * s64 + x2 * c64
    np.testing.assert_allclose(got, want, rtol=0, atol=4 * EPS32 * float(np.abs(x).max()))


@pytest.mark.parametrize("interleaved", [False, True])
def test_rope_invariants_with_true_rotations(cpu, cpu_ops, interleaved):
    """With cos/sin of real angles every pair keeps its norm, position 0 of a table whose first row is angle 0 is the
    identity, and rope / rope_i agree after the permutation that interleaves the two halves."""
    b, h, t, d, pos0 = 1, 3, 6, 8, 2
    ang = rng.uniform_pm1(9, (pos0 + t) * (d // 2)).reshape(-1, d // 2).astype(np.float64) * 3.0
    ang[0] = 0.0
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    x = rng.normal(7, b * h * t * d).reshape(b, h, t, d)
    got = _rope(cpu, cpu_ops, x, c, s, pos0, interleaved)
    if interleaved:
        n_in, n_out = x[..., 0::2] ** 2 + x[..., 1::2] ** 2, got[..., 0::2] ** 2 + got[..., 1::2] ** 2
    else:
        n_in, n_out = x[..., :d // 2] ** 2 + x[..., d // 2:] ** 2, got[..., :d // 2] ** 2 + got[..., d // 2:] ** 2
    np.testing.assert_allclose(n_out, n_in, rtol=1e-5)
    at0 = _rope(cpu, cpu_ops, x[:, :, :1], c, s, 0, interleaved)
    np.testing.assert_array_equal(at0, x[:, :, :1])
    # rope on the de-interleaved vector == de-interleaved rope_i
    perm = np.concatenate([np.arange(0, d, 2), np.arange(1, d, 2)])
    a = _rope(cpu, cpu_ops, np.ascontiguousarray(x[..., perm]), c, s, pos0, False)
    bi = _rope(cpu, cpu_ops, x, c, s, pos0, True)
    np.testing.assert_array_equal(a, bi[..., perm])


@pytest.mark.parametrize("shape_l,shape_r,axis", [((1, 4, 0, 64), (1, 4, 5, 64), 2), ((1, 4, 7, 64), (1, 4, 1, 64), 2), ((2, 3), (2, 5), 1),
                                                  ((2, 3), (4, 3), 0), ((2, 3, 4), (2, 3, 1), 2), ((2, 1, 4), (2, 6, 4), 1)])
def test_cat_is_numpy_concatenate(cpu, cpu_ops, shape_l, shape_r, axis):
    """cpu_ops.rs:128-167: two [d1, d2] views copied side by side, bit for bit."""
    l = rng.normal(13, int(np.prod(shape_l))).reshape(shape_l)
    r = rng.normal(14, int(np.prod(shape_r))).reshape(shape_r)
    got = cpu_ops.cat(LB.copy(l, shape_l, cpu), LB.copy(r, shape_r, cpu), axis)
    want = np.concatenate([l, r], axis)
    assert tuple(got.dims()) == want.shape
    np.testing.assert_array_equal(got.data_vec().reshape(want.shape), want)


@pytest.mark.parametrize("shape", [(1, 32, 16, 16), (2, 3, 5, 5), (1, 1, 7, 7), (1, 2, 64, 64)])
def test_causal_mask_keeps_the_lower_triangle(cpu, cpu_ops, shape):
    """cpu_ops.rs:33-56: element (i1, i2) survives iff i2 <= i1, everything else is -inf; applying it twice changes nothing."""
    x = rng.normal(15, int(np.prod(shape))).reshape(shape)
    once = cpu_ops.causal_mask(LB.copy(x, shape, cpu)).data_vec().reshape(shape)
    keep = np.arange(shape[-1])[None, :] <= np.arange(shape[-2])[:, None]
    np.testing.assert_array_equal(once, np.where(keep, x, np.float32(-np.inf)))
    twice = cpu_ops.causal_mask(LB.copy(once, shape, cpu)).data_vec().reshape(shape)
    np.testing.assert_array_equal(twice, once)


@pytest.mark.parametrize("shape", [(1, 32, 1, 129), (1, 4, 16, 16), (2, 2, 33, 300), (1, 1, 3, 1024)])
def test_custom_softmax_against_float64(cpu, cpu_ops, shape):
    """cpu_ops.rs:6-31: max, exp(x - max), sum in index order, divide.  Float64 statement to 1e-5 (2e-6 observed), rows
    sum to one, a shift of the row changes nothing beyond rounding, and masked (-inf) entries come out as exact zeros."""
    x = rng.normal(16, int(np.prod(shape)), 3.0).reshape(shape)
    got = cpu_ops.custom_softmax(LB.copy(x, shape, cpu)).data_vec().reshape(shape)
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(-1, keepdims=True))
    np.testing.assert_allclose(got, e / e.sum(-1, keepdims=True), rtol=1e-5, atol=1e-30)
    np.testing.assert_allclose(got.astype(np.float64).sum(-1), 1.0, rtol=0, atol=1e-5)
    shifted = cpu_ops.custom_softmax(LB.copy(x + np.float32(8.0), shape, cpu)).data_vec().reshape(shape)
    np.testing.assert_allclose(shifted, got, rtol=2e-5, atol=1e-30)
    xm = x.copy()
    xm[..., shape[-1] // 2:] = -np.inf
    gm = cpu_ops.custom_softmax(LB.copy(xm, shape, cpu)).data_vec().reshape(shape)
    assert not gm[..., shape[-1] // 2:].any()
    np.testing.assert_allclose(gm.astype(np.float64).sum(-1), 1.0, rtol=0, atol=1e-5)


def test_mask_then_softmax_row_zero_is_one_hot(cpu, cpu_ops):
    """The composition model.rs:236-242 uses: the first query sees only key 0."""
    shape = (1, 2, 9, 9)
    x = rng.normal(17, int(np.prod(shape))).reshape(shape)
    p = cpu_ops.custom_softmax(cpu_ops.causal_mask(LB.copy(x, shape, cpu))).data_vec().reshape(shape)
    np.testing.assert_array_equal(p[..., 0, :], np.broadcast_to(np.eye(9, dtype=np.float32)[0], (1, 2, 9)))
    assert np.all(np.triu(p, 1) == 0)
