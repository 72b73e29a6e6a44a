"""The reference's own lazy-buffer tests (ug-core/tests/lb_tests.rs, ug-core/src/common_tests.rs),
written once and run against any device: the CPU oracle (CPU suite) and the HIP device (GPU suite).
Expected values come from tests/golden/reference_vectors.json."""
import json
import os

import numpy as np

import ug_amd
from ug_amd import F32, LazyBuffer as LB, Schedule

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))


def f32(x):
    return np.asarray(x, dtype=np.float32)


def eq(a, b):
    np.testing.assert_array_equal(np.asarray(a, dtype=np.float32), f32(b))


# common_tests.rs:6-13
def lb_add(dev):
    lhs = LB.cst(40.0, (5, 2), dev)
    rhs = LB.cst(2.0, (5, 2), dev)
    lb = lhs.binary("add", rhs)
    eq(lb.data_vec(), GOLD["lb_add"]["expect"])


# common_tests.rs:15-22
def lb_mm(dev):
    lhs = LB.cst(1.0, (4, 2), dev)
    rhs = LB.cst(2.0, (2, 3), dev)
    eq(lhs.matmul(rhs).data_vec(), GOLD["lb_mm"]["expect"])


# common_tests.rs:24-34 (dim 1 pins the contiguous-per-argument layout and zero-filled allocation)
def lb_cat(dev):
    g = GOLD["lb_cat"]
    args = [LB.copy(f32(g[k]), (2, 2), dev) for k in ("arg0", "arg1", "arg2")]
    eq(LB.cat(args, 0).data_vec(), g["expect_dim0"])
    eq(LB.cat(args, 1).data_vec(), g["expect_dim1"])


# lb_tests.rs:5-49: one schedule item for 40 + 2
def schedule_one_item(dev):
    lb = LB.cst(40.0, (5, 2), dev).binary("add", LB.cst(2.0, (5, 2), dev))
    s = Schedule.create_one(lb)
    items = s.items()
    assert len(items) == 1 and items[0]["kind"] == "kernel"
    return s


# lb_tests.rs:66-97: a compiled schedule can be re-run after its input changed
def lb_copy(dev):
    g = GOLD["lb_copy"]
    lhs = LB.copy(f32(g["input"]), (2, 3), dev)
    lb = lhs.binary("add", LB.cst(2.0, (2, 3), dev)).binary("mul", LB.cst(0.5, (2, 3), dev))
    cs = Schedule.create_one(lb).compile()
    cs.run()
    eq(lb.data_vec(), g["expect"])
    data = f32(g["input"])
    for k, v in g["poke"].items():
        data[int(k)] = v
    lhs.write(data)
    cs.run()
    eq(lb.data_vec(), g["expect_after"])


# lb_tests.rs:99-109
def schedule_broadcast(dev):
    rhs = LB.cst(2.0, (), dev).broadcast((5, 2))
    lb = LB.cst(40.0, (5, 2), dev).binary("add", rhs)
    eq(lb.data_vec(), GOLD["lb_add"]["expect"])


def _add_one(slices):
    src, dst = slices
    dst.copy_host_to_device(src.to_vec() + np.float32(1.0))


# lb_tests.rs:111-149
def lb_custom(dev):
    g = GOLD["lb_custom"]
    buf = LB.copy(f32([0, 1, 2, 3, 4, 5]), (2, 3), dev)
    lb = LB.custom(_add_one, [buf], (2, 3), F32, dev).binary("mul", LB.cst(2.0, (2, 3), dev))
    cs = Schedule.create_one(lb).compile()
    cs.run()
    eq(lb.data_vec(), g["expect"])
    buf.write(f32([0, 0, -8, 3, 4, -2]))
    cs.run()
    eq(lb.data_vec(), g["expect_after"])


# lb_tests.rs:151-172
def lb_layout(dev):
    g = GOLD["lb_layout"]
    lb = LB.copy(f32([0, 1, 2, 3, 4, 5]), (2, 3), dev)
    t = lb.transpose(0, 1)
    eq(t.data_vec(), g["transposed"])
    m = t.transpose(0, 1).merge_dims(0)
    assert m.dims() == [6]
    eq(m.data_vec(), g["merged"])


# lb_tests.rs:174-205: in-place ops re-run on every realize
def lb_custom_in_place(dev):
    g = GOLD["lb_custom_in_place"]

    def add_one(slices):
        (dst,) = slices
        dst.copy_host_to_device(dst.to_vec() + np.float32(1.0))

    lb = LB.copy(f32([0, 1, 2, 3, 4, 5]), (2, 3), dev)
    lb = lb.custom_ip(add_one).custom_ip(add_one).custom_ip(add_one)
    eq(lb.data_vec(), g["expect"])
    lb.write(f32([3, 0, -8, 6, 7, -2]))
    eq(lb.data_vec(), g["expect_after"])


# lb_tests.rs:207-229
def lb_set(dev):
    g = GOLD["lb_set"]
    dst = LB.copy(f32([0, 1, 2, 3, 4, 5]), (2, 3), dev)
    src = dst.binary("mul", dst)
    eq(src.data_vec(), g["squares"])
    eq(dst.data_vec(), [0, 1, 2, 3, 4, 5])
    dst2 = dst.set(src)
    eq(dst2.data_vec(), g["squares"])
    vs = LB.copy(f32([3, 1, 2]), (3,), dev)
    dst3 = dst2.set_l(vs, (3,))
    eq(dst3.data_vec(), g["after_set_l"])


ALL = [lb_add, lb_mm, lb_cat, schedule_one_item, lb_copy, schedule_broadcast, lb_custom, lb_layout, lb_custom_in_place, lb_set]


# ---- the benchmark workloads as lazy graphs ---------------------------------------------------------------
def softmax_graph(src):
    """ug-llama/src/model.rs:94-101 == config 1: max-reduce, subtract, exp, sum-reduce, divide."""
    return ug_amd.llama.softmax(src)


from ug_amd.graphs import fused_reduce_graph  # noqa: E402,F401  (config 2; shared with bench.py and smoke())
