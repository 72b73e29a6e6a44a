"""Lazy graphs of the BASELINE configs as ug's own code builds them, for bench.py, smoke() and the tests."""
from .api import LazyBuffer as LB


def fused_reduce_graph(a, b, dev):
    """Config 2: ((a*b) + (a*0.5)).reduce(Sum, 0).narrow(0, 0, 1); the tensor operand stays on the
    left so the result keeps its shape (op::binary takes the lhs shape, ug-core/src/lang.rs:507-520), and the
    narrow turns the shape-keeping reduce (lazy_buffer.rs:453-467) into a one-element store."""
    n = a.dims()[0]
    half = LB.cst(0.5, (n,), dev)
    return a.binary("mul", b).binary("add", a.binary("mul", half)).reduce("sum", 0).narrow(0, 0, 1)
