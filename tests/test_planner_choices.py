"""Which kernel form and access width the planner picks for a shape, checked without a device (dry-run mode plans
and compiles, nothing executes).  The measurements behind each choice are in the planner's comments."""

import numpy as np
import pytest

import theano_amd as th
from theano_amd import hip, tensor as T


def _plan(dtype, shape, build, views=None):
    from theano_amd.hip import HipArray
    x = T.TensorType(dtype, (False,) * len(shape))("x")
    f = th.function([x], [th.Out(build(x), device=True)])
    a = HipArray.empty(shape, dtype)
    f(a if views is None else views(a))
    return hip.last_plan()


REDUCTIONS = [
    # odd lengths and alignments: full-width vectors through element-aligned pointers
    ("float32", (67108863,), None, ["|rr|", "|v4|", "|ua|"]),
    ("float16", (1000, 134217), 1, ["|rr|", "|v8|", "|ua|"]),
    ("int8", (268435455,), None, ["|rr|", "|v16|", "|ua|"]),
    ("float32", (2164802, 31), 0, ["|rc|", "|v4|", "|ua|"]),
    ("float32", (8192, 8192), 0, ["|rc|", "|v4|", "|x16|b512|"]),               # aligned: tall, narrow blocks
    ("float32", (67041, 1001), 0, ["|rc|", "|v4|", "|x64|b512|", "|ua|"]),       # rows off the cache lines: wide ones
    # few rows: one row lane up to seven rows
    ("float32", (2, 33554432), 0, ["|rc|", "|x256|", "|u2|"]),
    ("float32", (3, 22369621), 0, ["|rc|", "|x256|", "|u4|", "|ua|"]),
    ("float32", (7, 9586980), 0, ["|rc|", "|x256|", "|u8|"]),
    ("float32", (8, 8388608), 0, ["|rc|", "|x64|"]),
    # few columns: the strip form, except where whole vectors of columns do as well
    ("float32", (22369621, 3), 0, ["|rs|c3|", "|v4|"]),
    ("int8", (89478485, 3), 0, ["|rs|c3|", "|v16|"]),
    ("float16", (8388608, 16), 0, ["|rc|", "|v8|"]),
    ("float64", (2581110, 13), 0, ["|rc|"]),
    # few columns and few rows: one thread per result
    ("float32", (1048576, 4, 4, 4), 1, ["|rg|", "|t1|"]),
    # nothing to reduce (the reduced extent is 1): one row of the column form, in vectors
    ("float32", (1, 67108864), 0, ["|rc|", "|v4|", "|x256|"]),
    ("float16", (300001, 1), 1, ["|rc|", "|v8|", "|ua|"]),
    # at most 64 bytes of column accumulators per thread
    ("int8", (16384, 16384), 0, ["|rc|", "|v8|"]),
]


@pytest.mark.parametrize("dtype,shape,axis,marks", REDUCTIONS)
def test_reduction_plans(dry_run, dtype, shape, axis, marks):
    plan = _plan(dtype, shape, lambda x: T.sum(x, axis=axis))
    for m in marks:
        assert m in plan + "|", (shape, axis, plan)


def test_elementwise_plans(dry_run):
    from theano_amd.hip import HipArray
    # a view that starts one element in keeps 16-byte accesses
    plan = _plan("float16", (1000001,), lambda x: x * 2 + 1, views=lambda a: a.view([1000000], [2], a.offset + 2))
    assert "|ew|" in plan and "|v8|" in plan and "|ua|" in plan, plan
    # rows that are no whole number of vectors, beside a row that broadcasts
    m = T.TensorType("float32", (False, False))("m")
    row = T.TensorType("float32", (True, False))("row")
    f = th.function([m, row], [th.Out(m * 2 + row, device=True)])
    f(HipArray.empty((4096, 1001), "float32"), HipArray.empty((1, 1001), "float32"))
    assert "|v4|" in hip.last_plan() and "|ua|rg|" in hip.last_plan(), hip.last_plan()
    # operands that are all transposed the same way: the dimensions are walked in the result's order
    plan = _plan("float32", (4096, 4096), lambda x: T.tanh(x.T) + 1)
    assert "|ew|nd1|" in plan and "|v4|" in plan, plan
    # a permuted read beside two operands in the result's layout: 32 x 128 tiles; in the majority: square ones
    x, y = T.fmatrix("x"), T.fmatrix("y")
    f = th.function([x, y], [th.Out(x.T * 2 + y, device=True)])
    f(HipArray.empty((4096, 8192), "float32"), HipArray.empty((8192, 4096), "float32"))
    assert "|et|" in hip.last_plan() and "|t32x128|" in hip.last_plan(), hip.last_plan()
    f = th.function([x, y], [th.Out(x.T * y.T, device=True)])
    f(HipArray.empty((4096, 8192), "float32"), HipArray.empty((4096, 8192), "float32"))
    assert "|t32x128|" not in hip.last_plan(), hip.last_plan()


def test_row_chain_plans(dry_run):
    from theano_amd.hip import HipArray
    for dtype, vec in (("float32", 4), ("float16", 8)):
        x = T.TensorType(dtype, (False, False))("x")
        f = th.function([x], [th.Out(T.nnet.softmax(x), device=True)])
        f(HipArray.empty((4096, 1001), dtype))
        assert "|rw|v%d|" % vec in hip.last_plan() and "|ua|" in hip.last_plan(), hip.last_plan()
        f(HipArray.empty((4096, 1000), dtype))
        assert "|rw|v%d|" % vec in hip.last_plan() and "|ua|" not in hip.last_plan(), hip.last_plan()
