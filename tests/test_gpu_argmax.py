"""GPU parity of MaxAndArgmax / argmax / argmin against the oracle (NumPy's
first-occurrence rule, as MaxAndArgmax.perform): every kernel form, ties, NaNs,
integer and float16 values, split reductions, strided inputs."""

import numpy as np
import pytest

import theano_amd as th
from theano_amd import hip, tensor as T
from oracle import graph_ref as G

pytestmark = pytest.mark.gpu


def run(var, outs, val):
    got = th.function([var], outs)(val)
    ref = G.evaluate([var], outs, [val])
    return got, ref, hip.last_plan()


def same(got, ref, what):
    for g, r in zip(got, ref):
        assert g.dtype == r.dtype and g.shape == r.shape, (what, g.dtype, r.dtype, g.shape, r.shape)
        assert np.array_equal(g, r, equal_nan=True), what


CASES = [((7,), (0,)), ((300000,), (0,)), ((5, 6), (0,)), ((5, 6), (1,)), ((5, 6), (0, 1)), ((3, 4100), (1,)),
         ((4100, 3), (0,)), ((1025, 1025), (0,)), ((1025, 1025), (1,)), ((1025, 1025), (0, 1)), ((33, 65, 17), (0,)),
         ((33, 65, 17), (1,)), ((33, 65, 17), (2,)), ((33, 65, 17), (0, 1)), ((33, 65, 17), (0, 2)), ((33, 65, 17), (1, 2)),
         ((33, 65, 17), (0, 1, 2)), ((5, 7, 9, 11), (0, 2)), ((5, 7, 9, 11), (1, 3)), ((5, 7, 9, 11), (0, 1, 3)),
         ((3, 4, 5, 6, 7), (0, 2, 4)), ((64, 8, 49), (0, 2)), ((2, 70000), (1,)), ((70000, 2), (0,))]


@pytest.mark.parametrize("shape,axes", CASES)
def test_shapes_axes_with_ties(shape, axes):
    rng = np.random.default_rng(31)
    x = T.TensorType("float32", (False,) * len(shape))("x")
    val = rng.integers(-3, 4, shape).astype("float32")            # few distinct values: ties everywhere
    got, ref, plan = run(x, T.max_and_argmax(x, axis=list(axes)), val)
    same(got, ref, "ties %s %s [%s]" % (shape, axes, plan))
    val = rng.standard_normal(shape).astype("float32")
    got, ref, plan = run(x, T.max_and_argmax(x, axis=list(axes), keepdims=True), val)
    same(got, ref, "normal %s %s [%s]" % (shape, axes, plan))


def test_nan_is_the_maximum_and_first_nan_wins():
    x = T.fmatrix("x")
    val = np.random.default_rng(32).standard_normal((64, 3000)).astype("float32")
    val[3, 2000] = np.nan
    val[3, 100] = np.nan
    val[10, 2999] = np.nan
    val[20, :] = -np.inf
    val[21, :] = np.inf
    val[30, :] = -1.0
    val[30, 1500] = 0.0                       # +0 after -0: equal values, the first one is the argmax
    val[30, 700] = -0.0
    for ax in (0, 1, None):
        got, ref, plan = run(x, T.max_and_argmax(x, axis=ax), val)
        same(got, ref, "nan axis %s [%s]" % (ax, plan))


@pytest.mark.parametrize("dtype", ["bool", "int8", "uint8", "int16", "int32", "uint32", "int64", "uint64", "float16",
                                   "float64"])
def test_dtypes_and_argmin(dtype):
    rng = np.random.default_rng(33)
    x = T.TensorType(dtype, (False, False))("x")
    if dtype == "bool":
        val = rng.integers(0, 2, (37, 513)).astype("bool")
    elif dtype.startswith("float"):
        val = rng.integers(-50, 50, (37, 513)).astype(dtype)
    else:
        info = np.iinfo(dtype)
        val = rng.integers(info.min // 2, info.max // 2, (37, 513)).astype(dtype)
        val[5, 7] = info.max
        val[6, 9] = info.min
    for ax in (0, 1, None):
        got, ref, plan = run(x, T.max_and_argmax(x, axis=ax), val)
        same(got, ref, "%s axis %s [%s]" % (dtype, ax, plan))
        got, ref, plan = run(x, [T.argmin(x, axis=ax), T.argmax(x, axis=ax, keepdims=True)], val)
        same(got, ref, "%s argmin axis %s [%s]" % (dtype, ax, plan))
        if not dtype.startswith("int"):       # -x wraps for the most negative signed integer, as in the reference
            assert np.array_equal(got[0], np.argmin(val, axis=ax))


def test_strided_views_zero_extents_and_errors():
    rng = np.random.default_rng(34)
    x = T.ftensor3("x")
    val = rng.integers(-2, 3, (9, 40, 21)).astype("float32")
    outs = T.max_and_argmax(x.dimshuffle(2, 0, 1), axis=[0, 2])
    got, ref, plan = run(x, outs, val)
    same(got, ref, "dimshuffled [%s]" % plan)
    m = T.fmatrix("m")
    f = th.function([m], T.max_and_argmax(m, axis=1))
    mv, iv = f(np.zeros((0, 4), "float32"))                    # theano/tensor/tests/test_basic.py:3314-3321
    assert mv.shape == (0,) and iv.shape == (0,) and iv.dtype == np.int64
    with pytest.raises(ValueError):
        f(np.zeros((4, 0), "float32"))
    # the reference's literal cases (test_basic.py:3114-3119, 3304-3309)
    v = T.lvector("v")
    mv, iv = th.function([v], T.max_and_argmax(v))(np.array([1, 2, 3, 2, -6]))
    assert mv == 3 and iv == 2 and iv.dtype == np.int64
    t = T.ltensor3("t")
    mv, iv = th.function([t], T.max_and_argmax(t, [1, -1]))(np.arange(24).reshape(3, 2, 4))
    assert np.array_equal(mv, [7, 15, 23]) and np.array_equal(iv, [7, 7, 7])


def test_lowest_values_everywhere_and_walks_that_do_not_follow_positions():
    """A thread keeps the first of equal values without comparing positions where positions only grow along its walk;
    where they do not (reduced dimensions of a transposed view, walked by stride) the full rule applies.  An
    accumulator that nothing ever beat - every element is the lowest value of its type - answers position 0."""
    rng = np.random.default_rng(37)
    for dtype, low in (("int8", -128), ("uint8", 0), ("int32", -2 ** 31), ("float32", -np.inf), ("float16", -np.inf)):
        m = T.TensorType(dtype, (False, False))("m")
        val = np.full((70, 5000), low, dtype)
        val[5, 4000:] = 1                                   # one row with something above the lowest value
        for ax in (0, 1, None):
            got, ref, plan = run(m, T.max_and_argmax(m, axis=ax), val)
            same(got, ref, "all lowest %s axis %s [%s]" % (dtype, ax, plan))
    t = T.ftensor3("t")
    val = rng.integers(-2, 3, (37, 41, 43)).astype("float32")
    for order in ((2, 1, 0), (1, 0, 2), (0, 2, 1), (2, 0, 1)):
        for axes in ((0, 1), (1, 2), (0, 2), (0, 1, 2), (1,)):
            out = T.max_and_argmax(t.dimshuffle(*order), axis=list(axes))
            got, ref, plan = run(t, out, val)
            same(got, ref, "transposed %s axes %s [%s]" % (order, axes, plan))


def test_argmax_through_the_generic_reduction_form():
    """Three reduced dimensions that do not collapse (axes 0, 2, 4 of a 6-d array) take the generic
    kernel, where the position operand is computed from a full index decomposition; ties and NaNs included."""
    rng = np.random.default_rng(36)
    t6 = T.TensorType("float32", (False,) * 6)("t6")
    val = rng.integers(-3, 4, (3, 4, 5, 6, 7, 2)).astype("float32")      # many ties: the first occurrence must win
    val[1, 2, 3, 4, 5, 1] = np.nan
    f = th.function([t6], T.max_and_argmax(t6, axis=(0, 2, 4)))
    mv, iv = f(val)
    assert "|rg|" in hip.last_plan(), hip.last_plan()
    ref_m, ref_i = G.max_and_argmax(val, (0, 2, 4))
    assert np.array_equal(mv, ref_m, equal_nan=True) and np.array_equal(iv, ref_i) and iv.dtype == np.int64
    i6 = T.TensorType("int16", (False,) * 6)("i6")
    vi = rng.integers(-300, 300, (3, 4, 5, 6, 7, 2)).astype("int16")
    mv, iv = th.function([i6], T.max_and_argmax(i6, axis=(0, 2, 4)))(vi)
    ref_m, ref_i = G.max_and_argmax(vi, (0, 2, 4))
    assert np.array_equal(mv, ref_m) and np.array_equal(iv, ref_i)


def test_gradient_of_max_through_max_and_argmax():
    rng = np.random.default_rng(35)
    x = T.fmatrix("x")
    val = rng.standard_normal((50, 70)).astype("float32")
    m, a = T.max_and_argmax(x, axis=1)
    g = th.grad(T.sum(m * m), x)
    got = th.function([x], [g, a])(val)
    ref = np.zeros_like(val)
    idx = np.argmax(val, axis=1)
    ref[np.arange(50), idx] = 2 * val[np.arange(50), idx]
    assert np.allclose(got[0], ref, rtol=1e-6) and np.array_equal(got[1], idx)


def test_full_size_argmax_of_config2_matrix():
    import workloads as W
    (val,) = W.c2_inputs("max_axis1", "full")
    x = T.fmatrix("x")
    f = th.function([x], T.max_and_argmax(x, axis=1) + T.max_and_argmax(x, axis=0) + T.max_and_argmax(x))
    m1, a1, m0, a0, ma, aa = f(val)
    assert np.array_equal(a1, np.argmax(val, axis=1)) and np.array_equal(m1, val.max(axis=1))
    assert np.array_equal(a0, np.argmax(val, axis=0)) and np.array_equal(m0, val.max(axis=0))
    assert aa == np.argmax(val) and ma == val.max()
