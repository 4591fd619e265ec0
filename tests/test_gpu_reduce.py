"""GPU parity of CAReduce against the oracle over shapes, masks, ops and dtypes."""

import numpy as np
import pytest

import theano_amd as th
from theano_amd import hip, tensor as T
from oracle import graph_ref as G
from conftest import assert_parity, assert_within_reference_error
from test_oracle_graph import CAREDUCE_CASES

pytestmark = pytest.mark.gpu

REDUCERS = {"sum": lambda v, ax: v.sum(axis=ax), "prod": lambda v, ax: v.prod(axis=ax),
            "max": lambda v, ax: v.max(axis=ax), "min": lambda v, ax: v.min(axis=ax)}


def check(var, out, val, what, tol=None):
    got = th.function([var], out)(val)
    ref = G.evaluate([var], [out], [val])[0]
    assert_parity(got, ref, what + " [" + hip.last_plan() + "]", tol=tol)


@pytest.mark.parametrize("shape,axis", CAREDUCE_CASES)
def test_reference_case_table(shape, axis):
    rng = np.random.default_rng(21)
    xf = T.TensorType("float32", (False,) * len(shape))("x")
    xi = T.TensorType("int32", (False,) * len(shape))("x")
    vf = rng.standard_normal(shape).astype("float32")
    vi = rng.integers(-4, 5, shape).astype("int32")
    zero = any(shape[a] == 0 for a in (range(len(shape)) if axis is None else axis))
    for name, fn in REDUCERS.items():
        if zero and name in ("max", "min"):
            with pytest.raises(ValueError):
                th.function([xf], fn(xf, axis))(vf)
            continue
        check(xf, fn(xf, axis), vf, "%s f32 %s %s" % (name, shape, axis))
        check(xi, fn(xi, axis), vi, "%s i32 %s %s" % (name, shape, axis))
    check(xi, T.any(xi > 0, axis=axis), vi, "any")
    check(xi, T.all(xi > -4, axis=axis), vi, "all")


# shape x reduce-mask patterns in the spirit of theano/gpuarray/tests/test_elemwise.py:262-346,
# including extents above 4096 and degenerate extents
MASK_CASES = [((4100, 3), [1, 0]), ((3, 4100), [0, 1]), ((4100, 3), [0, 1]), ((3, 4100), [1, 0]), ((5000,), [1]),
              ((1, 5000), [0, 1]), ((33, 1, 65), [1, 0, 1]), ((33, 65, 17), [0, 1, 0]), ((33, 65, 17), [1, 0, 1]),
              ((33, 65, 17), [1, 1, 0]), ((33, 65, 17), [0, 1, 1]), ((33, 65, 17), [1, 0, 0]), ((33, 65, 17), [0, 0, 1]),
              ((5, 7, 9, 11), [1, 0, 1, 0]), ((5, 7, 9, 11), [0, 1, 0, 1]), ((5, 7, 9, 11), [1, 0, 0, 1]),
              ((5, 7, 9, 11), [0, 1, 1, 0]), ((5, 7, 9, 11), [1, 1, 1, 1]), ((5, 7, 9, 11), [1, 0, 1, 1]),
              ((3, 4, 5, 6, 7), [1, 0, 1, 0, 1]), ((3, 4, 5, 6, 7, 2), [1, 0, 1, 0, 1, 0]), ((2, 3, 4, 5, 6, 7, 2, 3), [0, 1] * 4),
              ((1025, 1025), [1, 0]), ((1025, 1025), [0, 1]), ((1025, 1025), [1, 1]), ((70000, 2), [1, 0]),
              ((2, 70000), [0, 1]), ((300000,), [1]), ((64, 8, 49), [1, 0, 1])]


@pytest.mark.parametrize("shape,mask", MASK_CASES)
def test_shapes_and_masks(shape, mask):
    rng = np.random.default_rng(22)
    axis = tuple(d for d, m in enumerate(mask) if m)
    x = T.TensorType("float32", (False,) * len(shape))("x")
    v = rng.standard_normal(shape).astype("float32")
    check(x, x.sum(axis=axis), v, "sum %s %s" % (shape, mask))
    check(x, x.max(axis=axis), v, "max %s %s" % (shape, mask))
    xi = T.TensorType("int16", (False,) * len(shape))("xi")
    vi = rng.integers(-300, 300, shape).astype("int16")
    check(xi, xi.sum(axis=axis), vi, "int16 sum %s %s" % (shape, mask))


def _reference_gpu_table():
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gpu_reduce_cases.json")) as f:
        d = json.load(f)
    return [(tuple(s), None if a is None else tuple(a), False) for s, a in d["cases"]] + [
        (tuple(s), None if a is None else tuple(a), True) for s, a in d["reference_skips"]]


@pytest.mark.parametrize("which", ["float32", "int64"])
def test_reference_gpu_shape_and_mask_table(which):
    """Every entry of the reference's GPU reduction table (theano/gpuarray/tests/test_elemwise.py:266-346: shapes
    with an extent above 4096 in each position x every reduce mask, degenerate and empty extents), and the
    entries it leaves out because GpuCAReduceCuda has no kernel for the mask - sum and max (min, prod for the
    small ones) against the oracle; float32 and int64 as there."""
    rng = np.random.default_rng(33)
    for shape, axis, skipped in _reference_gpu_table():
        x = T.TensorType(which, [s == 1 for s in shape])("x")
        n = int(np.prod(shape, dtype="int64"))
        v = (rng.standard_normal(shape).astype("float32") if which == "float32"
             else rng.integers(-2 ** 40, 2 ** 40, shape).astype("int64"))
        red = [shape[a] for a in (range(len(shape)) if axis is None else axis)]
        names = ["sum", "max"] + (["min", "prod"] if n <= 4096 else [])
        for name in names:
            out = REDUCERS[name](x, axis)
            if 0 in red and name in ("max", "min"):
                with pytest.raises(ValueError):
                    th.function([x], out)(v)
                continue
            vv = (v % 7 - 3) if (name == "prod" and which == "int64") else v
            check(x, out, vv, "%s %s %s %s%s" % (name, which, shape, axis, " (not in the reference's run)" if skipped else ""))


@pytest.mark.parametrize("dtype", ["bool", "int8", "uint8", "int16", "uint16", "int32", "uint32", "int64", "uint64",
                                   "float16", "float32", "float64"])
def test_dtype_coverage(dtype):
    rng = np.random.default_rng(23)
    x = T.TensorType(dtype, (False, False))("x")
    if dtype == "bool":
        v = rng.integers(0, 2, (77, 130)).astype("bool")
    elif np.dtype(dtype).kind in "iu":
        v = rng.integers(0 if dtype[0] == "u" else -3, 4, (77, 130)).astype(dtype)
    else:
        v = rng.uniform(0.5, 1.5, (77, 130)).astype(dtype)
    tol = dict(rtol=1e-12, atol=1e-12) if dtype == "float64" else None
    for axis in ((0,), (1,), None):
        check(x, x.sum(axis=axis), v, "sum %s %s" % (dtype, axis), tol)
        check(x, x.max(axis=axis), v, "max %s %s" % (dtype, axis), tol)
        check(x, x.min(axis=axis), v, "min %s %s" % (dtype, axis), tol)
        if dtype != "float16":
            check(x, x.prod(axis=axis), v, "prod %s %s" % (dtype, axis), tol)
        if dtype != "bool" and np.dtype(dtype).kind != "f":
            check(x, T.sum(x, axis=axis, dtype="float64"), v, "sum to f64")


BIT_REDUCERS = {"and_": np.bitwise_and, "or_": np.bitwise_or, "xor": np.bitwise_xor}


def _np_bit_reduce(ufunc, v, axis):
    """NumPy's answer the way theano/tensor/tests/test_elemwise.py:334-347, 443-456 builds it: one axis at
    a time, highest first, with the op's identity (-1 for and, 0 for or / xor) where an axis is empty."""
    axes = range(v.ndim) if axis is None else [a + v.ndim if a < 0 else a for a in axis]
    for a in sorted(axes, reverse=True):
        v = ufunc.reduce(v, axis=a)
    return np.asarray(v)


@pytest.mark.parametrize("dtype", ["int8", "uint8", "int32"])
@pytest.mark.parametrize("opname", sorted(BIT_REDUCERS))
def test_bitwise_careduce_reference_case_table(opname, dtype):
    """CAReduce{and_, or_, xor} on integers (theano/tensor/tests/test_elemwise.py:352-366, 443-460, run there for
    int8 / uint8): the reference's shape x axis table with its 0 / 1 inputs and with random bit patterns, then
    shapes long enough for every kernel form and for split reductions.  Bit-exact against NumPy and the oracle."""
    from theano_amd import scalar as scal
    from theano_amd.tensor.elemwise import CAReduce
    rng = np.random.default_rng(31)
    info = np.iinfo(dtype)
    big = [((4100, 3), (0,)), ((3, 4100), (1,)), ((300000,), None), ((1025, 1025), (0,)), ((1025, 1025), (1,)),
           ((1025, 1025), None), ((33, 65, 17), (0, 2)), ((2100, 2100), None)]
    for shape, axis in list(CAREDUCE_CASES) + big:
        x = T.TensorType(dtype, [s == 1 for s in shape])("x")
        out = CAReduce(getattr(scal, opname), axis=axis)(x)
        assert out.type.dtype == dtype
        f = th.function([x], out)
        samples = [(rng.random(shape) < 0.5).astype(dtype),
                   rng.integers(info.min, int(info.max) + 1, shape, dtype="int64").astype(dtype)]
        if opname == "and_":      # mostly-ones patterns, so that an and over many elements is not simply 0
            samples.append((rng.integers(info.min, int(info.max) + 1, shape, dtype="int64") |
                            rng.integers(info.min, int(info.max) + 1, shape, dtype="int64") | 0x55).astype(dtype))
        for v in samples:
            got = f(v)
            want = _np_bit_reduce(BIT_REDUCERS[opname], v, axis)
            ref = G.evaluate([x], [out], [v])[0]
            what = "%s %s %s %s [%s]" % (opname, dtype, shape, axis, hip.last_plan())
            assert got.dtype == want.dtype == ref.dtype and got.shape == want.shape, what
            assert np.array_equal(got, want) and np.array_equal(got, ref), what


def test_1024_thread_row_plan():
    """Few results with long reduce domains (128 to 1024 results of at least 8192 vectors each) take the
    1024-threads-per-result form of the row kernel instead of a split: the plan behind batch-norm's
    per-channel statistics.  Single reductions, the two-reduced-dimension variant, a fused prologue with two
    inputs, several accumulators with an epilogue, float16 storage - all against the oracle."""
    rng = np.random.default_rng(41)
    x = T.fmatrix("x")
    for shape in ((128, 32768), (200, 40004)):
        v = rng.standard_normal(shape).astype("float32")
        for name in ("sum", "max", "min"):
            check(x, REDUCERS[name](x, 1), v, "%s %s" % (name, shape))
            assert "|t1024|" in hip.last_plan(), hip.last_plan()
        vp = rng.uniform(0.999, 1.001, shape).astype("float32")
        check(x, x.prod(axis=1), vp, "prod %s" % (shape,))
        assert "|t1024|" in hip.last_plan()
    t, u = T.ftensor3("t"), T.ftensor3("u")
    tv, uv = (rng.standard_normal((6, 160, 7000)).astype("float32") for _ in range(2))
    check(t, t.sum(axis=(0, 2)), tv, "outer x kept x inner")
    assert "|t1024|a1|" in hip.last_plan(), hip.last_plan()
    outs = [T.sum(t * u, axis=(0, 2)), T.sum(T.sqr(t - u), axis=(0, 2)) / np.float32(42000.0), T.max(t + u, axis=(0, 2))]
    got = th.function([t, u], outs)(tv, uv)
    plan = hip.last_plan()
    ref = G.evaluate([t, u], outs, [tv, uv])
    for k, (g, r) in enumerate(zip(got, ref)):
        assert_parity(g, r, "two-input prologue, output %d [%s]" % (k, plan))
    f = th.function([t, u], outs)
    assert len([n for n in f.toposort() if type(n.op).__name__ == "HipCAReduce"]) == 1 and "|t1024|" in plan, plan
    # float16 storage, float32 statistics with float32 accumulators, per-channel epilogue (mean and mean of squares)
    h = T.TensorType("float16", (False,) * 4)("h")
    hv = rng.normal(0.5, 2.0, (16, 128, 70, 64)).astype("float16")
    hf = T.cast(h, "float32")
    m = np.float32(16 * 70 * 64)
    outs = [T.sum(hf, axis=(0, 2, 3), acc_dtype="float32") / m, T.sum(T.sqr(hf), axis=(0, 2, 3), acc_dtype="float32") / m]
    got = th.function([h], outs)(hv)
    plan = hip.last_plan()
    assert "|t1024|" in plan, plan
    truth = [hv.astype("float64").mean(axis=(0, 2, 3)), (hv.astype("float64") ** 2).mean(axis=(0, 2, 3))]
    ref = G.evaluate([h], outs, [hv])
    for g, r, w in zip(got, ref, truth):
        # float32 accumulators over 71680 terms: the sequential oracle itself is ~1e-4 from the float64 value, the
        # tree-ordered kernel closer
        assert_within_reference_error(g, r, w, "float16 statistics [%s]" % plan)


def test_precision_of_default_accumulator():
    # theano/tensor/tests/test_elemwise.py:953-966
    x = T.fvector("x")
    v = np.asarray([1e8, 1, -1e8], dtype="float32")
    assert float(th.function([x], x.sum())(v)) == 1.0
    big = np.ones(1 << 22, "float32") * np.float32(0.1)
    got = float(th.function([x], x.sum())(big))
    assert got == np.float32(big.astype("float64").sum())


def test_nan_propagation_and_negative_zero():
    x = T.fmatrix("x")
    v = np.array([[1.0, np.nan, 3.0], [4.0, 5.0, 6.0], [-np.inf, np.inf, 0.0]], dtype="float32")
    for axis in ((0,), (1,), None):
        check(x, x.max(axis=axis), v, "max nan %s" % (axis,))
        check(x, x.min(axis=axis), v, "min nan %s" % (axis,))
        check(x, x.sum(axis=axis), v, "sum nan %s" % (axis,))


def test_strided_inputs_and_explicit_dtypes():
    rng = np.random.default_rng(24)
    x = T.ftensor3("x")
    v = rng.standard_normal((31, 47, 53)).astype("float32")
    xt = x.dimshuffle(2, 0, 1)
    for axis in ((0,), (1,), (2,), (0, 2), (1, 2), None):
        got = th.function([x], xt.sum(axis=axis))(v)
        ref = G.evaluate([x], [xt.sum(axis=axis)], [v])[0]
        assert_parity(got, ref, "transposed view %s" % (axis,))
    xi = T.imatrix("xi")
    vi = rng.integers(-2 ** 30, 2 ** 30, (513, 257)).astype("int32")
    check(xi, T.sum(xi, axis=0, dtype="int64"), vi, "int64 sum")
    check(xi, T.sum(xi, axis=1, dtype="int32", acc_dtype="int32"), vi, "wrapping int32 sum")
    check(xi, T.sum(xi, axis=None, dtype="float32", acc_dtype="float64"), vi, "float sum of ints")


def test_fused_prologue_and_multi_output():
    rng = np.random.default_rng(25)
    x, y = T.fmatrix("x"), T.fmatrix("y")
    r = T.frow("r")
    xv, yv = rng.standard_normal((301, 515)).astype("float32"), rng.standard_normal((301, 515)).astype("float32")
    rv = rng.standard_normal((1, 515)).astype("float32")
    outs = [T.sum(T.sqr(x - y) * r, axis=1), T.sum(abs(x) * y, axis=0), T.max(x * r + y), T.mean(x, axis=0),
            T.var(x, axis=1), T.std(y, axis=0)]
    f = th.function([x, y, r], outs)
    got = f(xv, yv, rv)
    ref = G.evaluate([x, y, r], outs, [xv, yv, rv])
    truth = G.evaluate([x, y, r], outs, [xv, yv, rv], wide=True)
    for k, (g, rr, w) in enumerate(zip(got, ref, truth)):
        if k < 4:
            assert_parity(g, rr, "fused reduce %d" % k)
        else:   # var / std: x - mean(x) is a float32 difference that the squares inherit, in the reference as here
            assert_within_reference_error(g, rr, w, "fused reduce %d" % k)
    a = T.imatrix("a")
    av = rng.integers(-5, 6, (200, 333)).astype("int32")
    g2 = th.function([a], [T.any(a > 4), T.all(a > -6), T.any(a > 5), T.all(a > 0)])(av)
    assert [bool(v) for v in g2] == [True, True, False, False]


def test_reductions_over_different_shapes_that_share_a_broadcast_weight():
    """Two losses over different batch sizes that share a (1, C) parameter: separate kernels, both right."""
    rng = np.random.default_rng(27)
    x, y = T.fmatrix("x"), T.fmatrix("y")
    w = T.frow("w")
    outs = [T.sum(T.exp(x) * w), T.sum(T.tanh(y) * w), T.sum(x * w, axis=0), T.sum(y * w, axis=0)]
    vals = [rng.standard_normal((4, 8)).astype("float32"), rng.standard_normal((6, 8)).astype("float32"),
            rng.standard_normal((1, 8)).astype("float32")]
    got = th.function([x, y, w], outs)(*vals)
    ref = G.evaluate([x, y, w], outs, vals)
    for k, (g, r) in enumerate(zip(got, ref)):
        assert_parity(g, r, "shared weight, output %d" % k)


def test_sums_over_results_of_a_reduction_over_the_same_elements_share_its_pass():
    """sum(g * (x - mean(x))) and its relatives: the mean leaves the prologue (sum(g * x) - mean * sum(g)), the
    reductions merge into the pass that computes the mean, their epilogues chained.  float32 and float64 data,
    row, column and per-channel layouts; values held to the float64 value like every difference of sums."""
    from theano_amd.hip import HipCAReduce
    rng = np.random.default_rng(28)
    for dtype, shape, axes in (("float32", (6, 37, 5, 9), (0, 2, 3)), ("float32", (300, 515), (1,)),
                               ("float32", (301, 64), (0,)), ("float64", (40, 33, 7), (0, 2))):
        nd = len(shape)
        tt = T.TensorType(dtype, (False,) * nd)
        x, g = tt("x"), tt("g")
        mean = T.mean(x, axis=axes, keepdims=True)
        istd = 1 / T.sqrt(T.mean(T.sqr(x - mean), axis=axes, keepdims=True) + np.asarray(1e-3, dtype))
        outs = [T.sum(g * (x - mean), axis=axes), T.sum((x - mean) * istd * g, axis=axes, keepdims=True) * istd,
                T.sum(g - mean, axis=axes), T.sum(x * g, axis=axes) / T.sum(x, axis=axes)]
        vals = [rng.normal(0.7, 1.5, shape).astype(dtype), rng.standard_normal(shape).astype(dtype)]
        f = th.function([x, g], outs)
        reds = [n for n in f.toposort() if isinstance(n.op, HipCAReduce)]
        if dtype == "float32" and axes != (1,):      # (last-axis islands are row chains; float64 variances keep two passes)
            assert len(reds) == 1 and len(reds[0].op.scalar_ops) <= 5, [str(n.op)[:60] for n in reds]
        got = f(*vals)
        ref = G.evaluate([x, g], outs, vals)
        truth = G.evaluate([x, g], outs, vals, wide=True) if dtype == "float32" else ref
        for k, (a, b, w) in enumerate(zip(got, ref, truth)):
            assert_within_reference_error(a, b, w, "%s %s output %d" % (dtype, shape, k),
                                          tol=None if dtype == "float32" else dict(rtol=1e-11, atol=1e-11))
        with th.config.change_flags(merge_dependent_reductions=False):
            plain = th.function([x, g], outs)
        if axes != (1,):
            assert len([n for n in plain.toposort() if isinstance(n.op, HipCAReduce)]) > 1
        for k, (a, b, w) in enumerate(zip(plain(*vals), ref, truth)):       # the unmerged kernels meet the same bar
            assert_within_reference_error(a, b, w, "%s %s separate kernels, output %d" % (dtype, shape, k),
                                          tol=None if dtype == "float32" else dict(rtol=1e-11, atol=1e-11))


@pytest.mark.parametrize("ratio", [1e3, 1e4])
def test_hoisted_sums_keep_their_accuracy_when_the_mean_dwarfs_the_spread(ratio):
    """sum(g * (x - mean)) run as sum(g * x) - mean * sum(g): the expanded terms are `ratio` times larger than the
    original ones, so the products must be formed without a float32 rounding (2**-24 |g x| per term would show as
    1e-4 ... 1e-2 of the result here).  Checked against NumPy in float64 with the mean as float32 data (what the
    reference's graph feeds its second reduction) and with the unrounded mean: the device has to be within the
    float32 bar of one of them, per channel."""
    from theano_amd.hip import HipCAReduce
    rng = np.random.default_rng(int(ratio))
    for shape, axes in (((7, 24, 9, 11), (0, 2, 3)), ((2000, 48), (0,))):
        nd = len(shape)
        tt = T.TensorType("float32", (False,) * nd)
        x, g = tt("x"), tt("g")
        mean = T.mean(x, axis=axes, keepdims=True)
        outs = [T.sum(g * (x - mean), axis=axes), T.sum((x - mean) * g * np.float32(0.5), axis=axes), mean]
        xv = (rng.standard_normal(shape) + ratio).astype("float32")
        gv = rng.uniform(0.5, 1.5, shape).astype("float32")
        f = th.function([x, g], outs)
        reds = [n for n in f.toposort() if isinstance(n.op, HipCAReduce)]
        assert len(reds) == 1, [str(n.op)[:60] for n in reds]           # the rewrite applied: one pass
        got = f(xv, gv)
        x64, g64 = xv.astype("float64"), gv.astype("float64")
        m64 = x64.mean(axis=axes, keepdims=True)
        # the reference's mean: the float64 accumulator rounded to a float32 sum, divided in float32
        count = np.float32(np.prod([shape[a] for a in axes]))
        assert_parity(got[2], x64.sum(axis=axes, keepdims=True).astype("float32") / count, "mean")
        m32 = got[2].astype("float64")
        for k, scale in ((0, 1.0), (1, 0.5)):
            want = [(scale * g64 * (x64 - m)).sum(axis=axes) for m in (m32, m64)]
            err = np.minimum(*[np.abs(got[k] - w) / (1e-6 + 1e-5 * np.abs(w)) for w in want])
            assert got[k].dtype == np.float32 and err.max() <= 1.0, (shape, k, float(err.max()))


def test_stored_elementwise_result_and_its_reduction_over_all_but_the_last_axis():
    """r = f(...) is an output and so is reduce(r, all axes but the last): one node (HipElemwiseReduce).  Through
    permuted views (NCHW read as NHWC) the kernel that stores r accumulates the per-channel results as well
    ('er' plan, partials merged by the reduction's final pass); with any other layout the library reduces the
    stored result.  Integer results bit-exact, float32 at the float32 bar; ragged extents, one group and many."""
    from theano_amd.hip import HipElemwiseReduce
    rng = np.random.default_rng(29)
    cases = [("int32", (3, 128, 7, 9)), ("int32", (5, 130, 33, 37)), ("int32", (2, 16, 4, 4)), ("float32", (9, 64, 20, 24)),
             ("float32", (4, 36, 50, 70)), ("int16", (6, 64, 18, 32))]
    for dtype, shape in cases:
        t4 = T.TensorType(dtype, (False,) * 4)
        a, b = t4("a"), t4("b")
        av, bv = a.dimshuffle(0, 2, 3, 1), b.dimshuffle(0, 2, 3, 1)
        if dtype == "float32":
            r = T.tanh(av) * bv + av
            vals = [rng.standard_normal(shape).astype(dtype) for _ in range(2)]
            outs = [r, T.sum(r, axis=(0, 1, 2))]
        else:
            r = ((av & bv) ^ (av >> 2)) % 51 + bv
            info = np.iinfo(dtype)
            vals = [rng.integers(info.min // 4, info.max // 4, shape).astype(dtype) for _ in range(2)]
            outs = [r, T.sum(r, axis=(0, 1, 2), dtype="int64")]
        f = th.function([a, b], outs)
        kinds = [type(n.op).__name__ for n in f.toposort() if type(n.op).__name__.startswith("Hip") and
                 type(n.op).__name__ not in ("HipDimShuffle", "HipToHost")]
        assert kinds == ["HipElemwiseReduce"], kinds
        got = f(*vals)
        plan = hip.last_plan()
        assert "|er|" in plan or "rf|" in plan, plan
        ref = G.evaluate([a, b], outs, vals)
        assert_parity(got[0], ref[0], "%s %s elementwise result [%s]" % (dtype, shape, plan))
        if dtype == "float32":
            # the sum of the values this kernel stored (a last-place difference of tanh per element is inside the
            # bar for r, but 14 000 of them do not cancel in a sum that itself nearly cancels)
            want = got[0].astype("float64").sum(axis=(0, 1, 2)).astype("float32")
            assert_parity(got[1], want, "%s %s sum of the stored result [%s]" % (dtype, shape, plan))
            # against the reference's sum: every stored element may differ from the reference's by its own bar
            # (checked above), so the sums may differ by the sum of those bars and by no more
            room = (1e-6 + 1e-5 * np.abs(ref[0].astype("float64"))).sum(axis=(0, 1, 2))
            assert np.all(np.abs(got[1].astype("float64") - ref[1]) <= room + 1e-6 + 1e-5 * np.abs(ref[1]))
        else:
            assert_parity(got[1], ref[1], "%s %s sum [%s]" % (dtype, shape, plan))
    # no permuted read: the same node, reduced by a second launch of the library's own choosing
    x = T.fmatrix("x")
    r = T.exp(x) * T.tanh(x) + T.log1p(x * x)       # too much arithmetic to be recomputed inside the reduction
    outs = [r, T.sum(r, axis=0)]
    xv = rng.standard_normal((700, 96)).astype("float32")
    f = th.function([x], outs)
    assert any(isinstance(n.op, HipElemwiseReduce) for n in f.toposort())
    got = f(xv)
    assert " + " in hip.last_plan(), hip.last_plan()
    for g, rr in zip(got, G.evaluate([x], outs, [xv])):
        assert_parity(g, rr, "unpermuted")
    # an empty leading extent: the results are the reductions' identities
    e = th.function([x], [x + 1, T.sum(x + 1, axis=0)])(np.zeros((0, 5), "float32"))
    assert e[0].shape == (0, 5) and np.array_equal(e[1], np.zeros(5, "float32"))


def test_split_any_all_finish_in_one_launch():
    """any / all over long reduce domains: the slices of a split reduction settle the result through one
    atomic add each on a single word per result (plan suffix 'tk'), which the last slice puts back to zero.
    Row and column forms, one and several results, every combination of answers, and the same function
    called again and again with inputs whose answers differ (a word left dirty would show at once)."""
    rng = np.random.default_rng(30)
    x = T.imatrix("x")
    both = th.function([x], [T.any(x > 0), T.all(x > 0), T.any(x > 5)])
    rows = th.function([x], [T.any(x > 0, axis=1), T.all(x > 0, axis=1)])
    cols = th.function([x], [T.any(x > 0, axis=0), T.all(x > 0, axis=0)])
    base = rng.integers(1, 5, (3000, 2048)).astype("int32")          # all positive, none above 5
    variants = []
    for kind in range(4):
        v = base.copy()
        if kind in (1, 3):
            v[rng.integers(0, 3000), rng.integers(0, 2048)] = -7      # all(x > 0) turns false
        if kind in (2, 3):
            v[2999, 2047] = 9                                         # any(x > 5) turns true, in the last slice
        variants.append(v)
    variants.append(-base)                                            # nothing positive at all
    for rep in range(2):
        for v in variants:
            got = both(v)
            assert "|tk|" in hip.last_plan() and "|s" in hip.last_plan().split("|m")[-1], hip.last_plan()
            assert [bool(g) for g in got] == [bool((v > 0).any()), bool((v > 0).all()), bool((v > 5).any())]
    wide = rng.integers(-3, 4, (4, 1 << 20)).astype("int32")
    wide[1] = np.abs(wide[1]) + 1
    wide[2] = -np.abs(wide[2])
    for _ in range(2):
        a, b = rows(wide)
        assert "|tk|" in hip.last_plan(), hip.last_plan()
        assert np.array_equal(a, (wide > 0).any(axis=1)) and np.array_equal(b, (wide > 0).all(axis=1))
    tall = rng.integers(-3, 4, (200000, 8)).astype("int32")
    tall[:, 1] = np.abs(tall[:, 1]) + 1
    tall[:, 2] = -np.abs(tall[:, 2])
    for _ in range(2):
        a, b = cols(tall)
        assert "|tk|" in hip.last_plan() and "|rc|" in hip.last_plan(), hip.last_plan()
        assert np.array_equal(a, (tall > 0).any(axis=0)) and np.array_equal(b, (tall > 0).all(axis=0))
    # the two-launch form gives the same answers
    import os
    os.environ["THX_RED_TICKET"] = "0"
    try:
        got = both(variants[3])
        assert "|tk|" not in hip.last_plan()
        assert [bool(g) for g in got] == [True, False, True]
    finally:
        del os.environ["THX_RED_TICKET"]


def test_more_work_than_one_dispatch_holds_is_strided_over_the_blocks(monkeypatch):
    """A dispatch carries at most 2^32 - 1 work-items.  Reductions with more (block of results) x (slice) pieces
    than that take the striding kernels (plan suffix 'gs'), in which a block handles pieces blockIdx.x,
    blockIdx.x + gridDim.x, ...  The limit is lowered here so that arrays of ordinary size reach them: row, column
    and generic forms, a second result, an argmax and a NaN in the last piece."""
    monkeypatch.setenv("THX_RED_MAX_DISPATCH", "4096")
    rng = np.random.default_rng(41)
    x = T.fmatrix("x")
    val = rng.standard_normal((5000, 96)).astype("float32")
    val[4999, 95] = np.nan
    for axis, form in ((1, "|rr|"), (0, "|rc|")):
        outs = [T.sum(x, axis=axis), T.max(x, axis=axis)]
        got = th.function([x], outs)(val)
        assert form in hip.last_plan() and "|gs|" in hip.last_plan(), hip.last_plan()
        ref = G.evaluate([x], outs, [val])
        assert np.allclose(got[0], ref[0], rtol=1e-6, atol=1e-6, equal_nan=True)
        assert np.array_equal(got[1], ref[1], equal_nan=True)
        mv, iv = th.function([x], T.max_and_argmax(x, axis=axis))(val)
        assert "|gs|" in hip.last_plan(), hip.last_plan()
        ref_m, ref_i = G.max_and_argmax(val, (axis,))
        assert np.array_equal(mv, ref_m, equal_nan=True) and np.array_equal(iv, ref_i)
    wide = rng.standard_normal((3, 70000)).astype("float32")          # few results: still split into slices
    got = th.function([x], T.sum(x, axis=1))(wide)
    assert np.allclose(got, wide.astype("float64").sum(axis=1), rtol=1e-6)
    tall = rng.integers(-9, 9, (70000, 40)).astype("float32")
    got = th.function([x], [T.sum(x, axis=0), T.min(x, axis=0)])(tall)
    assert np.array_equal(got[0], tall.sum(axis=0)) and np.array_equal(got[1], tall.min(axis=0))
    t6 = T.TensorType("int32", (False,) * 6)("t6")
    v6 = rng.integers(-100, 100, (3, 14, 5, 16, 7, 12)).astype("int32")
    got = th.function([t6], T.sum(t6, axis=(0, 2, 4)))(v6)
    assert "|rg|" in hip.last_plan() and "|gs|" in hip.last_plan(), hip.last_plan()
    assert got.dtype == np.int64 and np.array_equal(got, v6.sum(axis=(0, 2, 4)))


def test_epilogue_chain_with_per_result_device_operands():
    """Per-channel algebra after a reduction (other per-channel arrays, results
    of an earlier reduction, host scalars) runs in the reduction's epilogue;
    factors that are constant along the reduced axes leave the sums."""
    from theano_amd.hip import HipCAReduce, HipElemwise
    rng = np.random.default_rng(26)
    t4 = T.TensorType("float32", (False,) * 4)
    pc = T.TensorType("float32", (True, False, True, True))
    x, g = t4("x"), t4("g")
    gamma, beta = pc("gamma"), pc("beta")
    mean = T.mean(x, axis=(0, 2, 3), keepdims=True)
    d = x - mean
    std = T.sqrt(T.mean(T.sqr(d), axis=(0, 2, 3), keepdims=True) + np.float32(1e-3))
    s1 = T.sum(g * gamma * d / (std * std), axis=(0, 2, 3), keepdims=True)
    s2 = T.sum((g / std) * d, axis=(0, 2, 3), keepdims=True)
    outs = [s1 * gamma + beta / std, (s2 - s1) * T.exp(beta), T.sum(g, axis=(0, 2, 3))]
    vals = [rng.standard_normal((6, 37, 5, 9)).astype("float32"), rng.standard_normal((6, 37, 5, 9)).astype("float32"),
            rng.uniform(0.5, 2, (1, 37, 1, 1)).astype("float32"), rng.standard_normal((1, 37, 1, 1)).astype("float32")]
    with th.config.change_flags(merge_dependent_reductions=False):
        f2 = th.function([x, g, gamma, beta], outs)
    kernels = [n for n in f2.toposort() if isinstance(n.op, (HipCAReduce, HipElemwise))]
    assert [type(n.op) for n in kernels] == [HipCAReduce, HipCAReduce], kernels
    assert any(type(i.type).__name__ == "HipArrayType" for i in kernels[1].inputs[len(kernels[1].inputs) - kernels[1].op.n_extra:])
    # by default the second reduction gives up the mean in its prologue and joins the first one's pass
    f = th.function([x, g, gamma, beta], outs)
    kernels = [n for n in f.toposort() if isinstance(n.op, (HipCAReduce, HipElemwise))]
    assert [type(n.op) for n in kernels] == [HipCAReduce], kernels
    assert any(type(i.type).__name__ == "HipArrayType" for i in kernels[0].inputs[len(kernels[0].inputs) - kernels[0].op.n_extra:])
    got = f(*vals)
    ref = G.evaluate([x, g, gamma, beta], outs, vals)
    truth = G.evaluate([x, g, gamma, beta], outs, vals, wide=True)
    for k, (a, a2, b, w) in enumerate(zip(got, f2(*vals), ref, truth)):
        # sums of g * (x - mean) are sums of signed terms near zero, and (s2 - s1) a difference of two of them
        assert_within_reference_error(a, b, w, "epilogue output %d" % k)
        assert_within_reference_error(a2, b, w, "epilogue output %d, separate kernels" % k)
    # a per-result operand of the wrong extent is refused like any broadcast mismatch
    bad = list(vals)
    bad[2] = np.ones((1, 36, 1, 1), "float32")
    with pytest.raises(ValueError):
        f(*bad)


@pytest.mark.gpu
def test_prod_gradient_with_zeros_and_prod_without_zeros():
    """Zero-aware gradient of Prod on random data with planted zeros (groups with none,
    one and several), against the oracle and against the closed form: the product of
    the other elements of the group."""
    from theano_amd.tensor.elemwise import ProdWithoutZeros
    rng = np.random.default_rng(33)
    xv = rng.uniform(0.5, 1.5, (37, 29))
    xv[3, 4] = 0.0
    xv[5, 1] = xv[5, 20] = 0.0
    xv[30, :] = 0.0
    x = T.dmatrix("x")
    for axis in (0, 1):
        ins, outs = [x], [th.grad(T.sum(T.prod(x, axis=axis)), x), ProdWithoutZeros(axis=axis)(x)]
        got = th.function(ins, outs)(xv)
        ref = G.evaluate(ins, outs, [xv])
        for g, r in zip(got, ref):
            assert np.allclose(g, r, rtol=1e-12, atol=0)
        want = np.empty_like(xv)
        for idx in np.ndindex(*xv.shape):
            group = xv[:, idx[1]] if axis == 0 else xv[idx[0], :]
            want[idx] = np.prod(np.delete(group, idx[axis]))
        assert np.allclose(got[0], want, rtol=1e-10)


@pytest.mark.gpu
def test_epilogue_operand_that_is_a_strided_view():
    """A per-result operand of a fused epilogue may be any view (every other element of a
    vector, a column of a matrix): the epilogue reads it at the result's index."""
    rng = np.random.default_rng(8)
    x, m = T.fmatrix("x"), T.fmatrix("m")
    v = T.fvector("v")
    outs = [T.sum(x, axis=1) * v[1::2] + m[:, 2], T.max(x, axis=0) / (abs(m.T[1]) + 1.0)]
    xv = rng.standard_normal((37, 37)).astype("float32")
    vals = [xv, rng.standard_normal((37, 5)).astype("float32"), rng.standard_normal(75).astype("float32")]
    f = th.function([x, m, v], outs)
    assert not any(type(n.op).__name__ == "HipElemwise" for n in f.toposort())     # both are epilogues
    for g, r in zip(f(*vals), G.evaluate([x, m, v], outs, vals)):
        assert_parity(g, r, "strided epilogue operand")


@pytest.mark.gpu
def test_transposed_reduction_result_is_not_fused_as_an_epilogue():
    """sum(x, 1).dimshuffle(2, 'x', 1, 0) * y: the consumer works in a transposed layout, so
    y is not a per-result operand of the reduction (with equal extents a shape check could
    not tell); only DimShuffles that insert or drop broadcast dimensions sit between a
    reduction and its epilogue."""
    rng = np.random.default_rng(10)
    x = T.TensorType("float32", (False,) * 4)("x")
    y = T.TensorType("float32", (False, True, False, False))("y")
    r = T.sum(x, axis=1)
    outs = [r.dimshuffle(2, "x", 1, 0) * y, r.dimshuffle(0, "x", 1, 2) * y]
    vals = [rng.standard_normal((5, 3, 5, 5)).astype("float32"), rng.standard_normal((5, 1, 5, 5)).astype("float32")]
    for g, w in zip(th.function([x, y], outs)(*vals), G.evaluate([x, y], outs, vals)):
        assert_parity(g, w, "transposed consumer of a reduction")
    f = th.function([x, y], outs[1:])
    assert not any(type(n.op).__name__ == "HipElemwise" for n in f.toposort())      # this one is an epilogue


def test_negated_max_of_a_negation_runs_as_min_with_the_same_values():
    """-max(-x) (the reference's spelling of tensor.min, rewritten to one min reduction for floats) against the
    oracle's evaluation of the written graph: NaN rows, signed zeros, infinities; integers keep the written form
    and agree at the most negative value, where the two forms differ."""
    rng = np.random.default_rng(5)
    for dtype in ("float32", "float64", "float16"):
        x = T.TensorType(dtype, (False, False))("x")
        v = rng.standard_normal((37, 300)).astype(dtype)
        v[3, 5] = np.nan
        v[4, :] = np.inf
        v[5, 7] = -np.inf
        v[6, :] = 0.0
        v[6, 11] = -0.0
        for axis in (0, 1, None):
            out = -T.max(-x, axis=axis)
            got = th.function([x], out)(v)
            ref = G.evaluate([x], [out], [v])[0]
            assert got.dtype == ref.dtype and np.array_equal(got, ref, equal_nan=True), (dtype, axis)
            assert np.array_equal(got, np.min(v, axis=axis), equal_nan=True)
    i = T.imatrix("i")
    iv = rng.integers(-100, 100, (20, 50)).astype("int32")
    iv[2, 3] = -2 ** 31
    out = -T.max(-i, axis=1)
    got = th.function([i], out)(iv)
    assert np.array_equal(got, G.evaluate([i], [out], [iv])[0])
    # -(-2**31) wraps to -2**31, the smallest value: the written form skips that element, a min would return it
    assert got[2] == np.delete(iv[2], 3).min() and np.array_equal(np.delete(got, 2), np.delete(iv.min(axis=1), 2))


def test_max_of_a_computed_value_and_its_gradient_see_the_same_bits():
    """The gradient of max compares the reduction's result with its operand for equality.  When the operand is
    a computed value, the kernel that reduces it and the kernel that compares it must agree to the last bit:
    the operand is stored once and read by both (never recomputed per kernel), and sqrt / division / exp have
    one spelled-out lowering.  Every reduced slice must find its maximum again."""
    rng = np.random.default_rng(11)
    x = T.TensorType("float32", (False,) * 4)("x")
    y = T.TensorType("float32", (False,) * 4)("y")
    xv = rng.standard_normal((16, 6, 64, 5)).astype("float32")
    yv = rng.uniform(0.5, 1.5, xv.shape).astype("float32")
    families = [lambda a, b: T.exp(T.minimum(T.sqrt(abs(a) + 0.5), 3.0)),
                lambda a, b: a * b + a / (b + 2.0),
                lambda a, b: T.tanh(a * 1.7 + b) / T.sqrt(b),
                lambda a, b: T.sqr(a) * b + b * 0.3 + a]
    for axis in ((0, 1), (1, 3), (0, 2, 3), (3,), None):
        for fam in families:
            e = fam(x, y)
            m = T.max(e, axis=axis, keepdims=True)
            hits = T.eq(m, e)
            # the comparison runs in an elementwise kernel (its result is an output), the max in a reduction
            got_hits, got_m, got_e = th.function([x, y], [hits, m, e], on_unused_input="ignore")(xv, yv)
            assert np.array_equal(got_e.max(axis=axis, keepdims=True), got_m), (axis, hip.last_plan())
            assert got_hits.any(axis=axis).all(), (axis, hip.last_plan())
            # and through the gradient: each slice passes its incoming gradient to (at least) one element
            g = th.grad(T.sum(T.max(e, axis=axis) * 1.0), x)
            gv, ev = th.function([x, y], [g, e], on_unused_input="ignore")(xv, yv)
            assert np.isfinite(gv).all()
            at_max = ev == ev.max(axis=axis, keepdims=True)
            assert np.array_equal(gv != 0, at_max & (gv != 0)) and (np.abs(gv) > 0).any(axis=axis).all(), axis


REAL_DTYPES = ("bool", "int8", "int16", "int32", "int64", "uint8", "uint16", "uint32", "uint64", "float16", "float32",
               "float64")
T_REDUCE_AXES = [None, 0, 1, [], [0], [1], [0, 1]]        # theano/tensor/tests/test_elemwise.py:816


def _reduce_dtype_data(rng, dtype, method, narrow):
    data = (rng.random((3, 4)) * 10).astype(dtype)         # test_elemwise.py:891-892
    return data[0:1] if method == "prod" and narrow else data


def _check_integer_of_a_float_accumulation(x, var, data, what):
    """A floating-point accumulation cast to an integer at the end: the accumulator's rounding depends on the
    order of the operations, so the integer agrees to a float32 accumulator's accuracy and to one unit, not bit
    for bit."""
    got = th.function([x], var)(data)
    ref = G.evaluate([x], [var], [data])[0]
    assert got.dtype == ref.dtype and got.shape == ref.shape, what
    g, r = got.astype("float64"), ref.astype("float64")
    assert np.all(abs(g - r) <= 1 + 1e-6 * abs(r)), (what, got, ref)


@pytest.mark.parametrize("method", ["sum", "prod"])
def test_custom_output_dtype_of_every_real_pair(method):
    """``T_reduce_dtype.test_reduce_custom_dtype`` (``theano/tensor/tests/test_elemwise.py:874-912``, run on the
    device by ``T_gpureduce_dtype``, ``theano/gpuarray/tests/test_elemwise.py:367-381``): every input dtype with every
    requested output dtype, the axis cycling through the reference's list; the reference only runs the function,
    here the value is held against the oracle (exact for integer results)."""
    rng = np.random.default_rng(41)
    idx = 0
    for input_dtype in REAL_DTYPES:
        x = T.matrix(dtype=input_dtype)
        for output_dtype in REAL_DTYPES:
            axis = T_REDUCE_AXES[idx % len(T_REDUCE_AXES)]
            var = getattr(x, method)(dtype=output_dtype, axis=axis)
            assert var.dtype == output_dtype
            narrow = output_dtype in ("float16", "int8", "uint8", "int16", "uint16")
            data = _reduce_dtype_data(rng, input_dtype, method, narrow)
            # float16 is accumulated in float32: a wider result carries that accumulator's rounding
            tol = (dict(rtol=1e-5, atol=1e-6) if input_dtype == "float16" and output_dtype == "float64" else
                   dict(rtol=1e-12, atol=1e-12) if output_dtype == "float64" else None)
            what = "%s %s -> %s axis %s" % (method, input_dtype, output_dtype, axis)
            if input_dtype.startswith("float") and not output_dtype.startswith("float"):
                _check_integer_of_a_float_accumulation(x, var, data, what)
            else:
                check(x, var, data, what, tol)
            idx += 1


@pytest.mark.parametrize("method", ["sum", "prod"])
def test_custom_accumulator_dtype_of_every_real_pair(method):
    """``T_reduce_dtype.test_reduce_custom_acc_dtype`` (``theano/tensor/tests/test_elemwise.py:914-950``): an
    accumulator that would lose precision is a TypeError, a float16 one is turned away when the kernel is
    built, every other one runs and matches the oracle's accumulation in that dtype."""
    from theano_amd import scalar as scal
    rng = np.random.default_rng(42)
    idx = 0
    for input_dtype in REAL_DTYPES:
        x = T.matrix(dtype=input_dtype)
        for acc_dtype in REAL_DTYPES:
            axis = T_REDUCE_AXES[idx % len(T_REDUCE_AXES)]
            idx += 1
            up = scal.upcast(input_dtype, acc_dtype)
            if acc_dtype == up or (input_dtype in T.discrete_dtypes and acc_dtype in T.continuous_dtypes):
                var = getattr(x, method)(acc_dtype=acc_dtype, axis=axis)
                assert var.owner.op.acc_dtype == acc_dtype
                if acc_dtype == "bool":             # 1 + 1 stored in an npy_bool: the reference's C code leaves a 2 in
                    continue                        # a boolean and its Python path an or - nothing to hold a value to
                if acc_dtype == "float16" and axis != []:   # no C code for it in the reference either (elemwise.py:1395-1398);
                    # over no axis at all nothing is accumulated (elemwise.py:1410-1417)
                    with pytest.raises(NotImplementedError, match="float16 accumulators"):
                        th.function([x], var)(np.ones((3, 4), input_dtype))
                    continue
                narrow = acc_dtype in ("float16", "int8", "uint8", "int16", "uint16") or var.dtype == "float16"
                data = _reduce_dtype_data(rng, input_dtype, method, narrow)
                tol = dict(rtol=1e-12, atol=1e-12) if var.dtype == "float64" and acc_dtype == "float64" else None
                what = "%s %s acc %s axis %s" % (method, input_dtype, acc_dtype, axis)
                if acc_dtype.startswith("float") and not var.dtype.startswith("float"):
                    _check_integer_of_a_float_accumulation(x, var, data, what)
                else:
                    check(x, var, data, what, tol)
            else:
                with pytest.raises(TypeError):
                    getattr(x, method)(acc_dtype=acc_dtype, axis=axis)


@pytest.mark.parametrize("shape,axis,form", [
    ((4096, 4, 4, 4), 1, "rg"), ((4096, 2, 8), 1, "rg"), ((4096, 4, 4, 4), 2, "rg"),   # few columns and few rows
    ((3, 40001), 0, "rc"), ((2, 40001), 0, "rc"), ((64, 3, 4097), 1, "rc"),            # odd rows: element-aligned vectors
    ((3, 13), 0, "rg"), ((64, 3, 7), 1, "rg"),                                         # too few columns for those
    ((4, 40000), 0, "rc"), ((3, 40000), 0, "rc"), ((16, 40001), 0, "rc"),
    ((4096, 4, 64), 1, "rc")])
def test_column_reductions_with_few_rows_choose_between_two_forms(shape, axis, form):
    """A sum over an axis that is not the last one runs column-wise (`rc`) unless nearly all of that kernel's
    lanes would idle, or there are two to four rows of too few columns to read as vectors: then one thread
    computes one result (`rg`).  Both give the reference's values (theano/tensor/elemwise.py:1307
    CAReduce.perform)."""
    rng = np.random.default_rng(77)
    x = T.TensorType("float32", (False,) * len(shape))("x")
    v = rng.standard_normal(shape).astype("float32")
    for name in ("sum", "max"):
        out = REDUCERS[name](x, axis)
        got = th.function([x], out)(v)
        assert "|%s|" % form in hip.last_plan(), (shape, axis, hip.last_plan())
        assert_parity(got, G.evaluate([x], [out], [v])[0], "%s %s axis %d [%s]" % (name, shape, axis, hip.last_plan()))
    xi = T.TensorType("int64", (False,) * len(shape))("xi")
    vi = rng.integers(-2 ** 62, 2 ** 62, shape)
    check(xi, xi.sum(axis=axis), vi, "int64 sum %s axis %d" % (shape, axis))


@pytest.mark.parametrize("dtype", ["int8", "float16", "float32", "float64", "int16"])
def test_rows_and_columns_that_are_no_whole_number_of_vectors(dtype):
    """Long rows whose length is odd or that start off a 16-byte boundary, and columns whose number is odd, are
    read as full-width vectors through element-aligned pointers (plans marked `|ua`), the incomplete vector at the
    end element by element: every element is counted once whatever the alignment, for one operand and for several
    that are out of line by different amounts.  Values are those of CAReduce.perform
    (theano/tensor/elemwise.py:1307)."""
    from theano_amd.hip import HipArray
    rng = np.random.default_rng(31)
    kind = np.dtype(dtype).kind

    def draw(shape):
        # floats on a grid of eighths: sums and products of two are exact, so the order of the additions and the
        # precision a product is kept in between (float32 inside a fused float16 kernel) do not show
        return (rng.integers(-100, 100, shape).astype(dtype) if kind == "i" else
                (rng.integers(-8, 9, shape) / 8.0).astype(dtype))
    tol = {"float16": {"rtol": 2e-3, "atol": 2e-3}}.get(dtype)
    vec, mat, cube = (T.TensorType(dtype, (False,) * k) for k in (1, 2, 3))
    x, y, m, w, c = vec("x"), vec("y"), mat("m"), mat("w"), cube("c")
    marked = 0
    for n in (1000003, 4099, 257, 31):                  # the last two: too short to bother / to vectorise
        v = draw(n)
        for name in ("sum", "max"):
            out = REDUCERS[name](x, None)
            got = th.function([x], out)(v)
            marked += "|ua|" in hip.last_plan()
            assert_parity(got, G.evaluate([x], [out], [v])[0], "%s of %d %s [%s]" % (name, n, dtype, hip.last_plan()), tol=tol)
    # every alignment of the first element and of the last
    base = draw(70000)
    dev = HipArray.from_numpy(base)
    f = th.function([x], [th.Out(T.sum(x), device=True), th.Out(T.min(x), device=True)])
    for lo in range(0, 17):
        for hi in (70000, 69999, 69993):
            got = f(dev.view([hi - lo], [base.itemsize], dev.offset + lo * base.itemsize))
            ref = G.evaluate([x], [T.sum(x), T.min(x)], [base[lo:hi]])
            for g, r in zip(got, ref):
                assert_parity(g.to_numpy(), r, "view [%d:%d] %s [%s]" % (lo, hi, dtype, hip.last_plan()), tol=tol)
    # rows of a matrix: each row starts somewhere else
    for shape in ((37, 4099), (5, 100001), (300, 515)):
        a, b = draw(shape), draw(shape)
        out = T.sum(m * w, axis=1)
        got = th.function([m, w], out)(a, b)
        marked += "|ua|" in hip.last_plan()
        assert_parity(got, G.evaluate([m, w], [out], [a, b])[0], "rows %s %s [%s]" % (shape, dtype, hip.last_plan()), tol=tol)
        # a stepped operand beside a contiguous one, and the rows in reverse order
        wide = draw((shape[0], 2 * shape[1]))
        out2 = T.max(m[::-1] + w[:, ::2], axis=1)
        got = th.function([m, w], out2)(a, wide)
        assert_parity(got, G.evaluate([m, w], [out2], [a, wide])[0], "stepped %s %s [%s]" % (shape, dtype, hip.last_plan()), tol=tol)
    # two operands out of line by different amounts
    a, b = draw(50001), draw(50002)
    out = T.sum(x * y[1:])
    got = th.function([x, y], out)(a, b)
    assert_parity(got, G.evaluate([x, y], [out], [a, b])[0], "different alignment %s [%s]" % (dtype, hip.last_plan()), tol=tol)
    # columns: an odd number of them, one and two reduced axes, a view that drops the first column
    for shape, axis in (((301, 4099), 0), ((7, 13, 1001), (0, 1)), ((5, 33, 515), 1), ((64, 3, 67), 1), ((2, 100003), 0)):
        a = draw(shape)
        var = mat("a") if len(shape) == 2 else cube("a")
        for name in ("sum", "min"):
            out = REDUCERS[name](var, axis)
            got = th.function([var], out)(a)
            marked += "|ua|" in hip.last_plan()
            assert_parity(got, G.evaluate([var], [out], [a])[0], "columns %s %s %s %s [%s]" % (name, shape, axis, dtype, hip.last_plan()), tol=tol)
        if len(shape) == 2:
            out = T.sum(var[:, 1:] * var[:, :-1], axis=0)
            got = th.function([var], out)(a)
            assert_parity(got, G.evaluate([var], [out], [a])[0], "shifted columns %s %s [%s]" % (shape, dtype, hip.last_plan()), tol=tol)
    assert marked >= (6 if np.dtype(dtype).itemsize < 8 else 4), marked


@pytest.mark.parametrize("dtype", ["bool", "int8", "uint8", "int16", "uint16"])
def test_sums_of_narrow_integers_at_their_extremes(dtype):
    """Sums of 8- and 16-bit integers have 64-bit accumulators (theano/tensor/elemwise.py:1741-1758); the row form
    adds the elements of one vector in 32 bits first.  Rows of nothing but the type's largest and smallest values,
    long enough to overflow 32 bits as a whole: bit for bit."""
    rng = np.random.default_rng(9)
    info = None if dtype == "bool" else np.iinfo(dtype)
    lo, hi = (0, 1) if info is None else (info.min, info.max)
    x = T.TensorType(dtype, (False, False))("x")
    for shape in ((3, 70001), (2, 300007), (65, 4096)):
        for fill in ("hi", "lo", "mixed"):
            v = (np.full(shape, hi) if fill == "hi" else np.full(shape, lo) if fill == "lo" else
                 rng.choice([lo, hi], shape)).astype(dtype)
            outs = [T.sum(x, axis=1), T.sum(x), T.sum(x, axis=0)] + ([T.sum(x * x, axis=1)] if dtype != "bool" else [])
            got = th.function([x], outs)(v)
            ref = G.evaluate([x], outs, [v])
            for k, (a, r) in enumerate(zip(got, ref)):
                assert a.dtype == r.dtype and np.array_equal(a, r), "%s %s %s output %d [%s]" % (dtype, shape, fill, k, hip.last_plan())
    big = np.full((1, 40000000), hi).astype(dtype)       # 40 000 000 x 65 535 = 2.6e12
    got = th.function([x], T.sum(x))(big)
    assert int(got) == 40000000 * int(hi), (dtype, int(got))


@pytest.mark.parametrize("dtype", ["float32", "float16", "int8", "float64", "int32"])
def test_many_rows_of_a_few_columns(dtype):
    """(n, C) arrays with C of 2 to 16 reduced over their rows run as one flat walk over the elements (plans `rs`):
    every element lands in its own column whatever C, the vector width and the length's remainder are; views that
    start off a vector boundary, two operands, and the cases the form does not take (positions, a strided
    operand).  Values are those of CAReduce.perform (theano/tensor/elemwise.py:1307), integers and the floats'
    grid of eighths bit for bit."""
    from theano_amd.hip import HipArray
    rng = np.random.default_rng(3)
    kind = np.dtype(dtype).kind
    draw = (lambda shape: rng.integers(-100, 100, shape).astype(dtype)) if kind == "i" else \
           (lambda shape: (rng.integers(-8, 9, shape) / 8.0).astype(dtype))
    tol = {"float16": {"rtol": 2e-3, "atol": 2e-3}}.get(dtype)
    mat, cube = T.TensorType(dtype, (False, False)), T.TensorType(dtype, (False, False, False))
    m, w, c3 = mat("m"), mat("w"), cube("c")
    strips = 0
    for cols in (2, 3, 5, 7, 11, 13, 16):
        for rows in (70001, 300000):
            a, b = draw((rows, cols)), draw((rows, cols))
            outs = [T.sum(m, axis=0), T.max(m, axis=0), T.sum(m * w, axis=0), T.min(m + w, axis=0)]
            ref = G.evaluate([m, w], outs, [a, b])
            for k, out in enumerate(outs):          # one reduction per kernel ...
                g = th.function([m, w], out, on_unused_input="ignore")(a, b)
                strips += "|rs|" in hip.last_plan()
                assert_parity(g, ref[k], "(%d, %d) %s output %d [%s]" % (rows, cols, dtype, k, hip.last_plan()), tol=tol)
            if cols <= 5:                           # ... and all four in one, with four accumulators per column
                got = th.function([m, w], outs)(a, b)
                for k, (g, r) in enumerate(zip(got, ref)):
                    assert_parity(g, r, "(%d, %d) %s fused output %d [%s]" % (rows, cols, dtype, k, hip.last_plan()), tol=tol)
    assert strips >= (40 if np.dtype(dtype).itemsize <= 4 else 24), strips
    # a view that starts one row and one element in; rows collapsed from two axes
    base = draw(3 * 100000 + 7)
    dev = HipArray.from_numpy(base)
    f = th.function([m], [th.Out(T.sum(m, axis=0), device=True)])
    for lo in (0, 1, 3, 4):
        view = dev.view([99990, 3], [3 * base.itemsize, base.itemsize], dev.offset + lo * base.itemsize)
        got = f(view)[0].to_numpy()
        ref = G.evaluate([m], [T.sum(m, axis=0)], [base[lo:lo + 3 * 99990].reshape(99990, 3)])[0]
        assert_parity(got, ref, "view from element %d %s [%s]" % (lo, dtype, hip.last_plan()), tol=tol)
    vol = draw((300, 301, 3))
    out = T.sum(c3, axis=(0, 1))
    got = th.function([c3], out)(vol)
    assert "|rs|" in hip.last_plan(), hip.last_plan()
    assert_parity(got, G.evaluate([c3], [out], [vol])[0], "two row axes %s [%s]" % (dtype, hip.last_plan()), tol=tol)
    if dtype == "int8":          # few enough vectors for one block, which then writes the results itself
        small = draw((4096, 16))
        got = th.function([m], T.sum(m, axis=0))(small)
        assert "|rs|" in hip.last_plan() and not hip.last_plan().split("|")[-1].startswith("s"), hip.last_plan()
        assert np.array_equal(got, small.sum(axis=0, dtype="int64"))
    # not for these: positions of the maxima, an operand that is a stepped view
    a = draw((70001, 3))
    val, pos = th.function([m], T.max_and_argmax(m, axis=0))(a)
    assert "|rs|" not in hip.last_plan()
    assert np.array_equal(pos, np.argmax(a, axis=0)) and np.array_equal(val, a.max(axis=0))
    wide_a = draw((70001, 6))
    out = T.sum(m[:, ::2], axis=0)
    got = th.function([m], out)(wide_a)
    assert "|rs|" not in hip.last_plan()
    assert_parity(got, G.evaluate([m], [out], [wide_a])[0], "stepped columns %s" % dtype, tol=tol)


@pytest.mark.parametrize("dtype", ["float32", "float16", "int8"])
def test_reductions_over_axes_of_extent_one(dtype):
    """An axis of extent 1 that is not declared broadcastable: the "reduction" copies every element through the
    accumulator's type and the epilogue (theano/tensor/elemwise.py:1307); long rows of such results are read and
    written as vectors (the column form with one row)."""
    rng = np.random.default_rng(4)
    draw = (lambda shape: rng.integers(-100, 100, shape).astype(dtype)) if np.dtype(dtype).kind == "i" else \
           (lambda shape: (rng.integers(-8, 9, shape) / 8.0).astype(dtype))
    for shape, axis in (((1, 300001), 0), ((300001, 1), 1), ((1, 37, 4099), 0), ((5, 1, 70000), (1,)), ((1, 1, 2048), (0, 1)), ((1, 100), 0)):
        x = T.TensorType(dtype, (False,) * len(shape))("x")
        v = draw(shape)
        for name in ("sum", "max"):
            out = REDUCERS[name](x, axis)
            got = th.function([x], out)(v)
            if v.size >= 65536:
                assert "|rc|" in hip.last_plan(), hip.last_plan()
            ref = G.evaluate([x], [out], [v])[0]
            assert got.dtype == ref.dtype and np.array_equal(got, ref), "%s %s %s %s [%s]" % (name, dtype, shape, axis, hip.last_plan())
    x = T.TensorType(dtype, (False, False))("x")
    v = draw((1, 100000))
    val, pos = th.function([x], T.max_and_argmax(x, axis=0))(v)
    assert np.array_equal(val, v[0]) and not pos.any()
