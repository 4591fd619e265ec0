"""GPU parity of indexing, inc/set_subtensor, reshape, alloc and join against
the oracle (NumPy's basic indexing / reshape / broadcast_to / concatenate), alone
and feeding fused elementwise and reduction kernels, forward and gradient."""
import numpy as np
import pytest

import theano_amd as th
from theano_amd import tensor as T
from theano_amd.hip import HipCAReduce, HipElemwise
from oracle import graph_ref as G
from conftest import assert_parity, assert_within_reference_error

pytestmark = pytest.mark.gpu


def both(ins, outs, vals):
    f = th.function(ins, outs)
    return f, f(*vals), G.evaluate(ins, outs, vals)


def test_views_feed_kernels_without_copies():
    rng = np.random.default_rng(51)
    x = T.ftensor3("x")
    y = T.fmatrix("y")
    xv = rng.standard_normal((40, 50, 64)).astype("float32")
    yv = rng.standard_normal((50, 64)).astype("float32")
    outs = [x[1:30:3, ::-2, 4:60] * 2 + 1, T.sum(x[-1] * y, axis=1), T.max(x[..., 1:-1], axis=(0, 2)),
            T.exp(x.reshape((-1, 64))[100:300]), T.sum(x.reshape((x.shape[0], -1)), axis=1),
            x[:, 100:, :] + 1, x[5, 6], T.max_and_argmax(x[:, ::2, 3], axis=0)[1]]
    f, got, ref = both([x, y], outs, [xv, yv])
    for k, (g, r) in enumerate(zip(got, ref)):
        assert_parity(g, r, "view case %d" % k)
    # indexing and reshaping a contiguous array launch nothing: one kernel per output that computes
    kernels = [n for n in f.toposort() if isinstance(n.op, (HipElemwise, HipCAReduce))]
    assert len(kernels) == 6


def test_reshape_of_strided_array_copies_once():
    rng = np.random.default_rng(52)
    x = T.imatrix("x")
    xv = rng.integers(-100, 100, (70, 90)).astype("int32")
    outs = [x.dimshuffle(1, 0).reshape((-1,)), T.flatten(x[::2, 1::3], 1), x[::-1].reshape((90, 70)) + 1]
    f, got, ref = both([x], outs, [xv])
    for k, (g, r) in enumerate(zip(got, ref)):
        assert g.dtype == r.dtype and np.array_equal(g, r), k
    with pytest.raises(ValueError):
        th.function([x], x.reshape((7, -1, 13)))(xv)


@pytest.mark.parametrize("dtype", ["float32", "int64", "float16", "bool"])
def test_alloc_join_stack_inc_set(dtype):
    rng = np.random.default_rng(53)
    m = T.TensorType(dtype, (False, False))
    x, y = m("x"), m("y")
    r = T.TensorType(dtype, (True, False))("r")
    if dtype == "bool":
        xv, yv, rv = [rng.integers(0, 2, s).astype(dtype) for s in ((33, 47), (33, 47), (1, 47))]
    else:
        xv, yv, rv = [rng.integers(-9, 9, s).astype(dtype) for s in ((33, 47), (33, 47), (1, 47))]
    outs = [T.alloc(r, 5, x.shape[0], 47), T.join(0, x, r, y[:7]), T.join(1, x[:, :5], y), T.stack([x, y], axis=1),
            T.set_subtensor(x, y[:3, 2:9], (slice(4, 7), slice(10, 17))), T.set_subtensor(x, r, (slice(None, None, 5),)),
            T.alloc(np.asarray(1, dtype), 3, 4)]
    if dtype != "bool":
        outs.append(T.inc_subtensor(x, y[:, ::2], (slice(None), slice(1, 25))))
        outs.append(T.inc_subtensor(x, r, (slice(2, 9),)))
    f, got, ref = both([x, y, r], outs, [xv, yv, rv])
    for k, (g, rr) in enumerate(zip(got, ref)):
        assert g.dtype == rr.dtype and g.shape == rr.shape and np.array_equal(g, rr), (dtype, k)
    assert np.array_equal(f(xv, yv, rv)[4], ref[4])            # inputs were not modified by the first call
    with pytest.raises(ValueError):
        th.function([x, y], T.join(0, x, y[:, :5]))(xv, yv)
    with pytest.raises(IndexError):
        th.function([x], x[40])(xv)


def test_gradients_through_views():
    rng = np.random.default_rng(54)
    x = T.ftensor3("x")
    y = T.fmatrix("y")
    r = T.frow("r")
    xv = rng.standard_normal((6, 9, 16)).astype("float32")
    yv = rng.standard_normal((9, 16)).astype("float32")
    rv = rng.standard_normal((1, 16)).astype("float32")
    cost = (T.sum(T.sqr(x[1:3, ::-2, 4])) + T.sum(T.exp(x.reshape((-1, 16))[3:7] * 0.1)) +
            T.sum(T.join(0, y, r, y[:2]) ** 3) + T.sum(T.alloc(r, 3, y.shape[0], 16) * x[:3]) +
            T.sum(T.sqr(T.inc_subtensor(x, y[:2, 1:3], (slice(1, 3), 0, slice(2, 4))))) +
            T.sum(T.set_subtensor(x, r, (2, slice(None, None, 2))) * x) +
            T.sum(T.stack([y, y * 2], axis=1)[:, 1] * y))
    grads = th.grad(cost, [x, y, r])
    f, got, ref = both([x, y, r], [cost] + grads, [xv, yv, rv])
    truth = G.evaluate([x, y, r], [cost] + grads, [xv, yv, rv], wide=True)
    for k, (g, rr, w) in enumerate(zip(got, ref, truth)):
        # the cost adds seven float32 sums of either sign (the oracle's own total is a few bars from the
        # float64 value): held to that value, no farther from it than the oracle is
        assert_within_reference_error(g, rr, w, "gradient %d" % k)


def test_minibatch_slices_of_a_large_matrix():
    """Consecutive row blocks of the configuration-2 matrix reduce to the same
    values as the whole matrix does."""
    import workloads as W
    (val,) = W.c2_inputs("sum_axis1", "full")
    x = T.fmatrix("x")
    parts = [T.sum(x[k * 2048:(k + 1) * 2048], axis=1) for k in range(4)]
    f = th.function([x], [T.join(0, *parts), T.sum(x, axis=1)])
    joined, whole = f(val)
    assert np.array_equal(joined, whole)


@pytest.mark.gpu
def test_shape_entries_are_symbolic_scalars():
    """x.shape[d] is a 0-d int64 variable (Shape_i, theano/compile/ops.py:377-470): it divides
    a sum, scales a tensor (travelling to the kernel by value), names extents for reshape and
    alloc, and follows the array it is called with."""
    rng = np.random.default_rng(3)
    x = T.fmatrix("x")
    n, m = x.shape
    assert n.type.ndim == 0 and n.type.dtype == "int64"
    outs = [T.sum(x, axis=0) / n, x * m + n, T.alloc(np.float32(2.0), m, n) + x.T, x.reshape((m, n)), T.sum(x) / (n * m)]
    f = th.function([x], outs)
    for shape in ((5, 7), (33, 2)):
        xv = rng.standard_normal(shape).astype("float32")
        got = f(xv)
        ref = G.evaluate([x], outs, [xv])
        from conftest import TOL
        for g, r in zip(got, ref):
            # float32 / int64 is a float32 division in C, whatever the result is stored in
            assert_parity(g, r, "shape arithmetic", tol=TOL["float32"])
        assert np.allclose(got[0], xv.astype("float64").sum(0) / shape[0]) and got[3].shape == shape[::-1]
    with pytest.raises(TypeError):
        x.reshape((T.sum(x),))            # a float is not a shape entry


@pytest.mark.gpu
def test_shapes_computed_from_extents_and_scalar_arguments():
    """reshape / alloc take arithmetic over extents (evaluated on the host from array metadata) and integer scalar
    variables (read on the host when the function runs): the idioms x.reshape((x.shape[0], -1)),
    x.reshape((x.shape[0], x.shape[1] * x.shape[2])), alloc(0., n, m + 1) of theano/tensor/basic.py:2769-2960,
    4701-4920, with the gradient flowing back through the reshape."""
    rng = np.random.default_rng(4)
    x = T.ftensor3("x")
    n, m = T.iscalar("n"), T.lscalar("m")
    outs = [x.reshape((x.shape[0], x.shape[1] * x.shape[2])), x.reshape((x.shape[0] * x.shape[1] // 2, 2, -1)),
            T.alloc(np.float32(1.5), x.shape[0] + 1, n, T.maximum(m, 2)), x.reshape((n, -1)) * 2,
            T.alloc(x[0, 0], n * 2 - 1, x.shape[2]), x.flatten(2).reshape((x.shape[0], x.shape[1], x.shape[2])) + 1,
            T.alloc(np.float32(0), T.minimum(x.shape[0], x.shape[1]) % 3, 4)]
    f = th.function([x, n, m], outs)
    for shape, nv, mv in (((4, 6, 5), 8, 3), ((2, 8, 3), 4, 1), ((6, 2, 7), 12, 9)):
        xv = rng.standard_normal(shape).astype("float32")
        got = f(xv, np.int32(nv), np.int64(mv))
        ref = G.evaluate([x, n, m], outs, [xv, np.int32(nv), np.int64(mv)])
        for g, r in zip(got, ref):
            assert_parity(g, r, "computed shapes %s" % (shape,))
        assert got[0].shape == (shape[0], shape[1] * shape[2]) and got[2].shape == (shape[0] + 1, nv, max(mv, 2))
        assert np.array_equal(got[3], xv.reshape(nv, -1) * 2)
    with pytest.raises(ValueError):
        f(np.zeros((4, 6, 5), "float32"), np.int32(7), np.int64(3))        # 120 elements do not split into 7 rows
    with pytest.raises(ValueError):
        th.function([n], T.alloc(np.float32(0), n - 5, 2))(np.int32(3))                # a negative extent
    # the gradient goes back through a computed shape
    w = T.fmatrix("w")
    cost = T.sum(T.sqr(x.reshape((x.shape[0], x.shape[1] * x.shape[2])) * w))
    gx = th.function([x, w], th.grad(cost, x))
    xv, wv = rng.standard_normal((3, 4, 5)).astype("float32"), rng.standard_normal((3, 20)).astype("float32")
    assert np.allclose(gx(xv, wv), (2 * xv.reshape(3, 20) * wv * wv).reshape(3, 4, 5), rtol=1e-5)


@pytest.mark.gpu
def test_symbolic_slices_and_givens_minibatches():
    """x[a:b], x[i], x[::s] with integer scalar variables (theano/tensor/subtensor.py:318-420)
    and the minibatch idiom: a shared data set, an index input and
    givens={x: data[i * n:(i + 1) * n]} (theano/compile/pfunc.py:365-420)."""
    rng = np.random.default_rng(12)
    x = T.fmatrix("x")
    a, b, s, i = T.lscalar("a"), T.lscalar("b"), T.lscalar("s"), T.iscalar("i")
    outs = [x[a:b] * 2.0, x[i], x[::s, 1:], T.sum(x[a:], axis=0), th.grad(T.sum(x[a:b, i] ** 2), x),
            T.set_subtensor(x[a:b, ::2], 1.5), T.inc_subtensor(x[i], x[-1])]
    f = th.function([x, a, b, s, i], outs)
    xv = rng.standard_normal((23, 9)).astype("float32")
    for av, bv, sv, iv in ((3, 11, 2, 4), (0, 23, 5, -2), (-7, -1, 3, 0), (5, 5, 1, 8)):
        got = f(xv, av, bv, sv, iv)
        ref = G.evaluate([x, a, b, s, i], outs, [xv, np.int64(av), np.int64(bv), np.int64(sv), np.int32(iv)])
        for g, r in zip(got, ref):
            assert_parity(g, r, "symbolic index %s" % ((av, bv, sv, iv),))
        assert np.array_equal(got[1], xv[iv]) and np.array_equal(got[2], xv[::sv, 1:])
    with pytest.raises(IndexError):
        f(xv, 0, 1, 1, 9)

    data = th.shared(rng.standard_normal((100, 16)).astype("float32"), name="data")
    w = th.shared(np.zeros(16, "float32"), name="w")
    n = 20
    cost = T.mean(T.sqr(T.sum(x * w, axis=1) - 1.0))
    step = th.function([i], cost, givens={x: data[i * n:(i + 1) * n]}, updates=[(w, w - 0.05 * th.grad(cost, w))])
    dv, wv = data.get_value(), np.zeros(16, "float32")
    for k in (0, 3, 4, 1):
        batch = dv[k * n:(k + 1) * n]
        r = batch @ wv - 1.0
        want = np.mean(r * r)
        wv = wv - 0.05 * (2.0 / n) * (batch.T @ r)
        assert np.allclose(step(k), want, rtol=1e-4)
    assert np.allclose(w.get_value(), wv, rtol=1e-4, atol=1e-6)
    with pytest.raises(TypeError):
        th.function([i], cost, givens={x: T.cast(data[i:i + 2], "float64")})


@pytest.mark.gpu
@pytest.mark.parametrize("k", range(5))
def test_composed_front_ends_on_the_device(k):
    """power / square / sign / rint / deg2rad / ptp, largest / smallest, isclose / allclose,
    floor_div / ceil_intdiv, the shape helpers, stacks, split, zeros / ones and Rebroadcast
    through the HIP path against NumPy (the cases of tests/test_oracle_graph.py)."""
    from test_oracle_graph import _front_end_cases
    name, ins, outs, vals, want = _front_end_cases()[k]
    got = th.function(ins, outs)(*vals)
    for g, w in zip(got, want):
        w = np.asarray(w)
        assert g.shape == w.shape, (name, g.shape, w.shape)
        if w.dtype.kind in "biu":
            assert np.array_equal(g, w), name
        else:
            assert np.allclose(g, w, rtol=1e-12, equal_nan=True), name
    if k == 4:
        x = T.dmatrix("x")
        with pytest.raises(ValueError):
            th.function([x], T.addbroadcast(x, 0) * 2.0)(np.zeros((2, 3)))


def test_reshape_takes_its_shape_as_one_integer_vector():
    """``reshape(x, shape_vector, ndim=n)`` (``theano/tensor/basic.py:4858-4960, 5049-5068``): the vector is an
    argument of the function, read on the host when it runs and never copied to the device; one element may be -1;
    a vector of the wrong length or a shape of the wrong size is a ValueError; the gradient flows back to x.
    ``alloc`` takes elements of such a vector.  Expected values are NumPy's own reshape / broadcast."""
    rng = np.random.default_rng(61)
    x, s = T.fmatrix("x"), T.lvector("s")
    y = x.reshape(s, ndim=3)
    assert y.type.ndim == 3 and y.type.broadcastable == (False, False, False)
    f = th.function([x, s], [y * 2 + 1, T.sum(T.reshape(x, s, ndim=3), axis=(0, 2)), th.grad(T.sum(T.sqr(y)), x)])
    assert not any(type(n.op).__name__ == "HostToHip" and n.inputs[0] is not None and n.inputs[0].type.ndim == 1
                   for n in f.toposort()), "the shape vector went to the device"
    xv = rng.standard_normal((12, 10)).astype("float32")
    for shp in ([2, 6, 10], [5, 4, 6], np.array([3, -1, 8]), np.array([-1, 1, 120], "int32")):
        got = f(xv, shp)
        want = xv.reshape(tuple(int(v) for v in shp))
        assert got[0].shape == want.shape and np.array_equal(got[0], want * 2 + 1)
        assert_parity(got[1], want.astype("float64").sum(axis=(0, 2)).astype("float32"), "sum of the reshaped array")
        assert np.array_equal(got[2], 2 * xv)
    for bad in ([12, 10], [7, 2, 9], [-1, -1, 10]):
        with pytest.raises(ValueError):
            f(xv, bad)
    with pytest.raises(ValueError, match="ndim"):
        T.reshape(x, s)                                    # the rank must be known when the graph is built
    with pytest.raises(TypeError):
        T.reshape(x, T.fvector(), ndim=2)                  # theano/tensor/basic.py:4888-4892
    assert T.reshape(x, T.constant(np.array([3, 40]))).type.ndim == 2      # a constant vector tells its length
    # elements of a shape vector as alloc's extents, and arithmetic over them
    v = T.fvector("v")
    g = th.function([v, s], T.alloc(v, s[0], s[1] * 2, v.shape[0]) + np.float32(1))
    vv = rng.standard_normal(7).astype("float32")
    got = g(vv, [3, 2, 99])
    assert got.shape == (3, 4, 7) and np.array_equal(got, np.broadcast_to(vv, (3, 4, 7)) + np.float32(1))
    with pytest.raises(ValueError):
        g(vv, [3])
    # the vector may also be computed on the device: then its values are fetched
    h = th.function([x, s], x.reshape(s * 2, ndim=2))
    assert np.array_equal(h(xv, [2, 15]), xv.reshape(4, 30))
