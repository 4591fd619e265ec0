"""Cases of the reference's own elemwise tests (``theano/tensor/tests/test_elemwise.py``) that the other test
files do not already restate: graph-level ones run on the CPU, value-level ones on the device."""
import numpy as np
import pytest

import theano_amd as th
from theano_amd import scalar as scal
from theano_amd import tensor as T

AXES = [None, 0, 1, [0, 1], np.array(1), [np.array(0), np.array(1)]]


def test_reduce_axes_of_every_kind():
    """``test_reduce_axes`` (:110-153): ints, lists, 0-d arrays and lists of 0-d arrays as ``axis`` of sum, mean,
    max, min, argmax and var, as functions and as methods."""
    for a in AXES:
        x = T.matrix()
        for res in (x.sum(a), x.mean(a), x.max(a), x.min(a), x.argmax(a), x.var(a), T.argmin(x, a)):
            want = 0 if (a is None or isinstance(a, list)) else 1
            assert res.type.ndim == want, (a, res)


def test_fill_methods_and_gradients_build():
    """``test_fill_var`` (:293), ``test_fill_grad`` (:297), ``test_elemwise_grad_broadcast`` (:1300),
    ``test_clip_grad_int`` (:1313), ``test_elemwise_grad_bool`` (:1186): graphs that once crashed while built."""
    T.matrix().fill(3)
    x = T.TensorType(th.config.floatX, [0, 1, 0])("x")
    y = T.TensorType(th.config.floatX, [0, 1, 0])("y")
    th.grad(T.second(x, y).sum(), y)
    x = T.TensorType("float32", (True, False, False, False))("x")
    y = T.TensorType("float32", (True, True, False, False))("y")
    th.grad(T.tanh(x).sum(), x)
    th.grad(T.tanh(x + y).sum(), y)
    gx, gy = th.grad(T.tanh(x + y).sum(), [x, y])
    assert gx.type.broadcastable == x.type.broadcastable and gy.type.broadcastable == y.type.broadcastable
    a, b, c = T.iscalar(), T.iscalar(), T.iscalar()
    th.grad(T.clip(a, b, c), [a, b, c])
    p, q = T.scalar(dtype="bool"), T.bscalar()
    th.grad(p * q, [p, q])


def test_mean_dtypes():
    """``T_mean_dtype`` (:969-1035): a mean is float64 for discrete inputs and keeps floating and complex dtypes; a
    custom dtype decides the result the same way, unsuitable ones raise TypeError from the inner sum, and the
    gradient can be taken wherever the result is real."""
    axes = [None, 0, 1, [], [0], [1], [0, 1]]
    for idx, dtype in enumerate(scal.all_dtypes):
        m = T.matrix(dtype=dtype).mean(axis=axes[idx % len(axes)])
        assert m.dtype == ("float64" if dtype in scal.discrete_dtypes else dtype), (dtype, m.dtype)
    idx = compiled = 0
    for input_dtype in scal.all_dtypes:
        x = T.matrix(dtype=input_dtype)
        for sum_dtype in scal.all_dtypes:
            axis = axes[idx % len(axes)]
            try:
                mean_var = x.mean(dtype=sum_dtype, axis=axis)
            except TypeError:
                pass
            else:
                assert mean_var.dtype == ("float64" if sum_dtype in scal.discrete_dtypes else sum_dtype)
                if ("complex" in input_dtype or "complex" in sum_dtype) and input_dtype != sum_dtype:
                    continue
                compiled += 1
                if "complex" not in mean_var.dtype:
                    th.grad(mean_var.sum(), x, disconnected_inputs="ignore")
            idx += 1
    assert compiled > 100


def test_comparisons_refuse_truth_tests_and_python_protocols():
    """``a < b < c`` must not silently drop ``a < b`` (``theano/tensor/var.py:52-95``); divmod, ceil / floor /
    trunc, the math methods, norm, squeeze, transpose, copy (``var.py:196-256, 300-330, 629-636, 686-698, 817``)."""
    import math
    a, b, c = T.vector("a"), T.vector("b"), T.vector("c")
    with pytest.raises(TypeError, match="boolean operations"):
        a < b < c
    with pytest.raises(TypeError):
        bool(a >= b)
    assert bool(a) and bool(a + b)
    q, r = divmod(a, b)
    assert str(q.owner.op.scalar_op) == "int_div" and str(r.owner.op.scalar_op) == "mod"
    q, r = divmod(3.0, b)
    assert q.owner.inputs[1] is b or q.owner.inputs[1].owner is not None
    for fn, name in ((math.ceil, "ceil"), (math.floor, "floor"), (math.trunc, "trunc")):
        assert str(fn(a).owner.op.scalar_op) == name
    for name in ("arccos", "arccosh", "arcsin", "arcsinh", "arctan", "arctanh", "ceil", "cos", "cosh", "deg2rad", "exp",
                 "exp2", "expm1", "floor", "log", "log10", "log1p", "log2", "rad2deg", "sin", "sinh", "sqrt", "tan",
                 "tanh", "trunc"):
        assert getattr(a, name)().owner.op is getattr(T, name)(a).owner.op or \
            getattr(a, name)().owner.op == getattr(T, name)(a).owner.op, name
    m = T.TensorType("float32", (False, True, False))("m")
    assert m.squeeze().type.broadcastable == (False, False)
    assert m.transpose(2, 0, 1).type.broadcastable == (False, False, True)
    assert m.transpose().type.broadcastable == (False, True, False) and m.swapaxes(0, 1).type.broadcastable == (True, False, False)
    assert m.norm(2, axis=0).type.ndim == 2 and m.norm(1, axis=0, keepdims=True).type.ndim == 3
    with pytest.raises(NotImplementedError):
        m.norm(0)
    assert m.copy(name="again").name == "again" and m.ravel().type.ndim == 1
    assert m.clip(0, 1).type == m.type and m.round().type == m.type and m.ptp(0).type.ndim == 2
    # size: the product of the extents, a 0-d int64 (var.py:289-290)
    assert m.size.type.dtype == "int64" and m.size.type.ndim == 0 and T.scalar().size.data == 1


@pytest.mark.gpu
def test_same_input_twice_six_operands_and_rank_limit():
    """``test_same_inputs`` (:320): ``x + x``; ``test_input_dimensions_overflow`` (:1215): six vectors of 2048
    elements added; ``test_too_big_rank`` (:104): a DimShuffle past the array rank limit raises ValueError when run."""
    rng = np.random.default_rng(0)
    x = T.matrix("x")
    xv = rng.standard_normal((2, 2)).astype("float32")
    assert np.array_equal(th.function([x], x + x)(xv), xv + xv)
    vs = [T.vector(n) for n in "abcdef"]
    s = vs[0]
    for v in vs[1:]:
        s = s + v
    vals = [rng.standard_normal(2 ** 11).astype("float32") for _ in vs]
    want = vals[0]
    for v in vals[1:]:
        want = want + v
    assert np.array_equal(th.function(vs, s)(*vals), want)
    v = T.vector("v")
    f = th.function([v], v.dimshuffle(*(("x",) * 8 + (0,))) * 2)
    with pytest.raises(ValueError, match="dimensions"):
        f(np.zeros(3, "float32"))


@pytest.mark.gpu
def test_gradients_of_all_any_clip_and_a_hinge_loss():
    """``TestBitOpReduceGrad`` (:1154-1182): gradients of all / any are zeros of the input's shape;
    ``test_clip_grad`` (:1251) at a value below, between and above the bounds; ``test_gt_grad`` (:1226): the
    hinge loss whose gradient once failed to be recognised as valid (the dot written as a broadcast product);
    ``test_mean_precision`` (:1037): the mean of [1e8, 1, -1e8] in float32 is 1/3."""
    rng = np.random.default_rng(1)
    x = T.bmatrix("x")
    x_random = rng.binomial(n=1, p=0.5, size=(5, 7)).astype("int8")
    for red in (x.all(), x.any()):
        f = th.function([x], th.grad(red, x))
        for xv in (x_random, np.zeros_like(x_random), np.ones_like(x_random)):
            g = f(xv)
            assert g.shape == xv.shape and np.all(g == 0)
    v, lo, hi = T.dvector("v"), T.dscalar("lo"), T.dscalar("hi")
    gv, glo, ghi = th.function([v, lo, hi], th.grad(T.clip(v, lo, hi).sum(), [v, lo, hi]))(
        np.asarray([-1.0, 0.5, 2.0]), 0.0, 1.0)
    assert np.array_equal(gv, [0.0, 1.0, 0.0]) and glo == 1.0 and ghi == 1.0
    inp, wrong_in = T.vector("inp"), T.vector("wrong")
    W = th.shared(np.random.RandomState(1234).uniform(-1, 1, (2, 2)).astype("float32"), name="weights")
    correct = T.sum(inp.dimshuffle(0, "x") * W, axis=0)
    wrong = T.sum(wrong_in.dimshuffle(0, "x") * W, axis=0)
    scores = T.ones_like(correct) - correct + wrong
    cost = (scores * (scores > 0)).sum()
    g = th.function([inp, wrong_in], th.grad(cost, inp))
    iv, wv = np.asarray([0.3, -0.2], "float32"), np.asarray([0.1, 0.4], "float32")
    Wv = W.get_value()
    sc = 1 - iv @ Wv + wv @ Wv
    assert np.allclose(g(iv, wv), -(Wv * (sc > 0)).sum(axis=1), rtol=1e-5, atol=1e-6)
    m = th.shared(np.asarray([1e8, 1, -1e8], dtype="float32"))
    assert np.allclose(th.function([], m.mean())(), 1.0 / 3)


@pytest.mark.gpu
def test_gpu_optimizer_cases_of_the_reference():
    """``theano/gpuarray/tests/test_opt.py``: ``test_reduce`` (:143) - sum / prod with a float32 accumulator, max
    and min over axis 0 run as one reduction node; ``test_local_gpu_elemwise_careduce`` (:362) - sqr / abs producers
    end up as the reduction's ``pre_scalar_op`` for axis None, 0 and 1; ``test_local_gpu_elemwise`` (:457) - int8 +
    float32 + float32 is one kernel whether the Composite is built by fusion or by the user, with several results,
    and on every other row of its operands."""
    from theano_amd.hip import HipCAReduce, HipElemwise
    rng = np.random.default_rng(3)

    def kernels(f, cls):
        return [n for n in f.toposort() if isinstance(n.op, cls)]

    val = rng.random((10, 11)).astype("float32")
    for method, param in (("sum", dict(acc_dtype="float32")), ("prod", dict(acc_dtype="float32")), ("max", {}), ("min", {})):
        m = T.fmatrix()
        f = th.function([m], getattr(m, method)(axis=0, **param))
        res = f(val)
        assert res.shape == (11,) and np.allclose(res, getattr(val, method)(axis=0), rtol=1e-5)
        assert len(kernels(f, HipCAReduce)) == 1 and not kernels(f, HipElemwise)

    x = T.matrix()
    data = rng.random((3, 4)).astype(th.config.floatX)
    for fn, pre in ((lambda v, axis: (v * v).sum(axis=axis), "sqr"), (lambda v, axis: abs(v).sum(axis=axis), "abs"),
                    (lambda v, axis: abs(v).max(axis=axis), "abs")):
        for axis in (None, 0, 1):
            f = th.function([x], fn(x, axis))
            (red,) = kernels(f, HipCAReduce)
            assert not kernels(f, HipElemwise) and pre in str(red.op.pre_scalar_op), (pre, axis, red.op)
            assert np.allclose(fn(data, axis), f(data), rtol=1e-5)

    a, b, c = T.bmatrix(), T.fmatrix(), T.fmatrix()
    a_v = (rng.random((4, 5)) * 10).astype("int8")
    b_v = (rng.random((4, 5)) * 10).astype("float32")
    c_v = (rng.random((4, 5)) * 10).astype("float32")
    f = th.function([a, b, c], a + b + c)
    assert len(kernels(f, HipElemwise)) == 1 and np.allclose(f(a_v, b_v, c_v), a_v + b_v + c_v)
    a_s, b_s, c_s = scal.int8(), scal.float32(), scal.float32()
    out_op = T.Elemwise(scal.Composite([a_s, b_s, c_s], [a_s + b_s + c_s]))
    f = th.function([a, b, c], out_op(a, b, c))
    assert len(kernels(f, HipElemwise)) == 1 and np.allclose(f(a_v, b_v, c_v), a_v + b_v + c_v)
    # several results (the part the reference's test never reaches: GpuElemwise took one output only)
    a_s = scal.float32()
    af = T.fmatrix()
    outs_op = T.Elemwise(scal.Composite([a_s, b_s, c_s], [a_s + b_s, a_s * c_s]))
    f = th.function([af, b, c], outs_op(af, b, c))
    assert len(kernels(f, HipElemwise)) == 1
    av = a_v.astype("float32")
    o0, o1 = f(av, b_v, c_v)
    assert np.allclose(o0, av + b_v) and np.allclose(o1, av * c_v)
    cs = th.shared(c_v)
    o0, o1 = th.function([af, b], outs_op(af[::2], b[::2], cs[::2]))(av, b_v)
    assert np.allclose(o0, av[::2] + b_v[::2]) and np.allclose(o1, av[::2] * c_v[::2])


def test_oracle_lets_an_extent_of_one_pass_beside_an_empty_operand():
    """``Elemwise.perform`` (``theano/tensor/elemwise.py:720-751``) raises only when the largest extent of a
    dimension is not 1; ``[] + [1]`` is the `empty` good case of every binary tester
    (``theano/tensor/tests/test_basic.py:680``).  (2, 3) + (1, 3) typed without broadcasting still raises."""
    from oracle import graph_ref as G
    a, b = T.vector("a"), T.vector("b")
    (out,) = G.evaluate([a, b], [a + b], [np.asarray([], "float32"), np.asarray([1], "float32")])
    assert out.shape == (0,) and out.dtype == np.float32
    x, y = T.matrix("x"), T.matrix("y")
    with pytest.raises(ValueError, match="mis-match"):
        G.evaluate([x, y], [x + y], [np.zeros((2, 3), "float32"), np.zeros((1, 3), "float32")])


@pytest.mark.gpu
def test_named_input_patterns_of_the_binary_testers():
    """``_good_broadcast_binary_normal`` (``theano/tensor/tests/test_basic.py:664-682``) by name - same_shapes,
    not_same_dimensions, scalar, row, column, integers, uint32, uint16, dtype_mixup_1 / 2, complex1 / 2, empty -
    for add, sub, mul, true_div, maximum and minimum against the oracle; and the two must-raise cases (:686-688)."""
    from oracle import graph_ref as G
    from conftest import assert_parity
    rng = np.random.default_rng(11)
    rand = lambda *s: rng.uniform(-1, 1, s).astype("float32")
    randint = lambda *s: rng.integers(-5, 6, s).astype("int32")
    randc = lambda *s: (rng.uniform(-1, 1, s) + 1j * rng.uniform(-1, 1, s)).astype("complex64")
    cases = dict(
        same_shapes=(rand(2, 3), rand(2, 3)), not_same_dimensions=(rand(2, 2), rand(2)), scalar=(rand(2, 3), rand(1, 1)),
        row=(rand(2, 3), rand(1, 3)), column=(rand(2, 3), rand(2, 1)), integers=(randint(2, 3), randint(2, 3)),
        uint32=(rng.integers(0, 9, (2, 3)).astype("uint32"), rng.integers(1, 9, (2, 3)).astype("uint32")),
        uint16=(rng.integers(0, 9, (2, 3)).astype("uint16"), rng.integers(1, 9, (2, 3)).astype("uint16")),
        dtype_mixup_1=(rand(2, 3), randint(2, 3)), dtype_mixup_2=(randint(2, 3), rand(2, 3)),
        complex1=(randc(2, 3), randc(2, 3)), complex2=(randc(2, 3), rand(2, 3)),
        empty=(np.asarray([], dtype="float32"), np.asarray([1], dtype="float32")))
    for name, (av, bv) in cases.items():
        # as the testers do: a dimension is typed broadcastable exactly when its extent is 1, except in `empty`
        bc = lambda v: [s == 1 for s in v.shape] if name != "empty" else [False] * v.ndim
        a, b = T.TensorType(str(av.dtype), bc(av))("a"), T.TensorType(str(bv.dtype), bc(bv))("b")
        bsafe = T.switch(T.eq(b, 0), T.ones_like(b), b) if bv.dtype.kind in "iu" else b
        outs = [a + b, a - b, a * b, a / bsafe]
        if av.dtype.kind != "c":
            outs += [T.maximum(a, b), T.minimum(a, b)]
        got = th.function([a, b], outs)(av, bv)
        ref = G.evaluate([a, b], outs, [av, bv])
        for k, (g, r) in enumerate(zip(got, ref)):
            assert_parity(g, r, "%s op %d" % (name, k))
    x, y = T.matrix("x"), T.matrix("y")
    f = th.function([x, y], x + y)
    for bad in ((rand(2, 3), rand(3, 2)), (rand(2, 3), rand(1, 2))):
        with pytest.raises(ValueError):
            f(*bad)


def test_composite_cases_of_the_scalar_tests():
    """``theano/scalar/tests/test_basic.py`` ``test_composite`` (:72-184): ``clone_float32`` leaves no float16
    variable, nested Composites are inlined, constants stay literals of the code, ``make_node`` accepts variables
    of other types and rebuilds, and the values of `test_straightforward`, `test_with_constants` and
    `test_many_outputs` come out of the oracle's evaluation of the Composite."""
    from theano_amd import gof
    from theano_amd.scalar import Composite
    from oracle import graph_ref as G

    def has_f16(comp):
        vs = set(comp.inputs) | set(comp.outputs)
        for n in gof.io_toposort(comp.inputs, comp.outputs):
            vs |= set(n.inputs) | set(n.outputs)
        return any(v.type.dtype == "float16" for v in vs)

    w, x, y = scal.int8(), scal.float16(), scal.float32()
    cz = Composite([x, y], [scal.tanh(x + scal.cast(y, "float16"))])
    c = Composite([w, x, y], [cz(x, y) - cz(x, y) ** 2 + scal.cast(x, "int16") + scal.cast(x, "float32") +
                              scal.cast(w, "float16") - scal.constant(np.float16(1.0))])
    assert has_f16(c) and not has_f16(c.clone_float32())
    v, w, x, y, z = scal.uint8(), scal.float16(), scal.float16(), scal.float16(), scal.float16()
    c = Composite([v, w, x, y, z], [scal.switch(v, scal.mul(w, x, y), z)])
    assert has_f16(c) and not has_f16(c.clone_float32())
    assert [i.type.dtype for i in c.clone_float32().inputs] == ["uint8"] + ["float32"] * 4

    x, y, z = scal.float64("x"), scal.float64("y"), scal.float64("z")
    C = Composite([x, y], [x + y])
    CC = Composite([x, y], [C(x * y, y)])
    assert not isinstance(CC.outputs[0].owner.op, Composite)
    e = scal.mul(scal.add(70.0, y), scal.div_proxy(x, y))
    node = Composite([x, y], [e]).make_node(x, y)
    assert "70.0" in node.op.c_code(node, ["x", "y"], ["z"])

    def run(comp, *vals):
        ins = [T.TensorType(i.type.dtype, ())() for i in comp.inputs]
        outs = T.Elemwise(comp)(*ins)
        outs = outs if isinstance(outs, (list, tuple)) else [outs]
        return [float(o) for o in G.evaluate(ins, list(outs), [np.asarray(v, i.type.dtype) for v, i in zip(vals, ins)])]

    assert run(Composite([x, y], [scal.mul(scal.add(x, y), scal.div_proxy(x, y))]), 1.0, 2.0) == [1.5]
    assert run(Composite([x, y], [e]), 1.0, 2.0) == [36.0]
    assert run(Composite([x, y, z], [x + y + z, x + y * z, x / y]), 1.0, 2.0, 3.0) == [6.0, 7.0, 0.5]
    # test_make_node_continue_graph (:165-184): operands that are results of other scalar computation
    si0, si1, si2 = scal.int8(), scal.int8(), scal.float32()
    sop = Composite([si0, si1, si2], [(si0 * si1) / si2])
    a, b, cc, d = scal.int8(), scal.int8(), scal.float32(), scal.float32()
    rebuilt = sop.make_node(a * d, b, cc)
    assert rebuilt.op.inputs_type[0].dtype == "float32"


def test_softmax_quotient_in_both_spellings_compiles_to_one_row_node(dry_run):
    """``Test_softmax_opt.test_basic`` and ``test_basic_keepdims``
    (``theano/tensor/nnet/tests/test_nnet.py:1472-1505``): ``exp(c) / exp(c).sum(axis=1)`` with the sum brought back
    by ``dimshuffle(0, 'x')`` or by ``keepdims=True`` is recognised as the softmax op - here: one row-chain node
    and no division node beside it."""
    for spell in (lambda c: T.exp(c) / T.exp(c).sum(axis=1).dimshuffle(0, "x"),
                  lambda c: T.exp(c) / T.exp(c).sum(axis=1, keepdims=True)):
        c = T.matrix()
        f = th.function([c], spell(c))
        work = [type(n.op).__name__ for n in f.toposort() if type(n.op).__name__.startswith("Hip")
                and type(n.op).__name__ not in ("HostToHip", "HipToHost")]
        assert work == ["HipRowChain"], work


@pytest.mark.gpu
def test_bitwise_operators_on_signed_integers():
    """``test_bitwise`` (``theano/tensor/tests/test_basic.py:4772-4819``): ``|``, ``^``, ``&`` and ``~`` on int8 ..
    int64 vectors against Python's operators on the same arrays, and ``xor_inplace`` leaves its result in the
    caller's array as well."""
    from theano_amd.tensor import inplace
    for dtype in ("int8", "int16", "int32", "int64"):
        x, y = T.vector(dtype=dtype), T.vector(dtype=dtype)
        l, r = np.asarray([0, 0, 1, 1], dtype=dtype), np.asarray([0, 1, 0, 1], dtype=dtype)
        for expr, want in ((x | y, l | r), (x ^ y, l ^ r), (x & y, l & r)):
            v = th.function([x, y], expr)(l, r)
            assert v.dtype == np.dtype(dtype) and np.array_equal(v, want), (dtype, v, want)
        v = th.function([x, y], inplace.xor_inplace(x, y), accept_inplace=True)(l, r)
        assert np.array_equal(v, [0, 1, 1, 0]) and np.array_equal(l, [0, 1, 1, 0])     # "test the in-place stuff"
        fn = th.function([x], ~x)
        top = np.iinfo(dtype).max
        for vals in ([0, 0, 1, 1], [0, 1, 0, 1], [-1, top, top - 1, np.iinfo(dtype).min]):
            a = np.asarray(vals, dtype=dtype)
            assert np.array_equal(fn(a), ~a), (dtype, a)
