"""Host-side mirror of the reference's Op interface: node construction, type
inference, error behaviour, gradients' graph structure and what the rewrite
pipeline (lift + fuse) produces."""
import os

import numpy as np
import pytest

import theano_amd as th
from theano_amd import scalar as scal
from theano_amd import tensor as T
from theano_amd.hip import HipCAReduce, HipElemwise, HipToHost, HostToHip
from theano_amd.tensor.elemwise import CAReduce, DimShuffle, Elemwise, Sum


def ops_of(f, cls):
    return [n for n in f.toposort() if isinstance(n.op, cls)]


def test_elemwise_make_node_pads_ranks_and_ands_broadcast_flags():
    x, v = T.fmatrix(), T.fvector()
    z = x + v
    assert z.type.broadcastable == (False, False) and z.type.dtype == "float32"
    assert isinstance(z.owner.inputs[1].owner.op, DimShuffle)
    assert z.owner.inputs[1].owner.op.new_order == ("x", 0)
    r, c = T.frow(), T.fcol()
    assert (r * c).type.broadcastable == (False, False)
    assert (r + r).type.broadcastable == (True, False)


def test_props_give_equality_and_hash():
    assert Elemwise(scal.add) == Elemwise(scal.add) and hash(Elemwise(scal.add)) == hash(Elemwise(scal.add))
    assert Elemwise(scal.add) != Elemwise(scal.mul)
    assert Sum(axis=(0,)) == Sum(axis=[0]) and Sum(axis=0) != Sum(axis=1)
    assert DimShuffle((False, False), (1, 0)) == DimShuffle((False, False), [1, 0])
    assert HipElemwise(scal.add) != Elemwise(scal.add)


def test_python_literals_pick_the_smallest_dtype():
    x = T.imatrix()
    assert (x % 97).type.dtype == "int32" and (x % 97).owner.inputs[1].owner.inputs[0].type.dtype == "int8"
    f = T.fmatrix()
    assert (f + 1e-5).type.dtype == "float32"  # floatX = float32 keeps float literals narrow
    assert (f * 2).type.dtype == "float32"
    assert (x / 2).type.dtype == "float32"     # `/` is true division: floatX for two integer operands (var.py:199-200)
    assert x.__div__(2).type.dtype == "int32"  # Python 2's `/`: integer division under int_division='int'
    assert T.true_div(x, 2).type.dtype == "float32"


def test_dimshuffle_rules():
    x = T.TensorType("float32", (False, True, False))()
    assert x.dimshuffle(2, 0).type.broadcastable == (False, False)
    assert x.dimshuffle(0, "x", 2, 1).type.broadcastable == (False, True, False, True)
    with pytest.raises(ValueError):
        x.dimshuffle(1, 2)  # drops a non-broadcastable dimension
    with pytest.raises(ValueError):
        x.dimshuffle(0, 0, 2)


def test_careduce_axis_normalisation_and_infer_shape():
    x = T.ftensor3()
    s = x.sum(axis=(-1, 0))
    assert s.owner.op.axis == (0, 2) and s.type.ndim == 1
    assert s.owner.op.infer_shape(s.owner, [(4, 5, 6)]) == ([5],)
    with pytest.raises(ValueError):
        x.sum(axis=3)
    assert T.all(x > 0).type.dtype == "bool" and T.any(x).owner.inputs[0].owner.op.scalar_op == scal.neq


def test_bit_ops_reject_floats_and_sub_rejects_bool():
    with pytest.raises(TypeError):
        T.fmatrix() & T.fmatrix()
    b = T.TensorType("bool", (False,))()
    with pytest.raises(TypeError):
        b - b
    assert (b + b).type.dtype == "bool"


def test_fusion_collapses_an_elementwise_chain_to_one_composite():
    x, y, z = T.fmatrix("x"), T.fmatrix("y"), T.fmatrix("z")
    f = th.function([x, y, z], T.sigmoid(x * y + z) * x + 2.0)
    ew = ops_of(f, HipElemwise)
    assert len(ew) == 1 and isinstance(ew[0].op.scalar_op, scal.Composite)
    assert len(ew[0].inputs) == 3                      # repeated x is one operand, the constant is a literal
    assert len(ops_of(f, HostToHip)) == 3 and len(ops_of(f, HipToHost)) == 1


def test_fusion_respects_broadcast_pattern_and_client_count():
    x, s = T.fmatrix("x"), T.TensorType("float32", (True, True))("s")
    # sin(s) has a scalar-shaped output: it is not pulled into the matrix-shaped consumer
    # (case 71 of theano/tensor/tests/test_opt.py:1107-1111)
    f = th.function([x, s], x + T.sin(s))
    assert len(ops_of(f, HipElemwise)) == 2
    # an expensive producer with two clients is computed once, not duplicated: without the sibling
    # merge it keeps a kernel of its own, with it both consumers and the producer are one kernel
    e = T.exp(x)
    g = th.function([x], [e + 1, e * 2])
    (only,) = ops_of(g, HipElemwise)
    from theano_amd import gof
    inner = gof.io_toposort(only.op.scalar_op.inputs, only.op.scalar_op.outputs)
    assert len(only.outputs) == 2 and sum(1 for n in inner if n.op == scal.exp) == 1


def test_config1_is_one_kernel_with_scalars_passed_by_value():
    import workloads
    ins, outs = workloads.c1_graph()
    f = th.function(ins, outs)
    ew = ops_of(f, HipElemwise)
    assert len(ew) == 1 and str(ew[0].op.scalar_op) == "Composite{mul(scalar_sigmoid(add(mul(i0, i1), i2)), i1)}"
    assert len(ops_of(f, HostToHip)) == 1              # a and b stay on the host


def test_reduce_prologue_fusion_and_sibling_merge():
    x, y = T.fmatrix("x"), T.fmatrix("y")
    f = th.function([x, y], T.sum(T.sqr(x - y), axis=1))
    assert len(ops_of(f, HipElemwise)) == 0
    (red,) = ops_of(f, HipCAReduce)
    assert red.op.pre_scalar_op is not None and len(red.inputs) == 2
    g = th.function([x], [T.any(x > 0), T.all(x > 0)])
    (red,) = ops_of(g, HipCAReduce)
    assert len(red.outputs) == 2 and red.op.scalar_ops == (scal.or_, scal.and_)


def test_reductions_sharing_only_a_broadcast_operand_stay_apart(dry_run):
    """Two reductions over arrays of different run-time shape that share a (1, C) weight must not
    merge into one kernel: a common operand that is broadcast in both proves nothing about the
    other operands' extents."""
    x, y = T.fmatrix("x"), T.fmatrix("y")
    w = T.frow("w")
    f = th.function([x, y, w], [T.sum(T.exp(x) * w), T.sum(T.tanh(y) * w)])
    assert len(ops_of(f, HipCAReduce)) == 2
    f(np.zeros((4, 8), "float32"), np.zeros((6, 8), "float32"), np.zeros((1, 8), "float32"))
    # a shared full-shaped operand still merges the two
    g = th.function([x, w], [T.sum(T.exp(x) * w), T.sum(T.tanh(x) * w)])
    (red,) = ops_of(g, HipCAReduce)
    assert len(red.outputs) == 2


def test_gradient_graph_contains_only_path_ops():
    x, y = T.fmatrix("x"), T.frow("y")
    cost = T.sum(T.tanh(x * y))
    gx, gy = th.grad(cost, [x, y])
    assert gx.type == x.type and gy.type == y.type   # the broadcast row gets its gradient summed back
    from theano_amd import gof
    for node in gof.io_toposort([x, y], [gx, gy]):
        assert isinstance(node.op, (Elemwise, CAReduce, DimShuffle)), node.op
    with pytest.raises(TypeError):
        th.grad(x, x)  # non-scalar cost


def test_lifter_refuses_ops_without_a_device_implementation():
    from theano_amd.gof import Apply, Op

    class HostOnly(Op):
        def make_node(self, x):
            return Apply(self, [x], [x.type()])
    x = T.fmatrix()
    with pytest.raises(NotImplementedError, match="no HIP implementation"):
        th.function([x], HostOnly()(x))


def test_host_ops_have_no_compute_path():
    x = T.fmatrix()
    node = (x + x).owner
    with pytest.raises(NotImplementedError):
        node.op.perform(node, [np.zeros((2, 2), "float32")] * 2, [[None]])


def test_device_outputs_and_inputs(dry_run):
    from theano_amd.hip import HipArray
    x = T.fmatrix()
    f = th.function([x], th.Out(x * 2, device=True))
    assert len(ops_of(f, HipToHost)) == 0
    out = f(np.zeros((3, 4), "float32"))
    assert isinstance(out, HipArray) and out.shape == (3, 4)
    out2 = f(out)  # a device array is accepted for a host-typed input
    assert isinstance(out2, HipArray)


def test_factors_constant_along_the_reduced_axes_leave_the_sum():
    """sum(c * x / d, axis) with c, d broadcast along the reduced axes becomes
    (c / d)' * sum(x, axis): one plain sum instead of a product per element, and
    the same values as the unrewritten graph within float32 rounding."""
    from theano_amd import gof
    from theano_amd.tensor import opt as topt
    from oracle import graph_ref as G
    t4 = T.TensorType("float32", (False,) * 4)
    pc = T.TensorType("float32", (True, False, True, True))
    x, g = t4("x"), t4("g")
    gamma, std = pc("gamma"), pc("std")
    outs = [T.sum(-(g * (gamma * x)) / (std * std), axis=(0, 2, 3)),
            T.sum((g / std) * x, axis=(0, 2, 3), keepdims=True),
            T.sum(g * x, axis=(0, 2, 3))]                      # nothing to pull out: left alone
    rng = np.random.default_rng(5)
    vals = [rng.standard_normal((5, 7, 3, 4)).astype("float32"), rng.standard_normal((5, 7, 3, 4)).astype("float32"),
            rng.uniform(0.5, 2, (1, 7, 1, 1)).astype("float32"), rng.uniform(0.5, 2, (1, 7, 1, 1)).astype("float32")]
    ref = G.evaluate([x, g, gamma, std], outs, vals)
    fg = gof.FunctionGraph([x, g, gamma, std], outs)
    topt.canonicalize(fg)
    sums = [n for n in fg.toposort() if isinstance(n.op, Sum)]
    for n in sums:                                                # every remaining sum reads g * x only
        (prod,) = n.inputs
        assert isinstance(prod.owner.op, Elemwise) and isinstance(prod.owner.op.scalar_op, scal.Mul)
        assert set(prod.owner.inputs) == {fg.inputs[0], fg.inputs[1]}
    got = G.evaluate(fg.inputs, fg.outputs, vals)
    for a, b in zip(got, ref):
        assert a.shape == b.shape and a.dtype == b.dtype
        np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-6)
    # integer sums are left alone: the int64 sum of an int32 product wraps differently from the product of sums
    xi = T.imatrix("xi")
    ci = T.TensorType("int32", (False, True))("ci")
    fg = gof.FunctionGraph([xi, ci], [T.sum(xi * ci, axis=1)])
    topt.canonicalize(fg)
    (n,) = [n for n in fg.toposort() if isinstance(n.op, Sum)]
    assert isinstance(n.inputs[0].owner.op.scalar_op, scal.Mul)


def test_batchnorm_gradient_is_one_statistics_pass_and_one_elementwise_pass(dry_run):
    """Configuration 5's gradient graph: per-channel factors leave the sums; the mean leaves the
    prologue of sum(g * (x - mean)), which becomes sum(g * x) - mean * sum(g); that reduction then
    depends on the statistics of x through its epilogue only and joins their pass.  One kernel reads
    x and g once and yields mean, standard deviation and the three per-channel sums (four float64
    accumulators - sum(x), sum((x - c)^2), sum(g), sum(g x): every sum the two epilogues need is one of them -
    the per-channel algebra chained in its epilogue, gamma a per-result device operand); one elementwise
    kernel follows.  The first is told that x and g are read again (they stay cacheable).  With the
    rewrite switched off the graph keeps its two statistics passes."""
    import workloads
    ins, outs = workloads.c5_graph(forward=False)

    def kernels_of(f):
        return [n for n in f.toposort() if isinstance(n.op, (HipElemwise, HipCAReduce)) and
                any(not any(i.type.broadcastable) for i in n.inputs if hasattr(i.type, "broadcastable") and i.type.ndim)]

    # (the form that runs when a channel's elements do not fit on chip; otherwise the whole graph is one held chain)
    with th.config.change_flags(held_chains=False):
        f = th.function(ins, [th.Out(o, device=True) for o in outs])
    kernels = kernels_of(f)
    assert [type(n.op) for n in kernels] == [HipCAReduce, HipElemwise]
    stats = kernels[0]
    assert len(stats.op.scalar_ops) == 4 and stats.op.acc_dtypes.count("float64") == 4
    n_red = len(stats.inputs) - stats.op.n_extra
    assert [str(i.type.dtype) for i in stats.inputs[:n_red] if not any(i.type.broadcastable)] == ["float16", "float16"]
    extras = stats.inputs[n_red:]
    assert any(type(e.type).__name__ == "HipArrayType" for e in extras)
    assert len(kernels[0].tag["reused_in"]) >= 2 and len(kernels[1].tag["reused_in"]) == 0
    small = workloads.c5_inputs("small")
    f(*small)                                      # plans and compiles every kernel (dry run)
    with th.config.change_flags(merge_dependent_reductions=False, held_chains=False):
        g = th.function(ins, [th.Out(o, device=True) for o in outs])
    assert [type(n.op) for n in kernels_of(g)] == [HipCAReduce, HipCAReduce, HipElemwise]


def test_batchnorm_graphs_become_one_held_chain(dry_run):
    """Per-channel statistics followed by the normalisation (reductions over axes (0, 2, 3) whose results
    feed elementwise work on the same array) form one HipRowChain over those axes: the kernel keeps each
    channel's elements on chip between the statistics and the store.  The three sums of the forward graph
    share one loop, the store is the second; a graph that only takes the statistics reads its operand once
    either way and stays with the reduction kernels.  When a call's shapes are turned away the chain runs
    its island as the separate kernels of the test above."""
    import workloads
    from theano_amd import hip
    from theano_amd.hip.rowchain import HipRowChain
    ins, outs = workloads.c5_graph(with_grad=False)
    f = th.function(ins, [th.Out(o, device=True) for o in outs])
    (chain,) = ops_of(f, HipRowChain)
    assert chain.op.program.axes == (0, 2, 3) and chain.op.program.held_passes == 2
    assert " void held(" in chain.op.src and " void row(" not in chain.op.src
    assert not ops_of(f, HipCAReduce) and not ops_of(f, HipElemwise)
    f(*workloads.c5_inputs("small", with_grad=False))
    assert "|rh|" in hip.last_plan()
    # statistics alone: nothing to keep the values for
    x = ins[0]
    xf = T.cast(x, "float32")
    mean = T.mean(xf, axis=(0, 2, 3), keepdims=True)
    var = T.mean(T.sqr(xf - mean), axis=(0, 2, 3), keepdims=True)
    g = th.function([x], [th.Out(mean, device=True), th.Out(var, device=True)])
    assert not ops_of(g, HipRowChain)
    # gradient: x and g both held at this size; turned away (THX_HELD=0) the same node runs its island unfused
    ins, outs = workloads.c5_graph(forward=False)
    h = th.function(ins, [th.Out(o, device=True) for o in outs])
    (chain,) = ops_of(h, HipRowChain)
    small = workloads.c5_inputs("small")
    h(*small)
    assert "|rh|" in hip.last_plan()
    os.environ["THX_HELD"] = "0"
    try:
        h2 = th.function(ins, [th.Out(o, device=True) for o in outs])
        h2(*small)
        assert "|rh|" not in hip.last_plan()
        inner = ops_of(h2, HipRowChain)[0].op._fallback_function
        assert [type(n.op) for n in inner.toposort() if isinstance(n.op, (HipCAReduce, HipElemwise))][-2:] == [HipCAReduce, HipElemwise]
    finally:
        del os.environ["THX_HELD"]


def test_inplace_pass_reuses_single_use_intermediates_only(dry_run):
    """The in-place pass (InplaceElemwiseOptimizer's role): an intermediate that
    one kernel computes and one elementwise kernel consumes is overwritten;
    function inputs, outputs, views and values with two readers never are."""
    x = T.fmatrix("x")
    f = th.function([x], T.exp(x) * 2.0 + 1.0, fuse=False)
    ew = ops_of(f, HipElemwise)
    assert [dict(n.op.inplace_pattern) for n in ew] == [{}, {0: 0}, {0: 0}]   # exp reads the input: not in place
    assert ew[1].op.destroy_map == {0: [0]}
    e = T.exp(x)
    g = th.function([x], [e + 1.0, e * 2.0], fuse=False)
    assert all(not n.op.inplace_pattern for n in ops_of(g, HipElemwise))       # e has two readers
    h = th.function([x], [e, e + 1.0], fuse=False)
    assert all(not n.op.inplace_pattern for n in ops_of(h, HipElemwise))       # e is an output
    k = th.function([x], T.sum(x, axis=0).dimshuffle("x", 0) + 1.0, fuse=False)
    assert all(not n.op.inplace_pattern for n in ops_of(k, HipElemwise))       # a view of the sum
    f(np.ones((3, 4), "float32"))
    assert not any(n.op.inplace_pattern for n in ops_of(th.function([x], T.exp(x) * 2.0 + 1.0, fuse=False,
                                                                    inplace=False), HipElemwise))


def test_max_and_argmax_interface(dry_run):
    """Output types, keepdims, the 0-d case, the zero gradient of argmax, the
    max-only rewrite and argmin's reversal (theano/tensor/basic.py:1273-1803,
    tests theano/tensor/tests/test_basic.py:3103-3218)."""
    from theano_amd.hip import HipMaxAndArgmax
    x = T.ftensor3("x")
    m, a = T.max_and_argmax(x, axis=[1, -1])
    assert m.type.dtype == "float32" and a.type.dtype == "int64" and m.type.ndim == 1 and a.type.ndim == 1
    assert isinstance(m.owner.op, T.MaxAndArgmax) and m.owner.op.axis == (1, 2)
    mk, ak = T.max_and_argmax(x, axis=0, keepdims=True)
    assert mk.type.broadcastable == (True, False, False) and ak.type.broadcastable == (True, False, False)
    s = T.fscalar("s")
    v0, i0 = T.max_and_argmax(s)
    assert v0 is s and i0.type.dtype == "int64" and int(i0.data) == 0
    with pytest.raises(ValueError):
        T.max_and_argmax(x, axis=3)
    # d argmax / dx is zero; d max / dx marks the positions equal to the maximum
    g = th.grad(T.sum(T.cast(T.argmax(x, axis=0), "float32")), x, disconnected_inputs="ignore")
    f = th.function([x], g)
    assert not ops_of(f, HipMaxAndArgmax)
    # nothing reads the argmax: a plain max reduction runs
    f = th.function([x], T.max_and_argmax(x, axis=2)[0])
    assert not ops_of(f, HipMaxAndArgmax) and len(ops_of(f, HipCAReduce)) == 1
    # argmin(x) = argmax(-x), the negation computed inside the reduction
    f = th.function([x], T.argmin(x, axis=1))
    (node,) = ops_of(f, HipMaxAndArgmax)
    assert not ops_of(f, HipElemwise) and str(node.op.pre_scalar_op) == "Composite{neg(i0)}"
    f(np.zeros((3, 5, 7), "float32"))


def test_plans_for_arrays_beyond_32_bit_limits(dry_run):
    """Planning only (no memory is touched in a dry run): more than 2^31 elements
    switch the kernels to 64-bit offsets; more vectors than one dispatch has
    work-items (2^32 - 1) switch the elementwise kernel to a grid-stride loop."""
    from theano_amd import hip
    v = T.TensorType("int8", (False,))("v")
    f = th.function([v], th.Out(v + np.int8(1), device=True))
    big = np.lib.stride_tricks.as_strided(np.zeros((), "int8"), shape=(2 ** 31 + 4096,), strides=(0,))
    f(big)
    assert "|i64|" in hip.last_plan() and "|gs" not in hip.last_plan()
    huge = np.lib.stride_tricks.as_strided(np.zeros((), "int8"), shape=(2 ** 37,), strides=(0,))
    f(huge)
    assert "|i64|" in hip.last_plan() and "|gs|" in hip.last_plan()
    g = th.function([v], T.sum(v))
    g(huge)
    assert "|i64|" in hip.last_plan()


def test_updates_replace_shared_values_after_the_call(dry_run):
    """function(..., updates=[(w, new_w)]): type checks of theano/compile/pfunc.py
    and the new value lands in the shared variable's container."""
    w = th.shared(np.zeros((3, 4), "float32"), name="w")
    x = T.fmatrix("x")
    f = th.function([x], T.sum(x * w), updates=[(w, w + x)])
    before = w.container[0]
    f(np.ones((3, 4), "float32"))
    assert w.container[0] is not before and w.container[0].shape == (3, 4)
    g = th.function([x], None, updates={w: w * 2 - x})
    assert g(np.ones((3, 4), "float32")) == []
    with pytest.raises(TypeError):
        th.function([x], [], updates=[(w, T.cast(w, "float64"))])      # dtype must not change
    with pytest.raises(TypeError):
        th.function([x], [], updates=[(x, x + 1)])                     # only shared variables are updated
    with pytest.raises(ValueError):
        th.function([x], [], updates=[(w, w + 1), (w, w + 2)])
    # a view of the shared value is copied, never stored as an alias of the old buffer
    h = th.function([], [], updates=[(w, w[::-1])])
    old = w.container[0]
    h()
    assert w.container[0].buffer is not old.buffer


def test_rop_matches_finite_differences_and_lop_matches_grad():
    """Jacobian-times-vector of an Elemwise / DimShuffle / Sum / Subtensor graph
    against central differences along the direction, and vector-times-Jacobian
    against grad of the weighted sum (theano/tests/test_rop.py:62-150 checks
    Rop the same way, against a scan-built Jacobian)."""
    from oracle import graph_ref as G
    rng = np.random.default_rng(5)
    x, v = T.dmatrix("x"), T.dmatrix("v")
    b = T.dvector("b")
    y = T.sum(T.tanh(x * b.dimshuffle("x", 0)) * x[:, ::-1], axis=0) + T.exp(b)
    jv = th.Rop(y, x, v)
    xv, vv, bv = rng.standard_normal((4, 3)), rng.standard_normal((4, 3)), rng.standard_normal(3)
    got = G.evaluate([x, v, b], [jv], [xv, vv, bv])[0]
    eps = 1e-6
    f = lambda xx: G.evaluate([x, b], [y], [xx, bv])[0]
    want = (f(xv + eps * vv) - f(xv - eps * vv)) / (2 * eps)
    assert np.allclose(got, want, rtol=1e-6, atol=1e-8)

    w = T.dvector("w")
    vj = th.Lop(y, x, w)
    ref = th.grad(T.sum(y * w), x)
    wv = rng.standard_normal(3)
    a, c = G.evaluate([x, b, w], [vj, ref], [xv, bv, wv])
    assert np.allclose(a, c, rtol=1e-12)

    # two variables at once: J_x v + J_b u
    u = T.dvector("u")
    both = G.evaluate([x, v, b, u], [th.Rop(y, [x, b], [v, u])], [xv, vv, bv, wv])[0]
    fb = lambda t: G.evaluate([x, b], [y], [xv + t * vv, bv + t * wv])[0]
    assert np.allclose(both, (fb(eps) - fb(-eps)) / (2 * eps), rtol=1e-6, atol=1e-8)


def _ops_of(fg):
    return [type(n.op).__name__ for n in fg.toposort()]


def test_softmax_ops_make_node_grad_and_rewrites():
    """The row-softmax Op family: interface checks (theano/tensor/nnet/nnet.py:62-72,
    303-315, 424-437), the rewrites that produce the ops (softmax_simplifier :888-925,
    local_softmax_with_bias :822-885, local_logsoftmax :749-769, local_logsoftmax_grad
    :772-804) and the lowering that leaves only Elemwise / CAReduce / DimShuffle nodes."""
    import warnings
    from theano_amd import gof
    from theano_amd.tensor import nnet as N, opt as topt
    from oracle import graph_ref as G
    rng = np.random.default_rng(3)
    x, y = T.dmatrix("x"), T.dmatrix("y")
    b = T.dvector("b")
    with pytest.raises(ValueError):
        N.softmax_op(T.lmatrix())
    with pytest.raises(ValueError):
        N.softmax_op(T.TensorType("float32", (False,) * 3)())
    with pytest.raises(ValueError):
        N.softmax_with_bias(x, x)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        assert N.softmax_op(b).type.ndim == 2          # vectors are padded to one row
    assert N.softmax_op == N.Softmax() and hash(N.softmax_op) == hash(N.Softmax())

    # the unstabilised quotient becomes the op: finite results where exp overflows
    fg = gof.FunctionGraph([x], [N.softmax_graph(x)])
    gof.merge_identical(fg)                        # the two exp(x) nodes become one
    gof.apply_local(fg, topt.CANONICALIZE + N.RECOGNIZE)
    assert _ops_of(fg) == ["Softmax"]
    xv = rng.standard_normal((5, 7)) * 3
    xv[0, 0] = 800.0
    got = G.evaluate(fg.inputs, fg.outputs, [xv])[0]
    assert np.isfinite(got).all() and np.allclose(got.sum(1), 1.0)

    # softmax(x + b) -> softmax_with_bias; log(softmax) -> logsoftmax, also in the gradient
    fg = gof.FunctionGraph([x, b], [N.softmax(x + b.dimshuffle("x", 0))])
    gof.apply_local(fg, topt.CANONICALIZE + N.RECOGNIZE)
    assert _ops_of(fg) == ["SoftmaxWithBias"]
    cost = T.sum(T.log(N.softmax(x)) * y)
    fg = gof.FunctionGraph([x, y], [cost, th.grad(cost, x)])
    gof.merge_identical(fg)
    gof.apply_local(fg, topt.CANONICALIZE + N.RECOGNIZE)
    names = _ops_of(fg)
    assert "LogSoftmax" in names and "SoftmaxGrad" not in names and names.count("Softmax") == 1

    # values and gradients of the ops (evaluated by the reference's perform formulas)
    # against the lowered Elemwise / CAReduce graphs and against closed forms
    yv, bv = rng.uniform(0, 1, (5, 7)), rng.standard_normal(7)
    sm, lsm, swb = N.softmax(x), N.logsoftmax(x), N.softmax_with_bias(x, b)
    outs = [sm, lsm, swb, th.grad(T.sum(sm * y), x), th.grad(T.sum(lsm * y), x), th.grad(T.sum(swb * y), b),
            th.grad(T.sum(th.grad(T.sum(sm * y), x) ** 2), x), th.Rop(sm, x, y)]
    as_ops = G.evaluate([x, y, b], outs, [xv, yv, bv])
    fg = gof.FunctionGraph([x, y, b], outs)
    topt.canonicalize(fg)
    assert set(_ops_of(fg)) <= {"Elemwise", "DimShuffle", "Sum", "Max", "CAReduce"}
    lowered = G.evaluate(fg.inputs, fg.outputs, [xv, yv, bv])
    for a, l in zip(as_ops, lowered):
        assert np.allclose(a, l, rtol=1e-10, atol=1e-12)
    e = np.exp(xv - xv.max(1, keepdims=True))
    p = e / e.sum(1, keepdims=True)
    from scipy.special import log_softmax
    assert np.allclose(as_ops[0], p) and np.allclose(as_ops[1], log_softmax(xv, axis=1))
    assert np.isfinite(as_ops[1]).all()                # row 0 holds 800: log(softmax) itself gives -inf there
    assert np.allclose(as_ops[3], p * (yv - (p * yv).sum(1, keepdims=True)))
    assert np.allclose(as_ops[4], yv - yv.sum(1, keepdims=True) * p)
    assert np.allclose(as_ops[7], as_ops[3])           # symmetric Jacobian


def test_softmax_op_graphs_compile_to_one_row_kernel():
    from theano_amd import hip
    from theano_amd.tensor import nnet as N
    x, y = T.fmatrix("x"), T.fmatrix("y")
    hip.set_dry_run(True)
    try:
        cost = T.sum(T.log(N.softmax(x)) * y)
        f = th.function([x, y], [N.softmax(x), th.grad(cost, x)])
        f(np.zeros((4, 64), "float32"), np.zeros((4, 64), "float32"))
        kernels = [type(n.op).__name__ for n in f.toposort() if type(n.op).__name__.startswith("Hip")
                   and type(n.op).__name__ not in ("HipDimShuffle", "HipToHost")]
        assert kernels == ["HipRowChain"], kernels
    finally:
        hip.set_dry_run(False)


def test_single_pass_variance_rewrite_keeps_the_values():
    """sum(sqr(x - mean(x))) rewritten to shifted sums in float64: the canonicalised graph,
    evaluated node by node, against the two-pass graph and against NumPy's float64 variance;
    also for a channel whose first element is an outlier, a constant channel, reduction over
    all axes, and float64 data (left alone)."""
    from theano_amd import gof, config
    from theano_amd.tensor import opt as topt
    from oracle import graph_ref as G
    rng = np.random.default_rng(9)
    x4 = T.TensorType("float16", (False,) * 4)("x")
    xf = T.cast(x4, "float32")
    outs = [T.var(xf, axis=(0, 2, 3), keepdims=True), T.mean(xf, axis=(0, 2, 3), keepdims=True), T.std(xf, axis=(0, 2, 3))]
    xv = rng.normal(0.5, 2.0, (6, 5, 7, 8)).astype("float16")
    xv[0, 1, 0, 0] = 3000.0          # the shift of channel 1 is an outlier
    xv[:, 2] = 1.25                   # a constant channel: variance exactly 0
    fg = gof.FunctionGraph([x4], outs)
    topt.canonicalize(fg)
    sums = [n for n in fg.toposort() if type(n.op).__name__ == "Sum"]
    assert len(sums) == 3 and all(n.inputs[0].type.ndim == 4 for n in sums), [str(n) for n in sums]
    assert sorted(n.outputs[0].type.dtype for n in sums) == ["float32", "float64", "float64"]
    got = G.evaluate(fg.inputs, fg.outputs, [xv])
    with config.change_flags(single_pass_variance=False):
        fg2 = gof.FunctionGraph([x4], outs)
        topt.canonicalize(fg2)
        assert len([n for n in fg2.toposort() if type(n.op).__name__ == "Sum"]) == 2
        two_pass = G.evaluate(fg2.inputs, fg2.outputs, [xv])
    x64 = xv.astype("float64")
    exact = [x64.var(axis=(0, 2, 3), keepdims=True), x64.mean(axis=(0, 2, 3), keepdims=True), x64.std(axis=(0, 2, 3))]
    for g, t, e in zip(got, two_pass, exact):
        assert g.dtype == t.dtype == np.float32 and g.shape == t.shape
        assert np.allclose(g, e, rtol=2e-6, atol=1e-7)
        assert np.allclose(t, e, rtol=2e-6, atol=1e-7)
    assert got[0][0, 2, 0, 0] == 0.0 and got[2][2] == 0.0

    m = T.fmatrix("m")
    fg = gof.FunctionGraph([m], [T.var(m), T.var(m, axis=0), T.var(m, axis=1, keepdims=True)])
    topt.canonicalize(fg)
    mv = rng.normal(-3.0, 0.1, (33, 17)).astype("float32")
    for g, e in zip(G.evaluate(fg.inputs, fg.outputs, [mv]),
                    [mv.astype("float64").var(), mv.astype("float64").var(0), mv.astype("float64").var(1, keepdims=True)]):
        assert np.allclose(g, e, rtol=1e-5)

    d = T.dmatrix("d")
    fg = gof.FunctionGraph([d], [T.var(d, axis=0)])
    topt.canonicalize(fg)
    assert len([n for n in fg.toposort() if type(n.op).__name__ == "Sum"]) == 2      # still two passes


def test_abstract_batch_norm_ops_lower_to_the_reference_formulas():
    """AbstractBatchNormTrain / TrainGrad / Inference nodes (theano/tensor/nnet/bn.py:364-676):
    evaluated with the reference's perform formulas, they agree with the graphs they are
    lowered to; their L_op (closed forms, incl. the second derivatives of bn.py:601-650)
    agrees with reverse mode through hand-written mean / var graphs."""
    from theano_amd import gof
    from theano_amd.tensor import nnet as N, opt as topt
    from oracle import graph_ref as G
    rng = np.random.default_rng(12)
    t4 = T.TensorType("float64", (False,) * 4)
    x, dy = t4("x"), t4("dy")
    g, b, rm, rv = [T.dvector(n) for n in ("g", "b", "rm", "rv")]          # one entry per channel: padded by the front end
    out, mean, invstd, nrm, nrv = N.batch_normalization_train(x, g, b, "spatial", 1e-4, 0.25, rm, rv)
    assert out.type.ndim == 4 and mean.type.ndim == 1 and nrv.type.ndim == 1
    node = out.owner
    assert isinstance(node.op, N.AbstractBatchNormTrain) and node.op.axes == (0, 2, 3) and len(node.outputs) == 5
    assert node.op == N.AbstractBatchNormTrain((0, 2, 3)) and node.op != N.AbstractBatchNormTrain((0,))
    with pytest.raises(ValueError):
        N.batch_normalization_train(x, g, b, "spatial", 1e-6)               # epsilon below 1e-5
    with pytest.raises(ValueError):
        N.batch_normalization_train(x, g, b, "spatial", 1e-4, 0.1, rm, None)
    with pytest.raises(ValueError):
        N.batch_normalization_train(x, T.dmatrix(), T.dmatrix(), "spatial")
    inf = N.batch_normalization_test(x, g, b, rm, rv, "spatial", 1e-4)
    cost = T.sum(out * dy)
    gx, gg, gb = th.grad(cost, [x, g, b])
    assert any(isinstance(n.op, N.AbstractBatchNormTrainGrad) for n in gof.io_toposort([x, dy, g, b], [gx]))
    second = th.grad(T.sum(gx * gx) + T.sum(gg * gg), [x, dy, g])
    ginf = th.grad(T.sum(inf * dy), [x, g, b, rm, rv])
    outs = [out, mean, invstd, nrm, nrv, inf, gx, gg, gb] + second + ginf
    ins = [x, dy, g, b, rm, rv]
    vals = [rng.normal(0.5, 2.0, (4, 5, 3, 6)), rng.standard_normal((4, 5, 3, 6)), rng.uniform(0.5, 1.5, 5),
            rng.standard_normal(5), rng.standard_normal(5), rng.uniform(0.5, 1.5, 5)]
    as_ops = G.evaluate(ins, outs, vals)
    fg = gof.FunctionGraph(ins, outs)
    topt.canonicalize(fg)
    assert not any(type(n.op).__name__.startswith("AbstractBatchNorm") for n in fg.toposort())
    lowered = G.evaluate(fg.inputs, fg.outputs, vals)
    for k, (a, l) in enumerate(zip(as_ops, lowered)):
        assert np.allclose(a, l, rtol=1e-9, atol=1e-11), k

    # the same quantities from plain graphs and reverse mode
    pad = lambda v: v.dimshuffle("x", 0, "x", "x")       # noqa: E731
    m = T.mean(x, axis=(0, 2, 3), keepdims=True)
    v = T.mean(T.sqr(x - m), axis=(0, 2, 3), keepdims=True)
    o2 = (x - m) * (pad(g) / T.sqrt(v + 1e-4)) + pad(b)
    hx, hg, hb = th.grad(T.sum(o2 * dy), [x, g, b])
    i2 = (x - pad(rm)) * (pad(g) / T.sqrt(pad(rv) + 1e-4)) + pad(b)
    plain = [o2, hx, hg, hb] + th.grad(T.sum(hx * hx) + T.sum(hg * hg), [x, dy, g]) + th.grad(T.sum(i2 * dy), [x, g, b, rm, rv])
    want = G.evaluate(ins, plain, vals)
    have = [as_ops[0]] + as_ops[6:]
    for k, (a, w) in enumerate(zip(have, want)):
        assert np.allclose(a, w, rtol=1e-7, atol=1e-9), k
    n_per = 4 * 3 * 6
    xv = vals[0]
    assert np.allclose(as_ops[3], vals[4] * 0.75 + xv.mean((0, 2, 3)) * 0.25)
    assert np.allclose(as_ops[4], vals[5] * 0.75 + xv.var((0, 2, 3)) * n_per / (n_per - 1) * 0.25)


def test_ops_and_graphs_pickle(dry_run):
    """Ops pickle by value of their props and compare equal afterwards, graphs keep their
    structure (the role of theano/misc/pkl_utils.py for this path): every op of the
    compiled benchmark graphs, and an uncompiled graph with gradients evaluated before
    and after a round trip."""
    import pickle
    import workloads as W
    from oracle import graph_ref as G
    for g in (W.c1_graph(), W.c3_graph(), W.c4_graph("all"), W.c5_graph(), W.c2_argmax_graph(1)):
        for n in th.function(*g).toposort():
            again = pickle.loads(pickle.dumps(n.op))
            assert again == n.op and hash(again) == hash(n.op), n.op
    # a chain node that has compiled its island as separate kernels (device handles inside) still pickles
    from theano_amd.hip.rowchain import HipRowChain
    os.environ["THX_HELD"] = "0"
    try:
        f = th.function(*W.c5_graph(with_grad=False))
        f(*W.c5_inputs("small", with_grad=False))
    finally:
        del os.environ["THX_HELD"]
    (chain,) = ops_of(f, HipRowChain)
    assert chain.op._fallback_function is not None
    again = pickle.loads(pickle.dumps(chain.op))
    assert again == chain.op and not hasattr(again, "_fallback_function")
    x = T.fmatrix("x")
    y = T.sum(T.exp(x) * T.nnet.sigmoid(x) + T.erf(x) % 3, axis=1)
    z = T.nnet.softmax(x)[:, ::2].reshape((-1,))
    gx = th.grad(T.sum(y) + T.sum(z * z), x)
    x2, outs2 = pickle.loads(pickle.dumps((x, [y, z, gx])))
    v = np.random.default_rng(0).standard_normal((4, 6)).astype("float32")
    for a, b in zip(G.evaluate([x], [y, z, gx], [v]), G.evaluate([x2], outs2, [v])):
        assert np.array_equal(a, b)


def test_sibling_elementwise_kernels_merge_into_one_with_several_results(dry_run):
    """An Adam step: both moment updates and the parameter update read g, m, v, p once and
    write three arrays in one kernel; kernels of different shapes, or one feeding the other
    through a reduction, stay apart."""
    p, g, m, v = [T.fmatrix(n) for n in "pgmv"]
    m2 = 0.9 * m + 0.1 * g
    v2 = 0.999 * v + 0.001 * T.sqr(g)
    p2 = p - 0.01 * m2 / (T.sqrt(v2) + 1e-8)
    f = th.function([p, g, m, v], [m2, v2, p2])
    (k,) = ops_of(f, HipElemwise)
    assert len(k.outputs) == 3 and len(k.inputs) == 4
    f(*[np.zeros((3, 4), "float32")] * 4)
    # different shapes: a row result and a matrix result do not merge
    r = T.frow("r")
    h = th.function([p, r], [p * 2.0, r * 3.0])
    assert len(ops_of(h, HipElemwise)) == 2
    # a dependency through a reduction keeps two kernels
    s = T.sum(p * 2.0, axis=0, keepdims=True)
    d = th.function([p], [T.exp(p), p / s])
    assert len(ops_of(d, HipElemwise)) == 2 or len(ops_of(d, HipCAReduce)) == 1


def test_nested_sums_and_products_become_one_reduction():
    """Sum(Sum(x, a), b) -> Sum(x, a + b') with the outer axes renumbered, Prod likewise, every
    axis -> None (theano/tensor/opt.py:5479-5563); an inner result that something else reads
    stays.  Values against NumPy."""
    from theano_amd import gof
    from theano_amd.tensor import opt as topt
    from oracle import graph_ref as G
    x = T.TensorType("float64", (False,) * 4)("x")
    xv = np.random.default_rng(1).uniform(0.5, 1.5, (3, 4, 5, 6))
    cases = [(T.sum(T.sum(x, axis=1), axis=1), xv.sum(axis=(1, 2)), (1, 2)),
             (T.sum(T.sum(x, axis=(0, 3)), axis=0), xv.sum(axis=(0, 1, 3)), (0, 1, 3)),
             (T.sum(T.sum(x, axis=2), axis=(0, 2)), xv.sum(axis=(0, 2, 3)), (0, 2, 3)),
             (T.prod(T.prod(x, axis=3), axis=0), xv.prod(axis=(0, 3)), (0, 3)),
             (T.sum(T.sum(x, axis=(1, 2))), xv.sum(), None),
             (T.sum(x, axis=(0, 1, 2, 3)), xv.sum(), None)]
    for out, want, axis in cases:
        fg = gof.FunctionGraph([x], [out])
        topt.canonicalize(fg)
        reds = [n for n in fg.toposort() if isinstance(n.op, CAReduce)]
        assert len(reds) == 1 and reds[0].op.axis == axis, (str(out), [str(n) for n in reds])
        assert np.allclose(G.evaluate(fg.inputs, fg.outputs, [xv])[0], want, rtol=1e-13)
    inner = T.sum(x, axis=1)
    fg = gof.FunctionGraph([x], [T.sum(inner, axis=1), inner * 2])
    topt.canonicalize(fg)
    assert len([n for n in fg.toposort() if isinstance(n.op, CAReduce)]) == 2
    # sum of a product of sums is not touched
    fg = gof.FunctionGraph([x], [T.sum(T.prod(x, axis=1), axis=1)])
    topt.canonicalize(fg)
    assert len([n for n in fg.toposort() if isinstance(n.op, CAReduce)]) == 2


def test_deep_chain_is_canonicalized_to_a_fixed_point_quickly(dry_run):
    """A rewrite whose result enables the next one (here: one per layer) is followed along the
    chain inside one sweep: a 40-layer network with its gradient compiles in seconds and ends
    up as one row-wise kernel plus the final sum."""
    import time, warnings
    from theano_amd.hip.rowchain import HipRowChain
    x = T.fmatrix("x")
    h = x
    for _ in range(40):
        h = T.tanh(h * 1.01 + T.mean(h, axis=1, keepdims=True)) * T.nnet.sigmoid(h)
    cost = T.sum(h * h)
    g = th.grad(cost, x)
    t0 = time.time()
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        f = th.function([x], [cost, g])
    assert time.time() - t0 < 30
    kinds = [type(n.op).__name__ for n in f.toposort()]
    assert kinds.count("HipRowChain") == 1 and kinds.count("HipElemwise") == 0, kinds


def test_sum_of_reciprocal_with_constant_numerator_terminates(dry_run):
    """sum(c / x): the constant leaves the sum once (c * sum(1 / x)) and the rewriter stops."""
    import warnings
    x = T.dmatrix("x")
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        f = th.function([x], T.sum(2.0 / x) + T.sum(T.ones_like(x) / x))
    assert f is not None


def test_sigmoid_and_softplus_stabilisation_rewrites(dry_run):
    """The patterns of theano/tensor/nnet/sigm.py:378-425, 588-640, 845-905 become sigmoid / softplus nodes."""
    from theano_amd.tensor import nnet
    x, t = T.dmatrix("x"), T.dmatrix("t")

    def kernels(v):
        return [str(n.op) for n in th.function([x, t], v, on_unused_input="ignore").toposort() if "Host" not in str(n.op)]

    assert kernels(T.log(nnet.sigmoid(x))) == ["HipElemwise{Composite{neg(scalar_softplus(neg(i0)))}}"]
    assert kernels(T.log(1 - nnet.sigmoid(x))) == ["HipElemwise{Composite{neg(scalar_softplus(i0))}}"]
    assert kernels(T.log1p(T.exp(x))) == ["HipElemwise{scalar_softplus}"]
    assert kernels(T.log1p(-nnet.sigmoid(x))) == ["HipElemwise{Composite{neg(scalar_softplus(i0))}}"]
    assert kernels(T.exp(x) / (1 + T.exp(x))) == ["HipElemwise{scalar_sigmoid}"]
    assert kernels(1.0 / (1.0 + T.exp(-x))) == ["HipElemwise{scalar_sigmoid}"]
    assert kernels(nnet.sigmoid(x) * T.exp(-x)) == ["HipElemwise{Composite{scalar_sigmoid(neg(i0))}}"]
    (k,) = kernels(3.0 * t / ((1 + T.exp(x)) * t))
    assert "exp" not in k and "scalar_sigmoid(neg(i1))" in k
    (k,) = kernels(nnet.binary_crossentropy(nnet.sigmoid(x), t))
    assert "log" not in k and k.count("scalar_softplus") == 2
    # the fused cross-entropy differentiates to sigmoid(x) - t, also at x = 0
    (k,) = kernels(th.grad(T.sum(nnet.sigmoid_binary_crossentropy(x, t)), x))
    assert k == "HipElemwise{Composite{sub(scalar_sigmoid(i0), i1)}}", k
    # 2 + exp(x) is not 1 + exp(x)
    (k,) = kernels(1.0 / (2.0 + T.exp(x)))
    assert "sigmoid" not in k


def test_activation_front_ends(dry_run):
    from theano_amd.tensor import nnet
    x = T.fmatrix("x")
    i = T.imatrix("i")
    assert nnet.hard_sigmoid(x).type.dtype == "float32" and nnet.hard_sigmoid(i).type.dtype == "float64"
    assert nnet.ultra_fast_sigmoid(x).type.dtype == "float32" and nnet.softsign(x).type.dtype == "float32"
    assert nnet.elu(x).type == x.type and nnet.selu(x).type.dtype == "float32"
    assert nnet.categorical_crossentropy(nnet.softmax(x), x).type.ndim == 1
    with pytest.raises(NotImplementedError):
        nnet.categorical_crossentropy(nnet.softmax(x), T.ivector("y"))
    with pytest.raises(Exception):
        th.grad(T.sum(nnet.ultra_fast_sigmoid(x)), x)      # no gradient, as in the reference


def test_exp_feeding_a_sum_and_a_division_is_recomputed_not_stored(dry_run):
    """Without the row-chain kernel a softmax is three launches - row max, sum of exp(x - max) computed on the
    fly, exp(x - max) / sum - because one exp per consumer is cheaper than writing the exponentials and
    reading them back; the flag that allows no transcendental in a duplicated producer gives four."""
    from theano_amd.hip import HipCAReduce
    x = T.fmatrix("x")
    e = T.exp(x - T.max(x, axis=1, keepdims=True))
    sm = e / T.sum(e, axis=1, keepdims=True)
    f = th.function([x], sm, rowchain=False)
    assert (len(ops_of(f, HipCAReduce)), len(ops_of(f, HipElemwise))) == (2, 1)
    with th.config.change_flags(duplicate_transcendentals=0):
        g = th.function([x], sm, rowchain=False)
    assert (len(ops_of(g, HipCAReduce)), len(ops_of(g, HipElemwise))) == (2, 2)
    # a per-row value broadcast against the reduction's operand is never recomputed per element
    r = T.exp(T.max(x, axis=1, keepdims=True))
    h = th.function([x], [T.sum(x * r, axis=0), x + r], rowchain=False)
    pro = [n for n in ops_of(h, HipCAReduce) if n.op.pre_scalar_op is not None]
    assert all("exp" not in str(n.op.pre_scalar_op) for n in pro)


def test_gradient_corner_cases_of_the_reference_elemwise_tests(dry_run):
    """theano/tensor/tests/test_elemwise.py:1154-1350: gradients through all / any and through integer-valued
    costs are zeros, comparisons pass no gradient, a gradient an op declares not implemented raises only when
    it is asked for, and gradients with respect to broadcast inputs build."""
    from oracle import graph_ref as G
    from theano_amd import gradient
    x = T.bmatrix("x")
    xv = np.random.RandomState(0).binomial(1, 0.5, (5, 7)).astype("int8")
    for red in (x.all(), x.any()):
        gx = th.grad(red, x)
        for v in (xv, np.zeros_like(xv), np.ones_like(xv)):
            g = G.evaluate([x], [gx], [v])[0]
            assert g.shape == v.shape and np.all(g == 0)
        th.function([x], gx)
    b, i8 = T.TensorType("bool", ())("b"), T.TensorType("int8", ())("i")
    assert [g.type.dtype for g in th.grad(b * i8, [b, i8])] == ["float32", "float32"]
    ints = [T.TensorType("int32", ())(n) for n in "xyz"]
    assert len(th.grad(T.clip(*ints), ints)) == 3
    s = T.fvector("s")
    scores = T.ones_like(s) - s + s * 2
    g = th.grad((scores * (scores > 0)).sum(), s)
    assert np.array_equal(G.evaluate([s], [g], [np.array([0.5, -3, 2], "float32")])[0], [1, 0, 1])
    t4 = T.TensorType("float32", (True, False, False, False))("x4")
    y4 = T.TensorType("float32", (True, True, False, False))("y4")
    gx4, gy4 = th.grad(T.tanh(t4 + y4).sum(), [t4, y4])
    assert gx4.type == t4.type and gy4.type == y4.type

    class Scale(scal.ScalarOp):
        nin = 2

        def __init__(self):
            self.output_types_preference = scal.upgrade_to_float
            self.name = "scale"

        def L_op(self, inputs, outputs, gout):
            n, v = inputs
            return [gradient.grad_not_implemented(self, 0, n), gout[0] * n]

    op = Elemwise(Scale())
    v = T.TensorType("float32", ())("v")
    th.grad(op(2, v), v)
    with pytest.raises(gradient.NullTypeGradError):
        th.grad(op(v, 2), v)
    with pytest.raises(gradient.NullTypeGradError):
        th.grad(T.exp(op(v, 2)) * 3, v)          # also through further nodes


def test_gradient_of_log_one_minus_sigmoid_cancels_to_minus_sigmoid(dry_run):
    """test_grad_useless_sum, theano/tensor/tests/test_elemwise.py:1262-1297: no Sum node for a broadcastable
    input, and the factor 1 - sigmoid(x) leaves the quotient, so the compiled kernel is -(g * sigmoid(x))."""
    from theano_amd import gof
    x = T.TensorType("float32", (True,))("x")
    g = th.grad(T.log(1.0 - T.nnet.sigmoid(x))[0], x)
    assert not any(isinstance(n.op, Sum) for n in gof.io_toposort([x], [g]))
    f = th.function([x], g)
    (k,) = ops_of(f, HipElemwise)
    assert str(k.op.scalar_op) == "Composite{neg(mul(i0, scalar_sigmoid(i1)))}"
    # a factor that gives the result its shape stays
    m, r = T.fmatrix("m"), T.frow("r")
    h = th.function([m, r], (r / m) * m)
    assert any("true_div" in str(n.op) or "mul" in str(n.op) for n in h.toposort())


def test_more_operands_than_a_kernel_takes_are_split(dry_run):
    """add / mul of 64 tensors (theano/gpuarray/tests/test_opt.py:531-572) compile to kernels of at most
    ``max_fused_inputs`` operands, and fusion does not grow a node past that limit afterwards."""
    sym = [T.fmatrix() for _ in range(64)]
    for op in (T.add, T.mul):
        f = th.function(sym, op(*sym) * 2.0)
        kernels = ops_of(f, HipElemwise)
        assert len(kernels) > 1 and all(len(n.inputs) <= th.config.max_fused_inputs for n in kernels)
        f(*[np.zeros((3, 4), "float32")] * 64)           # plans and compiles


def test_results_of_a_composite_that_nothing_reads_are_dropped():
    """theano/tensor/tests/test_opt.py:1364-1382 (local_useless_composite): one node, one output; the gradient of
    a Composite stays unimplemented (theano/scalar/basic.py:4096-4097)."""
    sx = scal.float32()
    comp = scal.Composite([sx], [sx + 1, sx - 1])
    X = T.fmatrix()
    o = Elemwise(scalar_op=comp)(X)
    assert len(o) == 2
    for k, name in ((0, "add"), (1, "sub")):
        f = th.function([X], o[k])
        (node,) = ops_of(f, HipElemwise)
        assert len(node.outputs) == 1 and name in str(node.op)
    f = th.function([X], o)
    (node,) = ops_of(f, HipElemwise)
    assert len(node.outputs) == 2
    with pytest.raises(NotImplementedError):
        th.grad(T.sum(o[0]), X)


def test_shape_patterns_of_reshape_and_alloc():
    """Entries of a shape: ints, extents of inputs, integer scalar inputs read at run time, arithmetic over those."""
    from theano_amd.tensor import views as V
    x = T.ftensor3("x")
    n = T.iscalar("n")
    r = x.reshape((x.shape[0], x.shape[1] * x.shape[2]))
    assert r.owner.op.pattern == ((0, 0), ("mul", (0, 1), (0, 2))) and len(r.owner.inputs) == 1
    assert r.type.broadcastable == (False, False)
    assert r.owner.op.resolve([(4, 6, 5)]) == (4, 30)
    r = x.reshape((n, -1, 1))
    assert r.owner.op.pattern == (("in", 1), -1, 1) and r.owner.inputs[1] is n and r.type.broadcastable == (False, False, True)
    assert r.owner.op.resolve([(4, 6, 5), ()], [None, np.int32(8)]) == (8, 15, 1)
    with pytest.raises(ValueError):
        r.owner.op.resolve([(4, 6, 5), ()])                       # needs the value, shapes alone do not say
    with pytest.raises(ValueError):
        r.owner.op.resolve([(4, 6, 5), ()], [None, np.int32(7)])  # 120 elements, 7 rows
    a = T.alloc(0.0, (x.shape[0] + 1) // 2, T.maximum(n, 1) - 0, 3)
    assert a.owner.op.pattern == (("floordiv", ("add", (1, 0), 1), 2), ("sub", ("max", ("in", 2), 1), 0), 3)
    assert a.owner.op.resolve([(), (5, 1, 1), ()], [None, None, np.int32(-4)]) == (3, 1, 3)
    assert str(a.owner.op) == "Alloc{floordiv(add(in1.shape[0], 1), 2), sub(max(in2, 1), 0), 3}"
    assert V.Reshape(r.owner.op.pattern) == r.owner.op and hash(V.Reshape(r.owner.op.pattern)) == hash(r.owner.op)
    for bad in (lambda: x.reshape((T.fscalar(),)), lambda: x.reshape((T.ivector(),)), lambda: V.Reshape([("pow", 1, 2)]),
                lambda: V.Alloc([-1]), lambda: V.Reshape([-1, -1])):
        with pytest.raises((TypeError, ValueError)):
            bad()


def test_inplace_module_names_and_types():
    """theano/tensor/inplace.py: 68 ``*_inplace`` Elemwise instances (the scalar op with transfer_type(0),
    inplace_pattern {0: 0}) and transpose_inplace."""
    from theano_amd.tensor import inplace as I
    assert len(I.__all__) == 69
    for name in I.__all__:
        if name == "transpose_inplace":
            continue
        op = getattr(I, name)
        assert isinstance(op, Elemwise) and op.inplace_pattern == ((0, 0),) and op.destroy_map == {0: [0]}
        assert type(op.scalar_op) is type(getattr(scal, name[:-len("_inplace")]))
        assert op.scalar_op.output_types_preference == scal.transfer_type(0)
    x, i = T.fmatrix(), T.imatrix()
    assert I.add_inplace(x, i).type == x.type           # the result takes the first operand's type
    assert I.add_inplace(i, x).type == i.type
    with pytest.raises(TypeError, match="incompatible data types"):
        I.lt_inplace(x, x)                              # a bool result cannot overwrite a float32 operand
    b = T.TensorType("bool", (False, False))()
    assert I.lt_inplace(b, b).type == b.type
    with pytest.raises(ValueError, match="broadcasted dimensions"):
        I.add_inplace(T.frow(), x)                      # the result is larger than the operand it would overwrite
    t = I.transpose_inplace(T.ftensor3())
    assert isinstance(t.owner.op, DimShuffle) and t.owner.op.new_order == (2, 1, 0)
    assert I.add_inplace == Elemwise(scal.Add(scal.transfer_type(0)), {0: 0})
    assert I.add_inplace != T.add


def test_graphs_with_inplace_operations_need_accept_inplace(dry_run):
    """theano/compile/function_module.py:183-190; protected variables and double destruction as the
    DestroyHandler and Supervisor of the reference report them."""
    from theano_amd import gof
    from theano_amd.tensor import inplace as I
    x, y = T.fmatrix("x"), T.fmatrix("y")
    with pytest.raises(TypeError, match="Graph must not contain inplace operations"):
        th.function([x, y], I.add_inplace(x, y))
    f = th.function([x, y], I.add_inplace(x, y), accept_inplace=True)
    assert f.writeback == [0] and [type(n.op).__name__ for n in f.nodes].count("HipElemwise") == 1
    # a chain over one buffer: the argument takes the last value; the other reader of x sees the old one,
    # in one fused kernel with it
    f = th.function([x, y], [I.mul_inplace(I.exp_inplace(x), y), x * 2], accept_inplace=True)
    assert f.writeback == [0] and [type(n.op).__name__ for n in f.nodes].count("HipElemwise") == 1
    # an intermediate that is overwritten: nothing to store back
    f = th.function([x, y], I.sub_inplace(x * y, y), accept_inplace=True)
    assert f.writeback == []
    with pytest.raises(gof.InconsistencyError, match="Multiple destroyers"):
        th.function([x], [I.exp_inplace(x), I.neg_inplace(x)], accept_inplace=True)
    with pytest.raises(gof.InconsistencyError, match="protected"):
        th.function([x], I.add_inplace(T.constant(np.ones((2, 2), "float32")), x), accept_inplace=True)
    with pytest.raises(NotImplementedError, match="view of a function argument"):
        th.function([x], I.exp_inplace(x.T), accept_inplace=True)
    with pytest.raises(ValueError, match="leaves its arguments alone"):
        th.function([x, y], I.add_inplace(x, y), accept_inplace=True, mode="check")
    # overwriting an intermediate is invisible to the caller: check mode takes it
    f = th.function([x, y], I.sub_inplace(x * y, y), accept_inplace=True, mode="check")
    assert isinstance(f, th.compile.CheckedFunction) and f.primary.writeback == []


def test_negated_max_of_a_negation_is_a_min(dry_run):
    """local_max_to_min (theano/tensor/opt_uncanonicalize.py:71-94): -max(-x) compiles to one min reduction
    for floating-point operands; integers keep the written form (the two differ at the most negative value
    and over unsigned types)."""
    x = T.fmatrix("x")
    f = th.function([x], -T.max(-x, axis=1))
    red = [n.op for n in f.toposort() if isinstance(n.op, HipCAReduce)]
    assert len(red) == 1 and isinstance(red[0].scalar_ops[0], scal.Minimum)
    assert red[0].pre_scalar_op is None and red[0].post_scalar_op is None
    assert not any(isinstance(n.op, HipElemwise) for n in f.toposort())
    i = T.imatrix("i")
    f = th.function([i], -T.max(-i, axis=1), rowchain=False)
    red = [n.op for n in f.toposort() if isinstance(n.op, HipCAReduce)]
    assert len(red) == 1 and isinstance(red[0].scalar_ops[0], scal.Maximum)
    from theano_amd.tensor import elemwise as E
    assert E.MulWithoutZeros is scal.MulWithoutZeros and E.mul_without_zeros is scal.mul_without_zeros


def test_tensor_type_value_helpers():
    """values_eq, may_share_memory, value_zeros, value_validity_msg, to_scalar_type, get_shape_info / get_size,
    convert_variable and filter_variable (theano/tensor/type.py:202-310, 552-610)."""
    t = T.TensorType("float32", (False, True))
    nan = np.array([[np.nan], [1.0]], "float32")
    assert t.values_eq(nan, nan.copy()) and not t.values_eq(nan, nan.astype("float64"))
    assert t.values_eq(nan, nan.astype("float64"), force_same_dtype=False) and not t.values_eq(nan, nan[:1])
    a = np.zeros(4)
    assert t.may_share_memory(a, a[1:]) and not t.may_share_memory(a, a.copy()) and not t.may_share_memory(a, 3)
    z = t.value_zeros((5, 1))
    assert z.dtype == np.float32 and z.shape == (5, 1) and not z.any()
    assert t.value_validity_msg(z) == "value is valid" and "broadcastable" in t.value_validity_msg(np.zeros((2, 2), "float32"))
    assert t.to_scalar_type() == scal.float32 and t.get_size(t.get_shape_info(z)) == 20
    both = T.TensorType("float32", (True, True))()
    assert t.filter_variable(both).type == t and T.fmatrix().type.filter_variable(both).type == T.fmatrix().type
    assert t.convert_variable(T.fmatrix()) is None and t.convert_variable(T.dmatrix()) is None
    v = t()
    assert t.filter_variable(v) is v
    with pytest.raises(TypeError, match="Cannot convert Type"):
        t.filter_variable(T.fmatrix())                   # a broadcastable dimension cannot be promised
    with pytest.raises(TypeError):
        t.filter_variable(both, allow_convert=False)
    c = t.filter_variable(np.ones((3, 1), "float32"))
    assert c.type == t and c.data.shape == (3, 1)


def test_gradient_only_operations(dry_run):
    """zero_grad / disconnected_grad / undefined_grad / grad_clip / grad_scale (theano/gradient.py:2022-2300):
    identity in the forward pass - compiled graphs do not contain them - and the documented effect on gradients."""
    from theano_amd import gradient as G
    x = T.fvector("x")
    f = th.function([x], [G.grad_clip(x * x, -1, 1).sum(), G.zero_grad(x) + G.disconnected_grad(x) + G.grad_scale(x, 2)])
    assert not any(isinstance(n.op, G._GradView) for n in f.toposort())
    g = th.grad(T.sum(G.zero_grad(T.exp(x)) * x), x)          # exp(x) counts as a constant: d/dx = exp(x)
    ops = [str(n.op) for n in th.function([x], g).toposort()]
    assert len(ops) == 3 and "exp" in ops[1] and "0.0" in ops[1], ops      # exp(x) + 0 * exp(x): zeros flow back
    g = th.grad(T.sum(G.disconnected_grad(T.exp(x)) * x), x)
    assert [str(n.op) for n in th.function([x], g).toposort()] == ["HostToHip", "HipElemwise{exp}", "HipToHost"]
    with pytest.raises(G.DisconnectedInputError):
        th.grad(T.sum(G.disconnected_grad(x)), x, disconnected_inputs="raise")
    assert th.grad(T.sum(G.zero_grad(x)), x, disconnected_inputs="raise") is not None    # connected, with zeros
    with pytest.raises(G.NullTypeGradError, match="mathematically undefined"):
        th.grad(T.sum(G.undefined_grad(x) * 2), x)
    with pytest.warns(UserWarning, match="deprecated"):
        G.consider_constant(x)
    with pytest.raises(ValueError):
        G.GradClip(1, -1)
    assert G.GradClip(0, 1) == G.GradClip(-5, 5) and G.zero_grad_ == G.ZeroGrad() and G.zero_grad_ != G.disconnected_grad_
    g = th.grad(T.sum(G.grad_scale(T.exp(x), 0.5)), x)
    assert "0.5" in " ".join(str(n.op) for n in th.function([x], g).toposort())


def test_operand_of_a_max_that_something_else_reads_is_stored_not_recomputed(dry_run):
    """A cheap elementwise result read by a sum and by another kernel is recomputed in each; read by a max or
    min (whose gradient compares the result with the operand for equality) it is computed and stored once."""
    x = T.fmatrix("x")
    e = T.exp(x * 2.0)
    f = th.function([x], [T.sum(e, axis=0), e * 3.0], rowchain=False)
    red = [n.op for n in f.toposort() if isinstance(n.op, HipCAReduce)]
    assert len(red) == 1 and red[0].pre_scalar_op is not None              # recomputed inside the sum
    for reducer in (T.max, T.min):
        f = th.function([x], [reducer(e, axis=0), e * 3.0], rowchain=False)
        red = [n.op for n in f.toposort() if isinstance(n.op, HipCAReduce)]
        assert len(red) == 1 and red[0].pre_scalar_op is None, red              # reads the stored values
    i = T.imatrix("i")
    f = th.function([i], [T.max(i * 2 + 1, axis=0), (i * 2 + 1) * 3], rowchain=False)   # integers are exact: recomputed
    red = [n.op for n in f.toposort() if isinstance(n.op, HipCAReduce)]
    assert len(red) == 1 and red[0].pre_scalar_op is not None
    # a batch-norm-shaped chain evaluates its closures once per loop: fine for a max whose result is only used
    # arithmetically, not when a later step tests it against the value for equality (the gradient of max)
    x4 = T.ftensor4("x4")
    e4 = T.exp(x4 * 0.5)
    m4 = T.max(e4, axis=(0, 2, 3), keepdims=True)

    def held_chains(f):
        return [n for n in f.toposort() if type(n.op).__name__ == "HipRowChain" and n.op.program.axes == (0, 2, 3)]
    assert len(held_chains(th.function([x4], e4 / m4 + T.sum(e4, axis=(0, 2, 3), keepdims=True)))) == 1
    g = th.grad(T.sum(T.max(e4, axis=(0, 2, 3)) * T.sum(e4, axis=(0, 2, 3))), x4)
    f = th.function([x4], g)
    assert not held_chains(f)
    red = [n.op for n in f.toposort() if isinstance(n.op, HipCAReduce)]
    assert red and all(r.pre_scalar_op is None or "exp" not in str(r.pre_scalar_op) for r in red)


def test_input_options(dry_run):
    """In(strict=, allow_downcast=, mutable=, borrow=) and function(allow_input_downcast=)
    (theano/compile/io.py:40-216, theano/compile/function.py:70-300)."""
    from theano_amd.compile import In
    x = T.fvector("x")
    v64, v32 = np.ones(4, "float64"), np.ones(4, "float32")
    f = th.function([x], x + 1)
    f(v32)
    with pytest.raises(TypeError, match="precision"):
        f(v64)                                                    # float64 values do not go into a float32 input
    th.function([x], x + 1, allow_input_downcast=True)(v64)
    th.function([In(x, allow_downcast=True)], x + 1)(v64)
    g = th.function([In(x, strict=True)], x + 1)
    g(v32)
    for bad in ([1.0, 2.0, 3.0, 4.0], np.ones(4, "float16"), v64):
        with pytest.raises(TypeError):
            g(bad)                                                # strict: no conversion at all
    f([1.0, 2.0])                                                  # without it Python numbers convert
    spec = In(x, mutable=True)
    assert spec.mutable and spec.borrow and In(x, borrow=True).mutable and not In(x).mutable
    assert In(x, name="data").name == "data" and In(x).name == "x"
    with pytest.raises(ValueError):
        In(x, strict=True, allow_downcast=True)
    with pytest.raises(NotImplementedError):
        In(x, value=v32)


def test_type_constructors_of_every_rank_and_their_plurals():
    """tensor5 ... tensor7 with their dtype prefixes, and matrices('a', 'b') / fvectors(3) ...
    (theano/tensor/basic.py:644-790)."""
    assert T.tensor5().type.ndim == 5 and T.ftensor6("u").type == T.TensorType("float32", (False,) * 6)
    assert T.ztensor7().type.dtype == "complex128" and T.btensor5().type.dtype == "int8" and T.ltensor7("q").name == "q"
    a, b = T.fmatrices("a", "b")
    assert a.type == b.type == T.fmatrix().type and (a.name, b.name) == ("a", "b")
    assert [v.type.ndim for v in T.tensor3s(2)] == [3, 3] and T.ivectors("k").type == T.ivector().type
    assert [v.name for v in T.dscalars(["p", "q", "r"])] == ["p", "q", "r"]
    assert T.lrows("r").type.broadcastable == (True, False) and T.dcols("c").type.broadcastable == (False, True)
    assert len(T.tensor7s("a", "b", "c")) == 3 and T.dtensor5s("u", "v")[1].type.ndim == 5


def test_batch_normalization_with_given_statistics_and_nnet_aliases(dry_run):
    """nnet.batch_normalization (theano/tensor/nnet/bn.py:14-97): 'low_mem' is one Elemwise over BNComposite whose
    written-out gradients equal those of the 'high_mem' expression; the scalar ops and in-place variants that
    sigm.py exports (:29-300)."""
    import pickle
    from oracle import graph_ref as G
    from theano_amd.tensor import nnet as N
    x = T.fmatrix("x")
    g, b, m, s = [T.frow(n) for n in "gbms"]
    ins = [x, g, b, m, s]
    lo, hi = N.batch_normalization(x, g, b, m, s), N.batch_normalization(x, g, b, m, s, "high_mem")
    assert isinstance(lo.owner.op.scalar_op, N.BNComposite) and len(lo.owner.inputs) == 5
    rng = np.random.default_rng(0)
    vals = [rng.standard_normal((5, 7)).astype("float32")] + [rng.uniform(0.5, 1.5, (1, 7)).astype("float32") for _ in range(4)]
    r = G.evaluate(ins, [lo, hi] + th.grad(T.sum(lo * x), ins) + th.grad(T.sum(hi * x), ins), vals)
    xv, gv, bv, mv, sv = [v.astype("float64") for v in vals]
    np.testing.assert_allclose(r[0], (xv - mv) / sv * gv + bv, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(r[1], r[0], rtol=1e-5, atol=1e-6)
    for a, c in zip(r[2:7], r[7:12]):
        np.testing.assert_allclose(a, c, rtol=3e-5, atol=2e-6)
    assert pickle.loads(pickle.dumps(lo.owner.op)) == lo.owner.op
    with pytest.raises(ValueError, match="low_mem"):
        N.batch_normalization(x, g, b, m, s, "medium_mem")
    f = th.function(ins, [lo] + th.grad(T.sum(lo * x), ins))
    assert sum(isinstance(n.op, HipElemwise) for n in f.toposort()) == 1        # forward and dx in one kernel
    assert N.ScalarSigmoid is scal.ScalarSigmoid and N.scalar_softplus is scal.scalar_softplus
    assert N.ultra_fast_scalar_sigmoid is scal.ultra_fast_scalar_sigmoid
    for op, base in ((N.sigmoid_inplace, scal.ScalarSigmoid), (N.softplus_inplace, scal.ScalarSoftplus),
                     (N.ultra_fast_sigmoid_inplace, scal.UltraFastScalarSigmoid)):
        assert isinstance(op.scalar_op, base) and op.destroy_map == {0: [0]} and op(x).type == x.type


def test_device_type_value_helpers(dry_run):
    """HipArrayType: filter_variable / convert_variable (a host variable is moved, a broader broadcast pattern is
    narrowed), may_share_memory for views of one allocation, value_zeros, get_size, values_eq(_approx)
    (theano/gpuarray/type.py:204-420)."""
    from theano_amd.hip.ops import HipArrayType
    from theano_amd.hip.runtime import HipArray
    t = HipArrayType("float32", (False, True))
    for v in (T.fcol(), T.TensorType("float32", (True, True))(), HipArrayType("float32", (True, True))(), t()):
        assert t.filter_variable(v).type == t
    own = t()
    assert t.filter_variable(own) is own and t.convert_variable(T.dmatrix()) is None and t.convert_variable(T.fmatrix()) is None
    with pytest.raises(TypeError, match="Cannot convert Type"):
        t.filter_variable(T.fmatrix())
    assert t.filter_variable(np.ones((2, 1), "float32")).type == t
    a = HipArray.empty((4, 1), "float32")
    assert t.may_share_memory(a, a.view((2, 1), (4, 4))) and not t.may_share_memory(a, HipArray.empty((4, 1), "float32"))
    assert not t.may_share_memory(a, np.zeros(3)) and t.get_size(t.get_shape_info(a)) == 16
    z = t.value_zeros((3, 1))
    assert isinstance(z, HipArray) and z.shape == (3, 1) and str(z.dtype) == "float32"
    assert t.values_eq(a, a) and t.values_eq_approx(a, a) and not t.values_eq(a, z)
    c = T.TensorType("float32", (True, True))("c")
    f = th.function([c], t.filter_variable(c) + 1)
    assert [type(n.op).__name__ for n in f.toposort()][0] == "HostToHip"


def test_shape_only_nodes_rerun_when_list_arguments_change_length(dry_run):
    """The extent `mean` divides by is kept between calls with equal argument shapes; the shapes are those of
    the filtered values, so two Python lists of different lengths (which have no `.shape` themselves) count as
    different and the extent is read again."""
    from theano_amd.tensor.basic import ShapeFloat
    x = T.fvector("x")
    f = th.function([x], T.mean(x))
    runs = []
    nodes = [n for n in f.nodes if isinstance(n.op, ShapeFloat)]
    assert nodes
    for k, th_ in enumerate(f.thunks):
        if th_[1] in nodes:
            perform = th_[0]

            def counted(node, ins, outs, _p=perform):
                runs.append(tuple(np.shape(i) for i in ins))
                return _p(node, ins, outs)
            f.thunks[k] = (counted,) + tuple(th_[1:])
    f([1, 2, 3])
    f([1, 2, 3])
    assert runs == [((3,),)]
    f([1, 2, 3, 4])
    assert runs == [((3,),), ((4,),)]
    f(np.zeros(4, "float32"))
    assert len(runs) == 2
    f(np.zeros(5, "float32"))
    assert len(runs) == 3


def test_reshape_with_a_shape_vector_argument(dry_run):
    """reshape(x, v, ndim=n) with v an integer vector argument (theano/tensor/basic.py:4858-4960, 5049-5068): the rank
    comes from ndim, the vector stays on the host, its elements are checked when the function runs."""
    from theano_amd.tensor.views import Reshape
    x, s = T.fmatrix("x"), T.lvector("s")
    y = x.reshape(s, ndim=3)
    assert isinstance(y.owner.op, Reshape) and y.type.ndim == 3 and str(y.owner.op) == "Reshape{in1[0], in1[1], in1[2]}"
    assert T.reshape(x, s, ndim=3).owner.op == y.owner.op
    f = th.function([x, s], y + 1)
    names = [type(n.op).__name__ for n in f.toposort()]
    assert names.count("HostToHip") == 1 and "HipReshape" in names
    xv = np.zeros((4, 6), "float32")
    assert f(xv, [2, 3, 4]).shape == (2, 3, 4) and f(xv, np.array([4, -1, 2])).shape == (4, 3, 2)
    for bad in ([2, 3], [5, 5, 1], [-1, -1, 6]):
        with pytest.raises(ValueError):
            f(xv, bad)
    with pytest.raises(ValueError, match="ndim"):
        T.reshape(x, s)
    with pytest.raises(ValueError):
        x.reshape((2, 12), ndim=3)
    z = T.alloc(np.float32(1.5), s[0], s[1] * 2)
    assert str(z.owner.op) == "Alloc{in1[0], mul(in1[1], 2)}"
    g = th.function([s], z)
    assert [type(n.op).__name__ for n in g.toposort()] == ["HipAlloc", "HipToHost"] and g([3, 4]).shape == (3, 8)


def test_grad_arguments_of_the_reference(dry_run):
    """``theano.grad``'s arguments and corner cases as the reference's tests state them
    (``theano/tests/test_gradient.py``: test_grad_name :205, test_downcast_dtype :394, test_grad_constant :414,
    test_dxdx :487, test_known_grads_integers :504, test_undefined_cost_grad :522, test_disconnected_cost_grad :540,
    TestConsiderConstant :603-640, TestDisconnectedGrad :698-770)."""
    import inspect
    import warnings
    from theano_amd import gradient as GR
    from oracle import graph_ref as G
    fx = lambda v: np.asarray(v, th.config.floatX)                          # noqa: E731
    assert list(inspect.signature(th.grad).parameters) == [
        "cost", "wrt", "consider_constant", "disconnected_inputs", "add_names", "known_grads", "return_disconnected",
        "null_gradients"]
    assert inspect.signature(th.grad).parameters["disconnected_inputs"].default == "raise"
    # names
    x, A = T.vector("x"), T.matrix("A")
    f = T.sum(x * T.sum(A * x.dimshuffle("x", 0), axis=1))
    f.name = "f"
    assert th.grad(f, x).name == "(df/dx)" and th.grad(f, x, add_names=False).name is None
    # what flows back to a float32 variable is float32, whatever the cost was promoted to
    xs = T.fscalar("x")
    y = xs * 2
    z = T.lscalar("z")
    c = y + z
    dc_dx, dc_dy, dc_dz, dc_dc = th.grad(c, [xs, y, z, c])
    assert dc_dx.dtype == "float32" and all(g.dtype in ("float32", "float64") for g in (dc_dy, dc_dz, dc_dc))
    # a tuple in, a tuple out
    assert isinstance(th.grad(c, (xs, y)), tuple) and isinstance(th.grad(c, [xs, y]), list)
    # consider_constant stops what goes through an expression, not what arrives at it
    a, b = T.scalar("a"), T.scalar("b")
    g_a = th.grad(a + b, a, consider_constant=[a])
    assert float(G.evaluate([a, b], [g_a], [fx(1.0), fx(0.5)])[0]) == 1.0
    w = a * 3
    with pytest.raises(GR.DisconnectedInputError):
        th.grad(w + b, a, consider_constant=[w])
    g = th.grad(w * w + a, a, consider_constant=[w])                        # only the direct term survives
    assert float(G.evaluate([a], [g], [fx(2.0)])[0]) == 1.0
    # d x / d x of an integer is 1
    i = T.iscalar("i")
    assert float(G.evaluate([i], [th.grad(i, i)], [np.int32(12)])[0]) == 1.0
    ge = T.scalar("ge")
    g = th.grad(cost=None, known_grads={i: ge}, wrt=i)
    assert float(G.evaluate([ge], [g], [fx(0.6)])[0]) == np.asarray(0.6, th.config.floatX)
    # a cost declared undefined / disconnected through known_grads
    j = T.iscalar("j")
    cost = i + j
    with pytest.raises(GR.NullTypeGradError):
        th.grad(cost, [i, j], known_grads={cost: GR.NullType()()})
    assert isinstance(th.grad(cost, i, known_grads={cost: GR.NullType()()}, null_gradients="return").type, GR.NullType)
    with pytest.raises(GR.DisconnectedInputError):
        th.grad(cost, [i, j], known_grads={cost: GR.DisconnectedType()()}, disconnected_inputs="raise")
    # what comes back for a variable outside the graph
    u = T.vector("u")
    with pytest.raises(GR.DisconnectedInputError):
        th.grad(T.sum(x), u)
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        zero = th.grad(T.sum(x), u, disconnected_inputs="warn")
    assert len(seen) == 1 and "not part of the computational graph" in str(seen[0].message)
    assert np.array_equal(G.evaluate([u], [zero], [fx(np.ones(3))])[0], np.zeros(3))
    assert th.grad(T.sum(x), u, disconnected_inputs="ignore", return_disconnected="None") is None
    d = th.grad(T.sum(x), u, disconnected_inputs="ignore", return_disconnected="Disconnected")
    assert isinstance(d.type, GR.DisconnectedType)
    for bad in (dict(disconnected_inputs="zero"), dict(return_disconnected="none"), dict(null_gradients="ignore")):
        with pytest.raises(ValueError):
            th.grad(T.sum(x), x, **bad)
    # reaching the cost through an integer-valued result only: connected, zeros
    gz = th.grad(T.sum(T.cast(T.gt(x, 0), "float32")), x)
    assert np.array_equal(G.evaluate([x], [gz], [fx(np.arange(3.0))])[0], np.zeros(3))
    # the first operand of fill is not connected (theano/scalar/basic.py:2283-2287)
    with pytest.raises(GR.DisconnectedInputError):
        th.grad(T.sum(T.fill(x, a)), x)


def test_function_takes_the_references_arguments_in_its_order(dry_run):
    """``theano.function(inputs, outputs=None, mode=None, updates=None, givens=None, no_default_updates=False,
    accept_inplace=False, name=None, rebuild_strict=True, allow_input_downcast=None, profile=None,
    on_unused_input=None)`` (``theano/compile/function.py:74-77``); unused inputs
    (``theano/compile/function_module.py:1594-1625``)."""
    import inspect
    import warnings
    params = inspect.signature(th.function).parameters
    assert list(params)[:12] == ["inputs", "outputs", "mode", "updates", "givens", "no_default_updates", "accept_inplace",
                                 "name", "rebuild_strict", "allow_input_downcast", "profile", "on_unused_input"]
    assert all(params[p].kind is inspect.Parameter.KEYWORD_ONLY for p in list(params)[12:])
    x, y = T.fvector("x"), T.fvector("y")
    s = th.shared(np.zeros(3, "float32"))
    f = th.function([x], x * 2, None, [(s, s + x)])                  # mode, then updates, by position
    assert f.update_targets == [s]
    assert th.function([x], None, updates=[(s, s + x)])(np.ones(3, "float32")) == []
    with pytest.raises(th.UnusedInputError, match="index 1 is not part"):
        th.function([x, y], x * 2)
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        th.function([x, y], x * 2, on_unused_input="warn")
    assert len(seen) == 1 and "on_unused_input='raise'" in str(seen[0].message)
    th.function([x, y], x * 2, on_unused_input="ignore")
    with pytest.raises(ValueError):
        th.function([x], x * 2, on_unused_input="never")


def test_shared_takes_the_references_arguments(dry_run):
    """``theano.shared(value, name=None, strict=False, allow_downcast=None, **kwargs)``
    (``theano/compile/sharedvalue.py:238-300``) with the device constructor's keywords."""
    import inspect
    assert list(inspect.signature(th.shared).parameters) == ["value", "name", "strict", "allow_downcast", "kwargs"]
    s = th.shared(np.zeros((1, 3), "float32"), "s", broadcastable=(True, False), borrow=True)
    assert s.name == "s" and s.type.broadcastable == (True, False)
    s.set_value(np.ones((1, 3), "float32"))
    with pytest.raises(TypeError):
        s.set_value(np.ones((1, 3), "float64"))             # would lose precision
    d = th.shared(np.zeros(3, "float32"), allow_downcast=True)
    d.set_value(np.ones(3, "float64"))
    assert d.get_value().dtype == np.float32
    with pytest.raises(TypeError):
        th.shared(np.zeros(3), colour="red")


def test_float16_softmax_and_its_gradient_are_one_row_chain(dry_run):
    """The row maximum of a float16 softmax has a float16 accumulator; it joins the row chain like the float32 one
    (a maximum picks one of the values whatever the arithmetic's width), so forward and gradient are one kernel and
    x is read once.  Sums keep their float32 accumulators (theano/tensor/elemwise.py:1395-1398)."""
    import numpy as np
    import theano_amd as th
    from theano_amd import tensor as T
    from theano_amd.hip import HipRowChain, HipCAReduce
    for dtype in ("float16", "float32"):
        x = T.TensorType(dtype, (False, False))("x")
        g = T.TensorType(dtype, (False, False))("g")
        sm = T.nnet.softmax(x)
        for outs in ([sm], [sm, th.grad(T.sum(sm * g), x)], [x - T.max(x, axis=1, keepdims=True)]):
            f = th.function([x, g], outs, on_unused_input="ignore")
            ops = [n.op for n in f.toposort()]
            assert sum(isinstance(o, HipRowChain) for o in ops) == 1, (dtype, ops)
            assert not any(isinstance(o, HipCAReduce) for o in ops), (dtype, ops)
            f(np.ones((8, 1001), dtype), np.ones((8, 1001), dtype))
