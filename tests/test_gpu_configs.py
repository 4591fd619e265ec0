"""The five benchmark configurations: parity against the oracle at reduced
size, size-independent properties at full size."""
import numpy as np
import pytest

import theano_amd as th
from theano_amd import hip, tensor as T
from oracle import graph_ref as G
from conftest import assert_parity, assert_within_reference_error
import workloads as W

pytestmark = pytest.mark.gpu


def parity(graph, vals, what, tol=None):
    ins, outs = graph
    got = th.function(ins, outs)(*vals)
    ref = G.evaluate(ins, outs, vals)
    for k, (g, r) in enumerate(zip(got, ref)):
        assert_parity(g, r, "%s output %d" % (what, k), tol=tol)
    return got


def test_config1_small_and_full():
    parity(W.c1_graph(), W.c1_inputs("small"), "c1 small")
    ins, outs = W.c1_graph()
    x, a, b = W.c1_inputs("full")
    got = th.function(ins, outs)(x, a, b)[0]
    t = (a * x + b).astype("float64")
    ref = (np.where(t < -88, 0.0, np.where(t > 15, 1.0, 1 / (1 + np.exp(-t)))) * x).astype("float32")
    assert_parity(got, ref, "c1 full")


@pytest.mark.parametrize("case", W.C2_CASES)
def test_config2(case):
    parity(W.c2_graph(case), W.c2_inputs(case, "small"), "c2 %s small" % case)
    ins, outs = W.c2_graph(case)
    (x,) = W.c2_inputs(case, "full")
    got = th.function(ins, outs)(x)[0]
    x64 = x.astype("float64")
    ref = {"sum_axis1": lambda: x64.sum(1), "max_axis1": lambda: x.max(1), "sum_axis0": lambda: x64.sum(0),
           "sum_all": lambda: x64.sum(), "prod_axis1": lambda: x64.prod(1)}[case]()
    assert_parity(got, np.asarray(ref).astype("float32"), "c2 %s full" % case)


def test_config3_softmax_and_gradient():
    parity(W.c3_graph(with_grad=False), W.c3_inputs("small", with_grad=False), "c3 fwd small")
    parity(W.c3_graph(), W.c3_inputs("small"), "c3 fwd+grad small")
    ins, outs = W.c3_graph()
    x, y = W.c3_inputs("full")
    out, dx = th.function(ins, outs)(x, y)
    # rows of a softmax sum to one, rows of its gradient sum to zero, argmax is preserved
    assert np.allclose(out.astype("float64").sum(1), 1.0, atol=1e-5)
    assert np.abs(dx.astype("float64").sum(1)).max() < 1e-5
    assert np.array_equal(out.argmax(1), x.argmax(1))
    rows = slice(0, 64)
    e = np.exp(x[rows].astype("float64") - x[rows].max(1, keepdims=True))
    sm = e / e.sum(1, keepdims=True)
    assert_parity(out[rows], sm.astype("float32"), "c3 full rows")
    # dx = sm * (y - sum(sm * y)): where y is close to the row's weighted mean the float32 difference has
    # lost digits before the multiply, in the reference's evaluation as much as here (the oracle is up to
    # 4 bars from the float64 value on such elements): held to the float64 value, no farther than the oracle is
    ref = G.evaluate(ins, outs, [x[rows], y[rows]])
    assert_within_reference_error(dx[rows], ref[1], sm * (y[rows] - (sm * y[rows]).sum(1, keepdims=True)), "c3 grad rows")


def test_config3_gradient_alone_full_size():
    """The gradient of config 3 given only x and y (no softmax among the results): one launch that reads x and y and
    writes dx; rows of dx sum to zero, the first rows equal the closed form and what the forward + gradient
    function returns."""
    from theano_amd.hip import HipRowChain
    parity(W.c3_graph(forward=False), W.c3_inputs("small"), "c3 grad alone small")
    ins, outs = W.c3_graph(forward=False)
    x, y = W.c3_inputs("full")
    f = th.function(ins, outs)
    kernels = [n for n in f.toposort() if type(n.op).__name__ in ("HipElemwise", "HipCAReduce", "HipRowChain")]
    assert len(kernels) == 1 and isinstance(kernels[0].op, HipRowChain), kernels
    (dx,) = f(x, y)
    assert dx.shape == x.shape and dx.dtype == np.float32
    assert np.abs(dx.astype("float64").sum(1)).max() < 1e-5
    rows = slice(0, 64)
    e = np.exp(x[rows].astype("float64") - x[rows].max(1, keepdims=True))
    sm = e / e.sum(1, keepdims=True)
    ref = G.evaluate(ins, outs, [x[rows], y[rows]])
    assert_within_reference_error(dx[rows], ref[0], sm * (y[rows] - (sm * y[rows]).sum(1, keepdims=True)), "c3 grad alone rows")
    ins2, outs2 = W.c3_graph()
    both = th.function(ins2, outs2)(x[:4096], y[:4096])
    assert_parity(dx[:4096], both[1], "gradient alone against forward + gradient")


def test_config4_integer_path():
    parity(W.c4_graph("all"), W.c4_inputs("small"), "c4 small")
    ins, outs = W.c4_graph("all")
    a, b, bias = W.c4_inputs("full")
    r, s, any_, all_ = th.function(ins, outs)(a, b, bias)
    ref = (((a & b) ^ (a >> 3)) % 97 + bias).transpose(0, 2, 3, 1)
    assert r.shape == ref.shape and np.array_equal(r, ref)
    assert np.array_equal(s, ref.astype("int64").sum((0, 1, 2)))     # checksum of the elementwise result
    assert np.array_equal(s, r.astype("int64").sum((0, 1, 2)))
    assert bool(any_) == bool((a > 0).any()) and bool(all_) == bool((a > 0).all())


def test_config5_batchnorm_float16():
    tol = dict(rtol=2e-3, atol=2e-3)
    parity(W.c5_graph(with_grad=False), W.c5_inputs("small", with_grad=False), "c5 fwd small", tol)
    parity(W.c5_graph(), W.c5_inputs("small"), "c5 fwd+grad small", tol)
    ins, outs = W.c5_graph(with_grad=False)
    x, gamma, beta = W.c5_inputs("full", with_grad=False)
    y = th.function(ins, outs)(x, gamma, beta)[0]
    # normalised activations: per-channel mean beta and standard deviation |gamma|
    yf = y.astype("float64")
    assert np.allclose(yf.mean((0, 2, 3)), beta.astype("float64").reshape(-1), atol=2e-3)
    assert np.allclose(yf.std((0, 2, 3)), np.abs(gamma.astype("float64")).reshape(-1), rtol=2e-3, atol=2e-3)
    ch = 7
    xc = x[:, ch].astype("float64")
    ref = gamma.astype("float64")[0, ch] * (xc - xc.mean()) / np.sqrt(xc.var() + 1e-5) + beta.astype("float64")[0, ch]
    assert_parity(y[:, ch], ref.astype("float16"), "c5 full channel", tol)


def test_config5_gradient_full_size():
    """The kernels the benchmark times for configuration 5's gradient, checked at full size
    (256, 256, 28, 28): per channel dbeta = sum(g) and dgamma = sum(g * xhat) against float64 NumPy over
    all 200 704 terms, dx against the closed form of AbstractBatchNormTrainGrad.perform
    (theano/tensor/nnet/bn.py:659-676) on whole channels; float16 results at the float16 bar."""
    tol = dict(rtol=2e-3, atol=2e-3)
    ins, outs = W.c5_graph(forward=False)
    x, gamma, beta, g = W.c5_inputs("full")
    f = th.function(ins, outs)
    dx, dgamma, dbeta = f(x, gamma, beta, g)
    assert dx.dtype == dgamma.dtype == dbeta.dtype == np.float16
    assert dx.shape == x.shape and dgamma.shape == gamma.shape and dbeta.shape == beta.shape
    m = x.shape[0] * x.shape[2] * x.shape[3]
    sum_g = np.zeros(x.shape[1]); sum_gxh = np.zeros(x.shape[1])
    mean, istd = np.zeros(x.shape[1]), np.zeros(x.shape[1])
    for c in range(x.shape[1]):                      # channel by channel: float64 copies of the whole arrays are 0.8 GB
        xc, gc = x[:, c].astype("float64"), g[:, c].astype("float64")
        mean[c] = xc.mean()
        istd[c] = 1.0 / np.sqrt(((xc - mean[c]) ** 2).mean() + np.float64(np.float32(1e-5)))
        sum_g[c] = gc.sum()
        sum_gxh[c] = (gc * (xc - mean[c]) * istd[c]).sum()
    assert_parity(dbeta.reshape(-1), sum_g.astype("float16"), "c5 full dbeta", tol)
    assert_parity(dgamma.reshape(-1), sum_gxh.astype("float16"), "c5 full dgamma", tol)
    gam = gamma.astype("float64").reshape(-1)
    for c in (0, 7, 130, 255):
        xc, gc = x[:, c].astype("float64"), g[:, c].astype("float64")
        xh = (xc - mean[c]) * istd[c]
        want = gam[c] * istd[c] * (gc - sum_g[c] / m - xh * sum_gxh[c] / m)
        assert_parity(dx[:, c], want.astype("float16"), "c5 full dx channel %d" % c, tol)
    # forward + gradient in one function (the other graph the benchmark compiles): same gradients
    ins2, outs2 = W.c5_graph()
    y, dx2, dgamma2, dbeta2 = th.function(ins2, outs2)(x, gamma, beta, g)
    assert_parity(dbeta2.reshape(-1), sum_g.astype("float16"), "c5 full fwd+grad dbeta", tol)
    assert_parity(dgamma2.reshape(-1), sum_gxh.astype("float16"), "c5 full fwd+grad dgamma", tol)
    assert_parity(dx2[:, 7], dx[:, 7], "c5 full fwd+grad dx", tol)
    xh = (x[:, 7].astype("float64") - mean[7]) * istd[7]
    assert_parity(y[:, 7], (gam[7] * xh + beta.astype("float64").reshape(-1)[7]).astype("float16"), "c5 full y", tol)


def test_nnet_row_functions_run_as_row_chains():
    """softmax_with_bias / logsoftmax / relu of tensor.nnet against the oracle's
    node-by-node evaluation of the same formulas (the ops' perform code,
    theano/tensor/nnet/nnet.py:440-446, 628-633, 2209-2252), forward and gradient."""
    from theano_amd.hip import HipRowChain
    rng = np.random.default_rng(41)
    x, y = T.fmatrix("x"), T.fmatrix("y")
    b = T.fvector("b")
    xv = (3 * rng.standard_normal((130, 777))).astype("float32")
    yv = rng.uniform(0, 1, (130, 777)).astype("float32")
    bv = rng.standard_normal(777).astype("float32")
    lsm = T.nnet.logsoftmax(x)
    swb = T.nnet.softmax_with_bias(x, b)
    outs = [lsm, swb, T.nnet.relu(x), T.nnet.relu(x, 0.1), th.grad(T.sum(lsm * y), x), th.grad(T.sum(swb * y), b)]
    f = th.function([x, y, b], outs)
    assert any(isinstance(n.op, HipRowChain) for n in f.toposort())
    got = f(xv, yv, bv)
    ref = G.evaluate([x, y, b], outs, [xv, yv, bv])
    truth = G.evaluate([x, y, b], outs, [xv, yv, bv], wide=True)
    for k, (g, r, w) in enumerate(zip(got, ref, truth)):
        # gradients of (log-)softmax subtract nearly equal float32 numbers: see assert_within_reference_error
        assert_within_reference_error(g, r, w, "nnet output %d" % k)
    assert np.allclose(np.exp(got[0]).sum(axis=1), 1.0, atol=1e-5)
    assert np.allclose(got[1].sum(axis=1), 1.0, atol=1e-5)


def test_batch_normalization_helpers_forward_grad_and_inference():
    """tensor.nnet.batch_normalization_train / _train_grad / _test (the graphs
    the reference lowers its AbstractBatchNorm ops to, theano/tensor/nnet/bn.py:679-789)
    against the oracle; the explicit gradient formula and grad() of the forward
    graph must agree with each other as well."""
    rng = np.random.default_rng(42)
    t4 = T.TensorType("float32", (False,) * 4)
    pc = T.TensorType("float32", (True, False, True, True))
    x, dy = t4("x"), t4("dy")
    g, b, rm, rv = pc("g"), pc("b"), pc("rm"), pc("rv")
    out, mean, invstd, nrm, nrv = T.nnet.batch_normalization_train(x, g, b, "spatial", 1e-5, 0.1, rm, rv)
    gx, gg, gb = T.nnet.batch_normalization_train_grad(x, dy, g, mean, invstd, "spatial")
    ax, ag, ab = th.grad(T.sum(out * dy), [x, g, b])
    inf = T.nnet.batch_normalization_test(x, g, b, rm, rv, "spatial", 1e-5)
    outs = [out, mean, invstd, nrm, nrv, gx, gg, gb, ax, ag, ab, inf]
    vals = [rng.normal(0.5, 2.0, (9, 33, 7, 11)).astype("float32"), rng.standard_normal((9, 33, 7, 11)).astype("float32"),
            rng.uniform(0.5, 1.5, (1, 33, 1, 1)).astype("float32"), rng.standard_normal((1, 33, 1, 1)).astype("float32"),
            rng.standard_normal((1, 33, 1, 1)).astype("float32"), rng.uniform(0.5, 1.5, (1, 33, 1, 1)).astype("float32")]
    ins = [x, dy, g, b, rm, rv]
    got = th.function(ins, outs)(*vals)
    ref = G.evaluate(ins, outs, vals)
    truth = G.evaluate(ins, outs, vals, wide=True)
    for k, (a, r, w) in enumerate(zip(got, ref, truth)):
        # x - mean and the two-term gradient formulas cancel leading digits in float32, in the reference's
        # evaluation order as in any other: see assert_within_reference_error
        assert_within_reference_error(a, r, w, "batch norm output %d" % k)
    xhat = (got[0] - vals[3]) / vals[2]
    assert np.allclose(xhat.mean(axis=(0, 2, 3)), 0, atol=1e-5) and np.allclose(xhat.std(axis=(0, 2, 3)), 1, atol=1e-3)


def test_more_than_2_to_31_elements_use_64_bit_indexing():
    """A 2^31 + 4096 element int8 vector (and its (2, n/2) view): elementwise,
    row and column reductions and argmax index with 64-bit offsets; results
    against NumPy on the whole array."""
    n = 2 ** 31 + 4096
    rng = np.random.default_rng(43)
    base = rng.integers(-100, 100, 1 << 20).astype("int8")
    val = np.tile(base, n // base.size + 1)[:n]
    val[n - 5] = 127                                   # the last maximum sits beyond 2^31
    val[7] = -128
    v = T.TensorType("int8", (False,))("v")
    f = th.function([v], [T.sum(v), T.max_and_argmax(v)[1], th.Out((v + np.int8(1)) ^ np.int8(3), device=True)])
    s, am, ew = f(val)
    assert "i64" in hip.last_plan()
    assert s == val.sum(dtype=np.int64)
    assert am == int(np.argmax(val))
    tail = ew.to_numpy()[n - 4096:]
    assert np.array_equal(tail, (val[n - 4096:] + np.int8(1)) ^ np.int8(3))
    del ew
    m = T.TensorType("int8", (False, False))("m")
    g = th.function([m], [T.sum(m, axis=1), T.sum(m, axis=0)])
    r1, r0 = g(val.reshape(2, n // 2))
    assert np.array_equal(r1, val.reshape(2, n // 2).sum(axis=1, dtype=np.int64))
    assert np.array_equal(r0[:4096], val.reshape(2, n // 2)[:, :4096].sum(axis=0, dtype=np.int64))
    assert r0.sum() == s


def test_sgd_steps_with_shared_weights_and_updates():
    """Ten steps of logistic regression on device-resident weights (shared
    variables updated by the function itself) against the same steps in NumPy."""
    rng = np.random.default_rng(44)
    n, d = 512, 96
    xv = rng.standard_normal((n, d)).astype("float32")
    tv = (rng.uniform(size=(n, 1)) < 0.5).astype("float32")
    w0 = (0.1 * rng.standard_normal((1, d))).astype("float32")
    w = th.shared(w0, name="w", broadcastable=(True, False))
    b = th.shared(np.zeros((1, 1), "float32"), name="b", broadcastable=(True, True))
    x, t = T.fmatrix("x"), T.fcol("t")
    z = T.sum(x * w, axis=1, keepdims=True) + b
    p = T.sigmoid(z)
    loss = T.mean(-t * T.log(p) - (1 - t) * T.log(1 - p))
    gw, gb = th.grad(loss, [w, b])
    lr = np.float32(0.5)
    step = th.function([x, t], loss, updates=[(w, w - lr * gw), (b, b - lr * gb)])
    wn, bn = w0.astype("float64"), np.zeros((1, 1))
    for _ in range(10):
        got = float(step(xv, tv))
        zn = (xv * wn).sum(axis=1, keepdims=True) + bn
        pn = 1 / (1 + np.exp(-zn))
        ref = float(np.mean(-tv * np.log(pn) - (1 - tv) * np.log(1 - pn)))
        assert abs(got - ref) < 1e-4 * max(1.0, abs(ref))
        dz = (pn - tv) / n
        wn = wn - 0.5 * (dz * xv).sum(axis=0, keepdims=True)
        bn = bn - 0.5 * dz.sum(keepdims=True)
    assert np.allclose(w.get_value(), wn, rtol=1e-3, atol=1e-4)
    assert np.allclose(b.get_value(), bn, rtol=1e-3, atol=1e-4)


def test_softmax_ops_and_the_rewrites_that_produce_them():
    """Softmax / SoftmaxGrad / LogSoftmax nodes (evaluated by the oracle with the
    reference's perform formulas, theano/tensor/nnet/nnet.py:316-323, 440-444, 628-633)
    against the kernels their lowered graphs compile to; the unstabilised quotient
    exp(x) / sum(exp(x)) and log(softmax(x)) are recognised, so that rows holding large
    values stay finite (softmax_simplifier :888-925, local_logsoftmax :749-769)."""
    from theano_amd.hip import HipRowChain
    N = T.nnet
    rng = np.random.default_rng(43)
    x, y = T.fmatrix("x"), T.fmatrix("y")
    xv = (3 * rng.standard_normal((257, 1000))).astype("float32")
    xv[0, 5] = 300.0                                 # exp overflows in float32
    yv = rng.uniform(0, 1, (257, 1000)).astype("float32")
    sm = N.softmax(x)
    cost = -T.sum(T.log(sm) * y)
    outs = [sm, N.softmax_graph(x), T.log(sm), th.grad(cost, x), N.softmax_grad(y, sm), th.Rop(sm, x, y)]
    f = th.function([x, y], outs)
    kernels = [n for n in f.toposort() if type(n.op).__name__.startswith("Hip") and
               type(n.op).__name__ not in ("HipDimShuffle", "HipToHost")]
    assert len(kernels) == 1 and isinstance(kernels[0].op, HipRowChain), kernels
    got = f(xv, yv)
    ref_outs = [sm, sm, N.logsoftmax(x), th.grad(-T.sum(N.logsoftmax(x) * y), x), N.softmax_grad(y, sm),
                N.softmax_grad(y, sm)]
    ref = G.evaluate([x, y], ref_outs, [xv, yv])
    truth = G.evaluate([x, y], ref_outs, [xv, yv], wide=True)
    for k, (g, r, w) in enumerate(zip(got, ref, truth)):
        assert np.isfinite(g).all(), k
        assert_within_reference_error(g, r, w, "softmax output %d" % k)


def test_rows_too_long_for_one_block_and_strided_rows_take_the_fused_multi_kernel_path():
    """Softmax, log-softmax and their gradients on long rows and on a transposed operand.  Rows of 50 000
    float32 elements fit the registers of one block of 1024 threads; rows of 100 000 stay on chip in the
    held form (registers plus LDS, per-element values recomputed in every pass over them); rows of 250 000
    are beyond one compute unit, and the row-chain node then runs its island as reductions with fused
    prologues / epilogues - 3 launches for a softmax - with the same results."""
    from theano_amd import hip
    from theano_amd.hip import HipRowChain
    rng = np.random.default_rng(43)
    x, y = T.fmatrix("x"), T.fmatrix("y")
    sm = T.nnet.softmax(x)
    outs = [sm, T.nnet.logsoftmax(x), th.grad(T.sum(sm * y), x)]
    f = th.function([x, y], outs)
    chains = [n for n in f.toposort() if isinstance(n.op, HipRowChain)]
    assert chains
    for cols, form in ((50000, "|rw|"), (100000, "|rh|"), (250000, None)):
        xv = (3 * rng.standard_normal((6, cols))).astype("float32")
        ev = np.exp(xv.astype("float64") - xv.max(axis=1, keepdims=True))
        one = th.function([x], sm)
        assert_parity(one(xv), (ev / ev.sum(axis=1, keepdims=True)).astype("float32"), "softmax of %d columns" % cols)
        (chain,) = [n for n in one.toposort() if isinstance(n.op, HipRowChain)]
        assert (getattr(chain.op, "_fallback_function", None) is None) == (form is not None)
        if form:
            assert form in hip.last_plan(), (cols, hip.last_plan())
    yv = rng.uniform(0, 1, xv.shape).astype("float32")
    got = f(xv, yv)
    ref = G.evaluate([x, y], outs, [xv, yv])
    truth = G.evaluate([x, y], outs, [xv, yv], wide=True)
    # Softmax.perform and SoftmaxGrad.perform add a row's 250 000 float32 terms one by one in float32
    # (nnet.py:321, 443); the device accumulates in double like the ops'
    # C code (nnet.py:396): held to the float64 value, no farther from it than the oracle is
    for k, (g, r, w) in enumerate(zip(got, ref, truth)):
        assert_within_reference_error(g, r, w, "long rows, output %d" % k)
    assert np.allclose(got[0].sum(axis=1), 1.0, atol=1e-5)
    plans = [n.op._fallback_function for n in chains if getattr(n.op, "_fallback_function", None) is not None]
    assert plans, "the one-kernel form was not expected to take these rows"
    # the softmax alone: row max, sum of exp (prologue-fused), normalise
    g = th.function([x], sm)
    g(xv)
    (chain,) = [n for n in g.toposort() if isinstance(n.op, HipRowChain)]
    kinds = [type(n.op).__name__ for n in chain.op._fallback_function.toposort() if type(n.op).__name__ != "HipDimShuffle"]
    assert sorted(kinds) == ["HipCAReduce", "HipCAReduce", "HipElemwise"], kinds
    # softmax and log-softmax of rows of 100 000 in one held chain
    xh = (3 * rng.standard_normal((6, 100000))).astype("float32")
    outs2 = [sm, T.nnet.logsoftmax(x)]
    f2 = th.function([x], outs2)
    got = f2(xh)
    assert "|rh|" in hip.last_plan()
    ref = G.evaluate([x], outs2, [xh])
    truth = G.evaluate([x], outs2, [xh], wide=True)
    for k, (g_, r, w) in enumerate(zip(got, ref, truth)):
        assert_within_reference_error(g_, r, w, "held rows, output %d" % k)
    # rows that are not contiguous: the same function on a transposed view
    z = T.fmatrix("z")
    h = th.function([z], T.nnet.softmax(z.T))
    zv = (2 * rng.standard_normal((700, 90))).astype("float32")
    e = np.exp(zv.T.astype("float64") - zv.T.max(axis=1, keepdims=True))
    assert_parity(h(zv), (e / e.sum(axis=1, keepdims=True)).astype("float32"), "softmax of a transposed view")


def test_elemwise_time_test_script_runs():
    """The timing script for the reference's own on-path benchmark (theano/misc/elemwise_time_test.py:
    2*x + x*x and tanh(x) over 200 000 floats) runs and reports sane call times."""
    from theano_amd.misc.elemwise_time_test import elemwise_op_time
    host, device = elemwise_op_time(N=200000, loops=30)
    for t in host + device:
        assert 1e-6 < t < 5e-2
    assert device[0] < host[0] and device[1] < host[1]      # no upload / download on the device-resident call


@pytest.mark.parametrize("dtype", ["float32", "float16", "float64"])
def test_row_chains_over_rows_that_are_no_whole_number_of_vectors(dtype):
    """Softmax over 1001 or 50257 classes: the row chain keeps full-width vectors (plans marked `|ua`), the last one
    of a row moved back so that it ends with the row; the elements it repeats are left out of the row's sums and
    maxima.  Rows of small integers make every sum exact, so a repeated or a missed element would show in the last
    digit; the softmax values are those of the reference's formula (theano/tensor/nnet/nnet.py:440-446)."""
    rng = np.random.default_rng(17)
    tol = {"float16": {"rtol": 2e-3, "atol": 2e-3}}.get(dtype)
    mat = T.TensorType(dtype, (False, False))
    x, g = mat("x"), mat("g")
    marked = 0
    for cols in (1001, 1023, 777, 4097, 50257, 9, 13, 33, 1000, 131):
        rows = 37 if cols < 5000 else 5
        xv = rng.integers(-3, 4, (rows, cols)).astype(dtype)
        gv = rng.integers(-2, 3, (rows, cols)).astype(dtype)
        sm = T.nnet.softmax(x)
        outs = [x - T.sum(x, axis=1, keepdims=True), T.max(x * g, axis=1, keepdims=True) + x, sm, th.grad(T.sum(sm * g), x)]
        f = th.function([x, g], outs)
        got = f(xv, gv)
        marked += "|ua" in hip.last_plan()
        ref = G.evaluate([x, g], outs, [xv, gv])
        truth = None
        for k, (a, r) in enumerate(zip(got, ref)):
            what = "%d columns %s output %d [%s]" % (cols, dtype, k, hip.last_plan())
            if k < 2 and dtype != "float16":
                assert np.array_equal(a, r), what
            elif k < 3:
                assert_parity(a, r, what, tol=tol)
            else:
                if truth is None:
                    truth = G.evaluate([x, g], outs, [xv, gv], wide=True)
                assert_within_reference_error(a, r, truth[k], what, tol=tol)
    assert marked >= 6, marked
    # rows of a view whose pitch is odd and that starts one element in
    base = rng.integers(-3, 4, (64, 1031)).astype(dtype)
    out = T.nnet.softmax(x[:, 1:1025])
    got = th.function([x], out)(base)
    assert_parity(got, G.evaluate([x], [out], [base])[0], "softmax of a shifted view %s [%s]" % (dtype, hip.last_plan()), tol=tol)
