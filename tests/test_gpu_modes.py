"""The debugging modes of ``function``: ``mode='check'`` (the in-place / aliasing checks of DebugMode,
theano/compile/debugmode.py BadDestroyMap / BadOptimization, done by running the graph again one kernel per
node) and ``mode='nan_guard'`` (NanGuardMode, theano/compile/nanguardmode.py)."""
import numpy as np
import pytest

import theano_amd as th
from theano_amd import hip, scalar as scal, tensor as T
from theano_amd.hip import HipArray
from theano_amd.tensor.elemwise import Elemwise

pytestmark = pytest.mark.gpu


def test_check_mode_passes_correct_functions_and_returns_their_results():
    rng = np.random.default_rng(61)
    x, y = T.fmatrix("x"), T.fmatrix("y")
    e = T.exp(x - T.max(x, axis=1, keepdims=True))
    sm = e / T.sum(e, axis=1, keepdims=True)
    outs = [sm, th.grad(T.sum(sm * y), x), T.sum(x * y, axis=0), T.argmax(x, axis=1), (x > y).sum()]
    xv, yv = rng.standard_normal((64, 300)).astype("float32"), rng.standard_normal((64, 300)).astype("float32")
    plain = th.function([x, y], outs)(xv, yv)
    f = th.function([x, y], outs, mode="check")
    assert isinstance(f, th.compile.CheckedFunction) and len(f.toposort()) < len(f.reference.toposort())
    for a, b in zip(f(xv, yv), plain):
        assert np.array_equal(a, b, equal_nan=True)
    for a, b in zip(f(HipArray.from_numpy(xv), HipArray.from_numpy(yv)), plain):      # device arguments
        assert np.array_equal(a, b, equal_nan=True)
    # shared variables with updates: the new values are compared too and applied once
    w = th.shared(np.ones((300,), "float32"), name="w")
    step = th.function([x], T.sum(x * w), updates=[(w, w * np.float32(0.5) + T.mean(x, axis=0))], mode="check")
    step(xv)
    assert np.allclose(w.get_value(), 0.5 + xv.mean(axis=0), rtol=1e-5, atol=1e-6)
    step(xv)
    assert np.allclose(w.get_value(), 0.5 * (0.5 + xv.mean(axis=0)) + xv.mean(axis=0), rtol=1e-5, atol=1e-6)
    h = T.TensorType("float16", (False, False))("h")                                     # float16: the wide tolerance
    th.function([h], [T.tanh(h * 3 + 1) * h, T.sum(h * h, axis=1)], mode="check")(xv.astype("float16"))


def test_check_mode_reports_an_overwritten_argument(monkeypatch):
    """A deliberately wrong in-place pass (it lets a kernel write over a function argument, which the real
    pass never does): harmless for a host argument, which is uploaded into a private buffer, but a device
    array handed in by the caller comes back changed."""
    from theano_amd.hip import opt as hip_opt
    rng = np.random.default_rng(62)
    x, y = T.fmatrix("x"), T.fmatrix("y")
    real = hip_opt.inplace_elemwise

    def broken(fgraph, *a, **k):
        out = real(fgraph, *a, **k)
        for node in fgraph.toposort():
            if isinstance(node.op, hip.HipElemwise) and not node.op.inplace_pattern and len(node.outputs) == 1:
                new = hip.HipElemwise(node.op.scalar_op, {0: 0}).make_node(*node.inputs).outputs[0]
                fgraph.replace(node.outputs[0], new)
        return out

    monkeypatch.setattr(hip_opt, "inplace_elemwise", broken)
    xv, yv = rng.standard_normal((33, 50)).astype("float32"), rng.standard_normal((33, 50)).astype("float32")
    f = th.function([x, y], (x + y) * 2, mode="check")
    assert np.allclose(f(xv, yv), (xv + yv) * 2)
    with pytest.raises(th.CheckModeError, match="argument 0"):
        f(HipArray.from_numpy(xv), HipArray.from_numpy(yv))


def test_check_mode_reports_results_that_depend_on_the_rewrites(monkeypatch):
    """A deliberately wrong rewrite (an elementwise fusion that drops a term) is caught by the comparison."""
    from theano_amd.hip import opt as hip_opt
    x = T.fmatrix("x")
    real = hip_opt.fuse_elemwise

    def broken(fgraph, *a, **k):
        out = real(fgraph, *a, **k)
        for node in fgraph.toposort():
            if isinstance(node.op, hip.HipElemwise) and "exp" in str(node.op):
                fgraph.replace(node.outputs[0], hip.HipElemwise(scal.sqr).make_node(node.inputs[0]).outputs[0])
        return out

    monkeypatch.setattr(hip_opt, "fuse_elemwise", broken)
    f = th.function([x], T.exp(x) + 1, mode="check")
    with pytest.raises(th.CheckModeError, match="output 0 differs"):
        f(np.full((4, 5), 2.0, "float32"))


def test_nan_guard_names_the_node():
    x = T.fmatrix("x")
    f = th.function([x], [T.log(x) * 2, T.sum(x, axis=0)], mode="nan_guard")
    ok = np.full((6, 7), 2.0, "float32")
    assert np.allclose(f(ok)[0], np.log(2.0) * 2)
    bad = ok.copy()
    bad[2, 3] = -1.0
    with pytest.raises(th.NanGuardError, match="NaN in output 0 of .*log"):
        f(bad)
    bad[2, 3] = 0.0
    with pytest.raises(th.NanGuardError, match="Inf"):
        f(bad)
    g = th.function([x], T.sum(x, axis=0))          # without the mode the same values pass through
    assert np.isnan(g(np.full((2, 2), np.nan, "float32"))).all()
    with pytest.raises(ValueError):
        th.function([x], x + 1, mode="fast")
