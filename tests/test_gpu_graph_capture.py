"""Recorded launch sequences (HIP graphs): a captured function replays to the results of its eager calls,
replay after replay, with other work of the library and synchronisations in between."""
import numpy as np
import pytest

import theano_amd as th
from theano_amd import hip, tensor as T
from theano_amd.compile import Out
from theano_amd.hip.runtime import HipArray
from theano_amd.hip.views import copy_into

pytestmark = pytest.mark.gpu


def _device_outs(outs):
    return [Out(o, device=True) for o in outs]


def test_replays_match_eager_calls_with_other_work_in_between():
    rng = np.random.default_rng(3)
    x, y = T.fmatrix("x"), T.fmatrix("y")
    e = T.exp(x - T.max(x, axis=1, keepdims=True))
    sm = e / T.sum(e, axis=1, keepdims=True)
    outs = [sm, T.sum(x * y), T.sum(x, axis=0), T.argmax(x * y, axis=1), T.any(x > 3.5), T.all(abs(y) < 10.0),
            T.sum(T.sqr(x) * y, axis=1) / T.sqrt(T.sum(T.sqr(y), axis=1) + 1.0)]
    shape = (3000, 1200)                                  # large enough for split reductions and their second launches
    for flags in ({}, {"rowchain": False}, {"fuse": False}):
        f = th.function([x, y], _device_outs(outs), **flags)
        eager = th.function([x, y], _device_outs(outs), **flags)
        assert len([n for n in f.toposort()]) >= 4
        xd = HipArray.from_numpy(rng.standard_normal(shape).astype("float32"))
        yd = HipArray.from_numpy(rng.standard_normal(shape).astype("float32"))
        results, graph = f.capture(xd, yd)
        other = th.function([x], Out(T.tanh(x) * 2 + T.sum(x), device=True))
        for replay in range(4):
            # new contents in the same argument arrays, unrelated work and a synchronisation between replays
            copy_into(HipArray.from_numpy(rng.standard_normal(shape).astype("float32") * (replay + 1)), xd)
            copy_into(HipArray.from_numpy(rng.standard_normal(shape).astype("float32")), yd)
            other(yd).to_numpy()
            graph.launch()
            got = [r.to_numpy() for r in results]
            want = [r.to_numpy() for r in eager(xd, yd)]
            for k, (g, w) in enumerate(zip(got, want)):
                assert g.dtype == w.dtype and np.array_equal(g, w, equal_nan=True), (flags, replay, k)
        del graph


def test_what_cannot_be_captured_is_refused():
    x = T.fmatrix("x")
    xd = HipArray.from_numpy(np.ones((4, 5), "float32"))
    with pytest.raises(TypeError, match="device results"):
        th.function([x], x + 1).capture(xd)
    f = th.function([x], Out(x + 1, device=True))
    with pytest.raises(TypeError, match="device array"):
        f.capture(np.ones((4, 5), "float32"))
    w = th.shared(np.ones((4, 5), "float32"))
    with pytest.raises(ValueError, match="updates"):
        th.function([x], Out(x + w, device=True), updates=[(w, w + x)]).capture(xd)
    # a capture left by an exception records nothing and leaves the library usable
    with pytest.raises(RuntimeError, match="stop"):
        with hip.capture():
            f(xd)
            raise RuntimeError("stop")
    assert np.array_equal(f(xd).to_numpy(), np.full((4, 5), 2, "float32"))
    with pytest.raises(ValueError, match="no capture is open"):
        hip.runtime.check(hip.runtime.lib.thx_capture_end(None))          # none open
