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


def test_chain_nodes_replay_too_held_and_turned_away():
    """Batch-normalisation graphs: a held chain (one kernel), and a chain that is turned away at run time and runs
    its island through the inner function - both record and replay to the eager results."""
    rng = np.random.default_rng(9)
    x4 = T.TensorType("float32", (False,) * 4)("x")
    g4 = T.TensorType("float32", (False,) * 4)("g")
    mean = T.mean(x4, axis=(0, 2, 3), keepdims=True)
    var = T.mean(T.sqr(x4 - mean), axis=(0, 2, 3), keepdims=True)
    y = (x4 - mean) / T.sqrt(var + np.float32(1e-5))
    dx = th.grad(T.sum(y * g4), x4)
    for shape in ((8, 12, 10, 14), (64, 4, 300, 300)):      # the second: too much per channel to hold, turned away
        f = th.function([x4, g4], _device_outs([y, dx]))
        eager = th.function([x4, g4], _device_outs([y, dx]))
        xd = HipArray.from_numpy(rng.standard_normal(shape).astype("float32"))
        gd = HipArray.from_numpy(rng.standard_normal(shape).astype("float32"))
        results, graph = f.capture(xd, gd)
        for replay in range(3):
            copy_into(HipArray.from_numpy(rng.normal(replay, 2.0, shape).astype("float32")), xd)
            hip.sync()
            graph.launch()
            got = [r.to_numpy() for r in results]
            want = [r.to_numpy() for r in eager(xd, gd)]
            for k, (a, b) in enumerate(zip(got, want)):
                assert np.array_equal(a, b), (shape, replay, k)


def test_a_recording_keeps_its_scratch_buffer_and_its_operands_alive():
    """A recorded split reduction holds the address of the partial-result buffer: when a later call needs a larger
    buffer the old one is set aside until the last recording is gone, never freed under it; growing the buffer
    inside a recording is refused.  The graph also holds the argument arrays and the shared variables' values of
    the moment, so dropping the caller's references (or a set_value) leaves replays reading live memory."""
    import gc
    from theano_amd.hip import runtime as R
    rng = np.random.default_rng(12)
    x = T.fmatrix("x")
    w = th.shared(rng.standard_normal((1, 700)).astype("float32"), broadcastable=(True, False))
    f = th.function([x], _device_outs([T.sum(x * w), T.sum(x + w, axis=0)]))     # both split into slices
    xv = rng.standard_normal((5000, 700)).astype("float32")
    wv = w.get_value()
    xd = HipArray.from_numpy(xv)
    results, graph = f.capture(xd)
    want = [r.to_numpy() for r in results]
    size0, held0, alive0 = R.scratch_state()
    assert alive0 >= 1 and size0 >= 8 << 20
    R.scratch_reserve(size0 + (4 << 20))                   # what an eager call with more partial results does
    size1, held1, alive1 = R.scratch_state()
    assert size1 >= size0 + (4 << 20) and held1 == held0 + 1 and alive1 == alive0
    del xd
    w.set_value(np.zeros((1, 700), "float32"))
    gc.collect()
    junk = [HipArray.from_numpy(np.full((5000, 700), 7, "float32")) for _ in range(3)]    # would reuse freed blocks
    graph.launch()
    got = [r.to_numpy() for r in results]
    for g, wnt in zip(got, want):
        assert np.array_equal(g, wnt)
    assert np.allclose(got[0], (xv.astype("float64") * wv).sum(), rtol=1e-6)
    with pytest.raises(ValueError, match="recording"):
        with hip.capture():
            R.scratch_reserve(size1 + (16 << 20))
    del graph, junk
    gc.collect()
    assert R.scratch_state()[1:] == (0, alive0 - 1)
