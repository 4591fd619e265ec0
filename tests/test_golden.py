"""The reference's own literal test vectors (tests/golden/reference_vectors.json,
each entry citing the lines it was transcribed from): the oracle reproduces
every one on the CPU, the HIP path on the GPU."""
import json
import os

import numpy as np
import pytest

import theano_amd as th
from theano_amd import tensor as T
from oracle import graph_ref as G

HERE = os.path.dirname(os.path.abspath(__file__))
VECTORS = json.load(open(os.path.join(HERE, "golden", "reference_vectors.json")))


def build(entry):
    """(inputs, outputs, values) of the graph an entry names."""
    dt = entry["dtype"]
    data = np.asarray(entry["input"])
    g = entry["graph"]
    if g == "prod_axis1":
        x = T.TensorType(dt, (False, False))("x")
        return [x], [T.prod(x, axis=1)], [data.astype(dt)]
    if g in ("prod_without_zeros_axis1", "prod_without_zeros_axis0"):
        from theano_amd.tensor.elemwise import ProdWithoutZeros
        x = T.TensorType(dt, (False, False))("x")
        return [x], [ProdWithoutZeros(axis=int(g[-1]))(x)], [data.astype(dt)]
    if g in ("prod_grad_axis1", "prod_grad_axis0"):
        x = T.TensorType(dt, (False, False))("x")
        return [x], [th.grad(T.sum(T.prod(x, axis=int(g[-1]))), x)], [data.astype(dt)]
    if g in ("prod_all_no_zeros_grad", "prod_all_no_zeros_second_grad"):
        x = T.TensorType(dt, (False, False))("x")
        gx = th.grad(T.prod(x, no_zeros_in_input=True), x)
        return [x], [gx if g.endswith("zeros_grad") else th.grad(T.sum(gx), x)], [data.astype(dt)]
    if g == "sum_all":
        x = T.TensorType(dt, (False,))("x")
        return [x], [T.sum(x)], [data.astype(dt)]
    if g == "max_and_argmax_all":
        x = T.TensorType(dt, (False,))("x")
        return [x], T.max_and_argmax(x), [data.astype(dt)]
    if g == "max_and_argmax_axes_1_2":
        x = T.TensorType(dt, (False,) * 3)("x")
        return [x], T.max_and_argmax(x, [1, -1]), [data.astype(dt)]
    if g == "x_times_2_times_3":
        x = T.TensorType(dt, (False,))("x")
        return [x], [x * 2 * 3], [data.astype(dt)]
    if g == "add3":
        xs = [T.TensorType(dt, (False, False))(n) for n in "xyz"]
        return xs, [xs[0] + xs[1] + xs[2]], [(np.zeros((5, 5), dt) + v).astype(dt) for v in data]
    if g == "true_div_int_times_float":
        ix, iy = T.imatrix("ix"), T.imatrix("iy")
        fx = T.fmatrix("fx")
        vals = [np.zeros((5, 5), "int32") + int(data[0]), np.zeros((5, 5), "int32") + int(data[1]),
                (np.zeros((5, 5), "float32") + data[2]).astype("float32")]
        return [ix, iy, fx], [T.true_div(ix, iy) * fx], vals
    if g == "mod_intdiv_int8":
        a, b = T.TensorType(dt, (False,))("a"), T.TensorType(dt, (False,))("b")
        return [a, b], [a % b, a // b], [data[0].astype(dt), data[1].astype(dt)]
    raise KeyError(g)


def expected(entry, n_out):
    e = entry["expected"]
    return [np.asarray(v) for v in e] if n_out > 1 else [np.asarray(e)]


def check(entry, got):
    want = expected(entry, len(got))
    for g, w in zip(got, want):
        g = np.asarray(g)
        if w.ndim == 0 and g.ndim > 0:              # constant-filled matrices of the fusion table
            assert np.allclose(g, float(w), rtol=1e-6), (entry["name"], g, w)
        elif g.dtype.kind in "iub":
            assert np.array_equal(g, w), (entry["name"], g, w)
        else:
            assert np.allclose(g, w, rtol=1e-6), (entry["name"], g, w)


@pytest.mark.parametrize("entry", VECTORS, ids=[v["name"] for v in VECTORS])
def test_oracle_reproduces_reference_vectors(entry):
    ins, outs, vals = build(entry)
    check(entry, G.evaluate(ins, outs, vals))


@pytest.mark.gpu
@pytest.mark.parametrize("entry", VECTORS, ids=[v["name"] for v in VECTORS])
def test_hip_path_reproduces_reference_vectors(entry):
    ins, outs, vals = build(entry)
    check(entry, th.function(ins, outs)(*vals))


@pytest.mark.parametrize("entry", VECTORS, ids=[v["name"] for v in VECTORS])
def test_vector_graphs_compile_without_a_rewrite_cycle(entry, dry_run):
    """The graph rewriter warns when rewrites keep undoing each other; none of the
    reference's test graphs may trigger that."""
    import warnings
    ins, outs, vals = build(entry)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        got = th.function(ins, outs)(*vals)
    want = expected(entry, len(got))
    assert [np.asarray(g).shape for g in got] == [w.shape if w.ndim else np.asarray(g).shape for g, w in zip(got, want)]


def test_fixture_file_matches_its_generator():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_vectors", os.path.join(HERE, "golden", "make_vectors.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert json.loads(json.dumps(mod.VECTORS)) == VECTORS
