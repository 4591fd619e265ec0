"""The 72 rows of the reference's elementwise-fusion test as data
(tests/golden/fusion_table.json, transcribed from theano/tensor/tests/test_opt.py:937-1112):
result dtype, value against the row's NumPy answer (oracle on the CPU, HIP path on the
GPU), and never more elementwise kernels than the reference's fused graph has Elemwise
nodes."""
import json
import os

import numpy as np
import pytest

import theano_amd as th
from theano_amd import tensor as T
from theano_amd.hip import HipElemwise
from oracle import graph_ref as G
from conftest import TOL

HERE = os.path.dirname(os.path.abspath(__file__))
ROWS = json.load(open(os.path.join(HERE, "golden", "fusion_table.json")))
SHAPE = (5, 5)


def build(row):
    def var(dtype, name):
        return T.TensorType(dtype, (False,) * len(SHAPE))(name)
    sym = {"fw": var("float32", "w"), "fx": var("float32", "x"), "fy": var("float32", "y"), "fz": var("float32", "z"),
           "dw": var("float64", "w"), "ix": var("int32", "x"), "iy": var("int32", "y"), "iz": var("int32", "z"),
           "fv": T.fvector("v"), "fs": T.fscalar("s")}
    rng = np.random.default_rng(100 + row["row"])
    filled = lambda dt, num: np.zeros(SHAPE, dtype=dt) + np.asarray(num, dt)       # noqa: E731
    val = {"fwv": filled("float32", 1), "fxv": filled("float32", 2), "fyv": filled("float32", 3),
           "fzv": filled("float32", 4), "dwv": filled("float64", 5), "ixv": filled("int32", 60),
           "iyv": filled("int32", 70), "izv": filled("int32", 70),
           "fvv": rng.random(SHAPE[0]).astype("float32"), "fsv": np.asarray(rng.random(), "float32")}
    out = eval(row["expr"], {"T": T, "abs": abs}, dict(sym))
    ins = [sym[n] for n in row["inputs"]]
    vals = [val[n + "v"] for n in row["inputs"]]
    with np.errstate(all="ignore"):
        want = eval(row["numpy"], {"np": np}, dict(val))
    return ins, out, vals, np.asarray(want)


def check(row, got, want):
    assert got.dtype == np.dtype(row["dtype"]), (row["row"], got.dtype)
    assert got.shape == np.broadcast_shapes(want.shape, got.shape)
    if got.dtype.kind in "iu":
        assert np.array_equal(got, want.astype(got.dtype)), row["row"]
    else:
        assert np.allclose(got, want, **TOL["float32"]), (row["row"], got.ravel()[:3], want.ravel()[:3])


@pytest.mark.parametrize("row", ROWS, ids=[str(r["row"]) for r in ROWS])
def test_oracle_gives_the_reference_answers(row):
    ins, out, vals, want = build(row)
    check(row, G.evaluate(ins, [out], vals)[0], want)


def test_fused_graphs_have_no_more_elementwise_kernels_than_the_reference(dry_run):
    for row in ROWS:
        ins, out, vals, _ = build(row)
        f = th.function(ins, [out])
        n = sum(1 for node in f.toposort() if isinstance(node.op, HipElemwise))
        assert n <= row["elemwise_nodes"], (row["row"], row["expr"], [str(x) for x in f.toposort()])
        f(*vals)


@pytest.mark.gpu
@pytest.mark.parametrize("row", ROWS, ids=[str(r["row"]) for r in ROWS])
def test_hip_path_gives_the_reference_answers(row):
    ins, out, vals, want = build(row)
    check(row, th.function(ins, [out])(*vals)[0], want)


def test_fixture_matches_its_generator():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_fusion_table", os.path.join(HERE, "golden", "make_fusion_table.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert [(r["expr"], r["numpy"], r["dtype"], r["elemwise_nodes"]) for r in ROWS] == [
        (e, a, d, n) for (e, i, n, a, d) in mod.ROWS]
