"""The five benchmark configurations as graph builders and seeded input
generators, shared by ``bench.py``, the GPU parity tests and ``smoke()``.

Every builder returns ``(inputs, outputs)`` of theano_amd variables; every
generator returns the NumPy inputs for a given scale.  ``scale='full'`` gives the
shapes the metric is quoted on, ``scale='small'`` shapes with the same strides,
broadcast patterns and dtypes that a CPU check finishes in seconds.
"""
import numpy as np

import theano_amd as th
from theano_amd import tensor as T

SEED = {"c1": 1001, "c2": 1002, "c2e": 1012, "c3": 1003, "c4": 1004, "c5": 1005}


# ---- config 1: fused Composite elementwise ----------------------------------
def c1_graph():
    x = T.fmatrix("x")
    a = T.TensorType("float32", (True, True))("a")
    b = T.TensorType("float32", (True, True))("b")
    return [x, a, b], [T.sigmoid(a * x + b) * x]


def c1_inputs(scale="full"):
    n = 4096 if scale == "full" else 250
    rng = np.random.default_rng(SEED["c1"])
    x = rng.standard_normal((n, n)).astype("float32")
    a = rng.uniform(-2, 2, (1, 1)).astype("float32")
    b = rng.uniform(-2, 2, (1, 1)).astype("float32")
    return [x, a, b]


# ---- config 2: CAReduce on a float32 matrix ---------------------------------
C2_CASES = ("sum_axis1", "max_axis1", "sum_axis0", "sum_all", "prod_axis1")


def c2_graph(case):
    x = T.fmatrix("x")
    out = {"sum_axis1": lambda: x.sum(axis=1), "max_axis1": lambda: x.max(axis=1), "sum_axis0": lambda: x.sum(axis=0),
           "sum_all": lambda: x.sum(), "prod_axis1": lambda: x.prod(axis=1)}[case]()
    return [x], [out]


def c2_argmax_graph(axis):
    """max_and_argmax of the configuration-2 matrix: the caller-side form of max."""
    x = T.fmatrix("x")
    return [x], T.max_and_argmax(x, axis=axis)


def c2_inputs(case, scale="full"):
    n = 8192 if scale == "full" else 384
    if case == "prod_axis1":
        rng = np.random.default_rng(SEED["c2e"])
        return [rng.uniform(0.9, 1.1, (n, n)).astype("float32")]
    rng = np.random.default_rng(SEED["c2"])
    return [rng.standard_normal((n, n)).astype("float32")]


# ---- config 3: row softmax and its gradient ----------------------------------
def c3_graph(with_grad=True, forward=True):
    x, y = T.fmatrix("x"), T.fmatrix("y")
    e = T.exp(x - T.max(x, axis=1, keepdims=True))
    out = e / T.sum(e, axis=1, keepdims=True)
    if not with_grad:
        return [x], [out]
    dx = th.grad(T.sum(out * y), x)
    return [x, y], ([out, dx] if forward else [dx])


def c3_inputs(scale="full", with_grad=True):
    rows, cols = (32768, 1024) if scale == "full" else (96, 1024)
    rng = np.random.default_rng(SEED["c3"])
    x = (3.0 * rng.standard_normal((rows, cols))).astype("float32")
    if not with_grad:
        return [x]
    y = rng.uniform(0, 1, (rows, cols)).astype("float32")
    return [x, y]


# ---- config 4: integer / boolean path through a dimshuffled view ---------------
def c4_graph(part="all"):
    a, b = T.itensor4("a"), T.itensor4("b")
    bias = T.TensorType("int32", (True, False, True, True))("bias")
    av, bv, biasv = a.dimshuffle(0, 2, 3, 1), b.dimshuffle(0, 2, 3, 1), bias.dimshuffle(0, 2, 3, 1)
    r = ((av & bv) ^ (av >> 3)) % 97 + biasv
    s = T.sum(r, axis=(0, 1, 2), dtype="int64")
    pos = a > 0
    outs = {"elemwise": [r], "sum": [r, s], "anyall": [T.any(pos), T.all(pos)],
            "all": [r, s, T.any(pos), T.all(pos)]}[part]
    ins = [a] if part == "anyall" else [a, b, bias]
    return ins, outs


def c4_inputs(scale="full", part="all"):
    shape = (64, 128, 56, 56) if scale == "full" else (3, 128, 7, 9)
    rng = np.random.default_rng(SEED["c4"])
    a = rng.integers(-2 ** 20, 2 ** 20, shape).astype("int32")
    b = rng.integers(-2 ** 20, 2 ** 20, shape).astype("int32")
    bias = rng.integers(-2 ** 20, 2 ** 20, (1, shape[1], 1, 1)).astype("int32")
    return [a] if part == "anyall" else [a, b, bias]


# ---- config 5: batch-norm style training graph, float16 storage ----------------
def c5_graph(with_grad=True, forward=True):
    h4 = T.TensorType("float16", (False,) * 4)
    pc = T.TensorType("float16", (True, False, True, True))
    x, g = h4("x"), h4("g")
    gamma, beta = pc("gamma"), pc("beta")
    xf = T.cast(x, "float32")
    mean = T.mean(xf, axis=(0, 2, 3), keepdims=True, acc_dtype="float32")
    var = T.mean(T.sqr(xf - mean), axis=(0, 2, 3), keepdims=True, acc_dtype="float32")
    yf = T.cast(gamma, "float32") * (xf - mean) / T.sqrt(var + np.float32(1e-5)) + T.cast(beta, "float32")
    y = T.cast(yf, "float16")
    if not with_grad:
        return [x, gamma, beta], [y]
    cost = T.sum(T.cast(y, "float32") * T.cast(g, "float32"))
    dx, dgamma, dbeta = th.grad(cost, [x, gamma, beta])
    grads = [T.cast(dx, "float16"), T.cast(dgamma, "float16"), T.cast(dbeta, "float16")]
    return [x, gamma, beta, g], ([y] + grads if forward else grads)


def c5_inputs(scale="full", with_grad=True):
    shape = (256, 256, 28, 28) if scale == "full" else (6, 16, 7, 8)
    rng = np.random.default_rng(SEED["c5"])
    x = rng.normal(0.5, 2.0, shape).astype("float16")
    gamma = rng.normal(1.0, 0.1, (1, shape[1], 1, 1)).astype("float16")
    beta = rng.normal(0.0, 0.1, (1, shape[1], 1, 1)).astype("float16")
    if not with_grad:
        return [x, gamma, beta]
    g = rng.standard_normal(shape).astype("float16")
    return [x, gamma, beta, g]


# ---- algorithmic bytes: every input read once per required pass, every output written once ----
def algorithmic_bytes(name, scale="full"):
    f4, i4, f2 = 4, 4, 2
    if name == "c1":
        n = 4096 if scale == "full" else 250
        return 2 * n * n * f4 + 8
    if name.startswith("c2_argmax"):  # max (float32) and argmax (int64) per kept index
        n = 8192 if scale == "full" else 384
        return n * n * f4 + n * (f4 + 8)
    if name.startswith("c2"):
        n = 8192 if scale == "full" else 384
        return n * n * f4 + (4 if name == "c2_sum_all" else n * f4)
    if name == "c3_fwd":
        r, c = (32768, 1024) if scale == "full" else (96, 1024)
        return 2 * r * c * f4
    if name == "c3_grad":
        r, c = (32768, 1024) if scale == "full" else (96, 1024)
        return 3 * r * c * f4
    if name == "c3_fwd_grad":
        r, c = (32768, 1024) if scale == "full" else (96, 1024)
        return 4 * r * c * f4
    shape4 = (64, 128, 56, 56) if scale == "full" else (3, 128, 7, 9)
    n4 = int(np.prod(shape4))
    if name == "c4_elemwise":
        return 3 * n4 * i4 + shape4[1] * i4
    if name == "c4_sum":  # elementwise result written, its per-channel int64 sum alongside
        return 3 * n4 * i4 + shape4[1] * i4 + shape4[1] * 8
    if name == "c4_anyall":
        return n4 * i4 + 2
    shape5 = (256, 256, 28, 28) if scale == "full" else (6, 16, 7, 8)
    n5 = int(np.prod(shape5))
    if name == "c5_fwd":  # one statistics read of x, then read x and write y (a two-pass variance reads x once more)
        return 3 * n5 * f2
    if name == "c5_grad":  # pass 1 reads x, g; pass 2 reads x, g and writes dx
        return 5 * n5 * f2
    raise KeyError(name)
