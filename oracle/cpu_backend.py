"""TEST INFRASTRUCTURE - not part of the product.  Only ``tests/`` and the
``cpu_baseline`` leg of ``bench.py`` may import this.

ctypes front end of ``oracle/cpu_backend.c``: the host loops Theano's C backend
runs for benchmark configurations 1, 3, 4 and 5, forward and gradient (OpenMP Elemwise nodes above
200000 elements, serial CAReduce nodes, intermediates materialised between
nodes; ``theano/tensor/elemwise.py:1100-1102``,
``theano/tensor/elemwise_cgen.py:406-409, 465-527``).  ``run(name, inputs)``
returns the outputs and the seconds spent inside the C call.

Pinned by tests/test_oracle_graph.py::test_cpu_backend_matches_graph_oracle
against the node-by-node NumPy evaluation of the same graphs.
"""
import ctypes
import time

import numpy as np

from . import graph_ref


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _i64(v):
    return ctypes.c_int64(int(v))


def c2_parallel(x, which):
    """(result, seconds) of one reduction of configuration 2 with OpenMP over the outputs:
    NOT what the reference does (its CAReduce loops are serial); reported for context only.
    ``which``: sum_axis1, max_axis1, sum_axis0, sum_all, prod_axis1."""
    L = graph_ref.lib()
    x = np.ascontiguousarray(x, "float32")
    R, C = x.shape
    code = ["sum_axis1", "max_axis1", "sum_axis0", "sum_all", "prod_axis1"].index(which)
    out = np.empty({2: C, 3: 1}.get(code, R), "float32")
    t0 = time.perf_counter()
    L.cpu_c2_parallel(_p(x), _p(out), _i64(R), _i64(C), ctypes.c_int(code))
    dt = time.perf_counter() - t0
    return (out.reshape(()) if code == 3 else out), dt


def run(name, inputs):
    """(outputs, seconds) of one configuration's CPU loops.  ``inputs`` are
    the C-contiguous NumPy arrays of ``workloads.<config>_inputs``."""
    L = graph_ref.lib()
    inputs = [np.ascontiguousarray(v) for v in inputs]
    if name == "c1":
        x, a, b = inputs
        out = np.empty_like(x)
        t0 = time.perf_counter()
        L.cpu_c1(_p(x), _p(a), _p(b), _p(out), _i64(x.size))
        return [out], time.perf_counter() - t0
    if name in ("c3_fwd", "c3_fwd_rowloop"):
        x = inputs[0]
        R, C = x.shape
        out = np.empty_like(x)
        if name == "c3_fwd":
            e, rowmax, rowsum = np.empty_like(x), np.empty(R, "float32"), np.empty(R, "float32")
            t0 = time.perf_counter()
            L.cpu_c3_chain(_p(x), _p(out), _p(e), _p(rowmax), _p(rowsum), _i64(R), _i64(C))
        else:
            t0 = time.perf_counter()
            L.cpu_c3_rowloop(_p(x), _p(out), _i64(R), _i64(C))
        return [out], time.perf_counter() - t0
    if name == "c3_fwd_grad":
        x, y = inputs
        R, C = x.shape
        out, dx = np.empty_like(x), np.empty_like(x)
        e, t, u = np.empty_like(x), np.empty_like(x), np.empty_like(x)
        rows = [np.empty(R, "float32") for _ in range(4)]
        t0 = time.perf_counter()
        L.cpu_c3_fwd_grad(_p(x), _p(y), _p(out), _p(dx), _p(e), _p(t), _p(u), _p(rows[0]), _p(rows[1]), _p(rows[2]),
                          _p(rows[3]), _i64(R), _i64(C))
        return [out, dx], time.perf_counter() - t0
    if name == "c5_grad":
        x, gamma, beta, g = inputs
        N, Ch, H, Wd = x.shape
        dx = np.empty_like(x)
        dgamma, dbeta = np.empty_like(gamma), np.empty_like(beta)
        xf, gf, d = [np.empty(x.shape, "float32") for _ in range(3)]
        mean, var, tmp = [np.empty(Ch, "float32") for _ in range(3)]
        t0 = time.perf_counter()
        L.cpu_c5_grad(_p(x), _p(gamma), _p(g), _p(dx), _p(dgamma), _p(dbeta), _p(xf), _p(gf), _p(d), _p(mean), _p(var),
                      _p(tmp), _i64(N), _i64(Ch), _i64(H * Wd))
        return [dx, dgamma, dbeta], time.perf_counter() - t0
    if name in ("c4_elemwise", "c4_sum"):
        a, b, bias = inputs
        N, Ch, H, Wd = a.shape
        r = np.empty((N, H, Wd, Ch), "int32")
        s = np.empty(Ch, "int64")
        t0 = time.perf_counter()
        L.cpu_c4_elemwise(_p(a), _p(b), _p(bias), _p(r), _i64(N), _i64(Ch), _i64(H), _i64(Wd))
        if name == "c4_sum":
            L.cpu_c4_sum(_p(r), _p(s), _i64(N * H * Wd), _i64(Ch))
        dt = time.perf_counter() - t0
        return ([r, s] if name == "c4_sum" else [r]), dt
    if name == "c4_anyall":
        a = inputs[0]
        pos = np.empty(a.shape, "bool")
        res = np.empty(2, "bool")
        t0 = time.perf_counter()
        L.cpu_c4_anyall(_p(a), _p(pos), _p(res[0:1]), _p(res[1:2]), _i64(a.size))
        return [res[0].copy().reshape(()), res[1].copy().reshape(())], time.perf_counter() - t0
    if name == "c5_fwd":
        x, gamma, beta = inputs
        N, Ch, H, Wd = x.shape
        y = np.empty_like(x)
        xf, d = np.empty(x.shape, "float32"), np.empty(x.shape, "float32")
        mean, var = np.empty(Ch, "float32"), np.empty(Ch, "float32")
        t0 = time.perf_counter()
        L.cpu_c5_fwd(_p(x), _p(gamma), _p(beta), _p(y), _p(xf), _p(d), _p(mean), _p(var), _i64(N), _i64(Ch),
                     _i64(H * Wd))
        return [y], time.perf_counter() - t0
    raise KeyError(name)
