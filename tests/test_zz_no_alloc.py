"""thx_reduce_call_static - the reduction entry point that never allocates device memory -
gives the results of thx_reduce_call bit for bit (the same kernels over the same slices; only the
home of the partial results differs), on calls in a row that share the fixed scratch array, and
refuses what it cannot do without allocating: a kernel that is not loaded yet, partial results
beyond the array's size."""
import ctypes

import numpy as np
import pytest

from theano_amd import scalar as scal
from theano_amd.hip import codegen, runtime
from theano_amd.hip.runtime import HipArray, check, lib, thx_array

pytestmark = pytest.mark.gpu

lib.thx_reduce_call_static.argtypes = lib.thx_reduce_call.argtypes
lib.thx_reduce_call_static.restype = ctypes.c_int
STATIC_BYTES = 4194304


def _handle(scalar_ops, acc, in_dt, out_dt, pre=None):
    src, name, acc_bytes = codegen.reduce_functor(scalar_ops, acc, in_dt, out_dt, pre)
    all_dt = tuple(in_dt) + tuple(out_dt)
    codes = (ctypes.c_int32 * len(all_dt))(*[scal.dtype_code(d) for d in all_dt])
    h = ctypes.c_void_p()
    check(lib.thx_reduce_new(src.encode(), name.encode(), len(in_dt), len(out_dt), 0, codes, acc_bytes, ctypes.byref(h)))
    return h


def _call(fn, h, x, axis, out_dtypes):
    """One call of `fn` (either entry point) reducing device array `x` over `axis`; returns (rc, results, plan)."""
    nd = x.ndim
    mask = (ctypes.c_uint8 * nd)(*[1 if d in axis else 0 for d in range(nd)])
    kept = tuple(s for d, s in enumerate(x.shape) if d not in axis)
    ins = (thx_array * 1)()
    x.as_thx(ins[0])
    outs = (thx_array * len(out_dtypes))()
    res = []
    for k, dt in enumerate(out_dtypes):
        o = HipArray.from_numpy(np.full(kept, -7, dt))    # a sentinel: a refused call must leave it alone
        o.as_thx(outs[k])
        res.append(o)
    rc = fn(h, ins, mask, outs, runtime.THX_BROADCAST)
    plan = runtime.last_plan()
    runtime.sync()
    return rc, [r.to_numpy() for r in res], plan


CASES = [
    # (big shape, small shape, axis): every call is a split reduction (partial results in scratch memory)
    ((2048, 4096), (700, 1024), (0, 1)),      # all axes: row form, one result, hundreds of slices
    ((4096, 512), (1500, 256), (0,)),         # axis 0: column form, row slices
    ((64, 16, 4096), (24, 16, 1024), (0, 2)),    # per-channel sums: row form with two reduced dimensions
]


@pytest.mark.parametrize("big,small,axis", CASES)
def test_static_scratch_matches_allocated_scratch(big, small, axis):
    runtime.init()
    rng = np.random.default_rng(77)
    h = _handle((scal.add,), ("float64",), ("float32",), ("float32",))
    xb = HipArray.from_numpy(rng.standard_normal(big).astype("float32"))
    xs = HipArray.from_numpy(rng.standard_normal(small).astype("float32"))
    # before any warm-up the kernels are not loaded: refused, nothing launched, outputs untouched
    rc, res, _ = _call(lib.thx_reduce_call_static, h, xb, axis, ["float32"])
    assert rc == 6 and b"not loaded" in lib.thx_last_error(), lib.thx_last_error()
    assert np.all(res[0] == -7)
    # the existing entry point: results to compare with, and the warm-up that loads the kernels
    rc, ref_b, plan_b = _call(lib.thx_reduce_call, h, xb, axis, ["float32"])
    check(rc)
    rc, ref_s, plan_s = _call(lib.thx_reduce_call, h, xs, axis, ["float32"])
    check(rc)
    assert "|s" in plan_b.split("|m")[-1] and "|s" in plan_s.split("|m")[-1], (plan_b, plan_s)   # both are split
    # two calls in a row on the fixed scratch array, the second smaller (fewer results and slices:
    # it must not see anything the first one left behind)
    rc, got_b, plan = _call(lib.thx_reduce_call_static, h, xb, axis, ["float32"])
    check(rc)
    assert plan == plan_b
    rc, got_s, plan = _call(lib.thx_reduce_call_static, h, xs, axis, ["float32"])
    check(rc)
    assert plan == plan_s
    assert np.array_equal(got_b[0], ref_b[0]) and np.array_equal(got_s[0], ref_s[0])
    # and both agree with float64 NumPy at the float32 bar
    for got, x in ((got_b[0], xb), (got_s[0], xs)):
        want = x.to_numpy().astype("float64").sum(axis=axis).astype("float32")
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    check(lib.thx_reduce_free(h))


def test_two_accumulators_and_integers_bit_exact():
    """any + all of one int32 array (two bool accumulators, one read) and an int64 sum."""
    runtime.init()
    rng = np.random.default_rng(78)
    i = scal.Scalar("int32")()
    pre = scal.Composite([i], [scal.gt(i, scal.ScalarConstant(scal.Scalar("int32"), np.int32(0))),
                               scal.gt(i, scal.ScalarConstant(scal.Scalar("int32"), np.int32(-5)))])
    h = _handle((scal.or_, scal.and_), ("bool", "bool"), ("int32",), ("bool", "bool"), pre)
    hs = _handle((scal.add,), ("int64",), ("int32",), ("int64",))
    for shape in ((3000, 2048), (1111, 512)):
        v = rng.integers(-4, 100, shape).astype("int32")
        x = HipArray.from_numpy(v)
        for handle, odt, want in ((h, ["bool", "bool"], [np.any(v > 0), np.all(v > -5)]),
                                  (hs, ["int64"], [v.sum(dtype="int64")])):
            rc, ref, plan = _call(lib.thx_reduce_call, handle, x, (0, 1), odt)
            check(rc)
            assert "|s" in plan.split("|m")[-1]
            rc, got, _ = _call(lib.thx_reduce_call_static, handle, x, (0, 1), odt)
            check(rc)
            for g, r, w in zip(got, ref, want):
                assert np.array_equal(g, r) and g == w


def test_partial_results_beyond_the_fixed_array_are_refused(monkeypatch):
    runtime.init()
    # many more slices than the planner's default, so that slices x results x 8 bytes exceeds the array
    monkeypatch.setenv("THX_RED_BLOCKS_PER_CU", "64")
    h = _handle((scal.add,), ("float64",), ("float32",), ("float32",))
    x = HipArray.from_numpy(np.ones((16384, 8192), "float32"))
    rc, ref, plan = _call(lib.thx_reduce_call, h, x, (0,), ["float32"])
    check(rc)
    S = int(plan.rsplit("|s", 1)[1])
    assert S * 8192 * 8 > STATIC_BYTES, plan
    assert np.all(ref[0] == 16384)
    rc, res, _ = _call(lib.thx_reduce_call_static, h, x, (0,), ["float32"])
    assert rc == 6 and b"fixed scratch array" in lib.thx_last_error(), lib.thx_last_error()
    assert np.all(res[0] == -7)
    monkeypatch.delenv("THX_RED_BLOCKS_PER_CU")
    # with the default split the same reduction fits
    rc, ref, plan = _call(lib.thx_reduce_call, h, x, (0,), ["float32"])
    check(rc)
    rc, got, _ = _call(lib.thx_reduce_call_static, h, x, (0,), ["float32"])
    check(rc)
    assert np.array_equal(got[0], ref[0])
    check(lib.thx_reduce_free(h))
