"""GPU parity of the elementwise path against the oracle, through the C-ABI."""
import numpy as np
import pytest

import theano_amd as th
from theano_amd import hip, tensor as T
from oracle import graph_ref as G
from conftest import assert_parity

pytestmark = pytest.mark.gpu


def run_both(ins, outs, vals):
    f = th.function(ins, outs)
    got = f(*vals)
    ref = G.evaluate(ins, outs, vals)
    return got, ref


def rand(rng, shape, dtype):
    if dtype == "bool":
        return rng.integers(0, 2, shape).astype("bool")
    if np.dtype(dtype).kind in "iu":
        lo = 0 if np.dtype(dtype).kind == "u" else -100
        return rng.integers(lo, 100, shape).astype(dtype)
    return rng.standard_normal(shape).astype(dtype)


# the input patterns of _good_broadcast_binary_normal, theano/tensor/tests/test_basic.py:664-684
BROADCAST_SHAPES = [((2, 3), (2, 3)), ((2, 2), (2,)), ((2, 3), (1, 1)), ((2, 3), (1, 3)), ((2, 3), (2, 1)),
                    ((3, 5), (1, 5)), ((2, 3, 4, 5), (1, 3, 1, 5)), ((0, 3), (0, 3)), ((5, 1031), (5, 1031)),
                    ((), ()), ((1,), (1,))]


@pytest.mark.parametrize("sa,sb", BROADCAST_SHAPES)
def test_binary_ops_over_broadcast_patterns(sa, sb):
    rng = np.random.default_rng(7)
    a = T.TensorType("float32", [s == 1 for s in sa])("a")
    b = T.TensorType("float32", [s == 1 for s in sb])("b")
    av, bv = rand(rng, sa, "float32"), rand(rng, sb, "float32") + 3
    outs = [a + b, a - b, a * b, a / b, T.maximum(a, b), T.minimum(a, b), a < b, T.eq(a, b), T.switch(a > 0, a, b)]
    got, ref = run_both([a, b], outs, [av, bv])
    for k, (g, r) in enumerate(zip(got, ref)):
        assert_parity(g, r, "binary op %d on %s %s" % (k, sa, sb))


@pytest.mark.parametrize("dtype", ["int8", "uint8", "int16", "uint16", "int32", "uint32", "int64", "uint64"])
def test_integer_ops_bit_exact(dtype):
    rng = np.random.default_rng(8)
    a, b = T.TensorType(dtype, (False, False))("a"), T.TensorType(dtype, (False, False))("b")
    av = rand(rng, (37, 53), dtype)
    bv = rand(rng, (37, 53), dtype)
    bv[bv == 0] = 3
    outs = [a + b, a * b, a - b, a % b, a // b, a & b, a | b, a ^ b, ~a, abs(a), T.sqr(a), a > b, T.neq(a, b),
            T.cast(a, "int8"), T.cast(a, "bool"), T.cast(a, "float32"), T.true_div(a, b)]
    got, ref = run_both([a, b], outs, [av, bv])
    for k, (g, r) in enumerate(zip(got, ref)):
        assert_parity(g, r, "%s op %d" % (dtype, k))


def test_int8_mod_and_intdiv_exhaustive_grid():
    # theano/tensor/tests/test_basic.py:878-896
    a, b = T.bcol("a"), T.brow("b")
    av = np.arange(-127, 128, dtype="int8")[:, None]
    bv = np.array([v for v in range(-127, 128) if v != 0], dtype="int8")[None, :]
    f = th.function([a, b], [a % b, a // b])
    m, d = f(av, bv)
    assert np.array_equal(m, np.array([[int(x) % int(y) for y in bv[0]] for x in av[:, 0]], dtype="int8"))
    assert np.array_equal(d, np.array([[int(x) // int(y) for y in bv[0]] for x in av[:, 0]], dtype="int8"))


def test_right_shift_equals_int_div():
    a = T.ivector("a")
    av = np.arange(-5000, 5000, dtype="int32")
    s, d = th.function([a], [a >> 3, a // 8])(av)
    assert np.array_equal(s, d) and np.array_equal(s, av >> 3)


def test_bool_ops():
    rng = np.random.default_rng(9)
    a, b = T.TensorType("bool", (False,))("a"), T.TensorType("bool", (False,))("b")
    av, bv = rand(rng, (1000,), "bool"), rand(rng, (1000,), "bool")
    got, ref = run_both([a, b], [a & b, a | b, a ^ b, ~a, a + b, a * b, T.cast(a, "int32")], [av, bv])
    for g, r in zip(got, ref):
        assert_parity(g, r, "bool")


@pytest.mark.parametrize("dtype", ["float32", "float64", "float16"])
def test_unary_math(dtype):
    rng = np.random.default_rng(10)
    x = T.TensorType(dtype, (False, False))("x")
    xv = (rng.uniform(0.1, 3.0, (61, 130))).astype(dtype)
    outs = [T.exp(x), T.log(x), T.sqrt(x), T.tanh(x), T.sigmoid(x - 1), T.softplus(x), T.sin(x), T.cos(x), T.sqr(x),
            T.inv(x), T.neg(x), abs(x - 1), T.sgn(x - 1), T.floor(x), T.ceil(x), T.log1p(x), T.expm1(x), x ** 2,
            T.clip(x, 0.5, 2.0), T.arctan(x)]
    got, ref = run_both([x], outs, [xv])
    tol = {"float64": dict(rtol=1e-12, atol=1e-12)}.get(dtype)
    if dtype == "float64":  # libm implementations differ in the last ulps for transcendental functions
        tol = dict(rtol=1e-12, atol=1e-12)
    for k, (g, r) in enumerate(zip(got, ref)):
        assert_parity(g, r, "%s unary %d" % (dtype, k), tol=tol)


def test_angle_units_and_range_tests_follow_the_c_text():
    """deg2rad / rad2deg multiply by a double constant and round once; InRange is two comparisons under C's
    conversions (theano/scalar/basic.py:3086-3150, 1434-1481): bit for bit against the oracle."""
    from theano_amd import scalar as scal
    from theano_amd.tensor.elemwise import Elemwise
    rng = np.random.default_rng(12)
    for dtype in ("float32", "float64", "float16", "int8", "int32", "uint16"):
        x = T.TensorType(dtype, (False, False))("x")
        xv = rand(rng, (37, 129), dtype) if np.dtype(dtype).kind in "iu" else rng.uniform(-720, 720, (37, 129)).astype(dtype)
        got, ref = run_both([x], [T.deg2rad(x), T.rad2deg(x)], [xv])
        for g, r in zip(got, ref):
            assert g.dtype == r.dtype and np.array_equal(g, r), dtype
    x, lo, hi = T.fmatrix("x"), T.TensorType("int8", (False, False))("lo"), T.TensorType("float64", (True, False))("hi")
    xv = rng.integers(-4, 5, (50, 70)).astype("float32")
    lov = rng.integers(-4, 5, (50, 70)).astype("int8")
    hiv = rng.integers(-4, 5, (1, 70)).astype("float64")
    outs = [Elemwise(scal.InRange(a, b))(x, lo, hi) for a in (False, True) for b in (False, True)]
    got, ref = run_both([x, lo, hi], outs, [xv, lov, hiv])
    for g, r in zip(got, ref):
        assert g.dtype == np.bool_ and np.array_equal(g, r)
    assert got[0].sum() > got[3].sum() > 0        # the closed range holds more points than the open one
    # gradients: a constant factor; none through a range test
    x = T.fmatrix("x")
    gx = th.grad(T.sum(T.deg2rad(x) * T.rad2deg(x)), x)
    xv = rng.standard_normal((9, 11)).astype("float32")
    got, ref = run_both([x], [gx], [xv])
    assert_parity(got[0], ref[0], "angle unit gradient")
    np.testing.assert_allclose(got[0], 2 * xv, rtol=1e-6)


def test_sigmoid_thresholds_and_nan_handling():
    x = T.fvector("x")
    xv = np.array([-100, -88.5, -88, -30, 0, 14.9, 15, 15.1, 100, np.nan, np.inf, -np.inf], "float32")
    got, ref = run_both([x], [T.sigmoid(x), T.maximum(x, 0), T.minimum(x, 0), T.isnan(x), T.isinf(x)], [xv])
    for g, r in zip(got, ref):
        assert_parity(g, r, "special values")


def test_division_operator_on_integer_tensors_is_numpy_true_division():
    """`x / y` on integer tensors is true division with a floatX result (``theano/tensor/var.py:199-206``,
    ``theano/scalar/basic.py:1891-1915``: ``(double)x / y`` rounded to floatX), never the truncating one.
    The expectation is NumPy's own `/`, not the oracle's walk over this package's graph."""
    rng = np.random.default_rng(77)
    i, j, b = T.imatrix("i"), T.imatrix("j"), T.bmatrix("b")
    iv = rng.integers(-2 ** 20, 2 ** 20, (61, 130)).astype("int32")
    jv = rng.integers(1, 1000, (61, 130)).astype("int32") * rng.choice([-1, 1], (61, 130)).astype("int32")
    bv = rng.integers(-128, 128, (61, 130)).astype("int8")
    bv[bv == 0] = 5
    f = th.function([i, j, b], [i / j, b / 2, 2 / i, b / b, i / b, 7 / b, (i / j) * 2])
    iv_nz = np.where(iv == 0, 3, iv).astype("int32")
    got = f(iv_nz, jv, bv)
    want = [iv_nz / jv, bv / 2, 2 / iv_nz, bv / bv, iv_nz / bv, 7 / bv, (iv_nz / jv) * 2]
    for k, (g, w) in enumerate(zip(got, want)):
        assert g.dtype == np.dtype(th.config.floatX), (k, g.dtype)
        assert_parity(g, w.astype(th.config.floatX), "true division %d" % k)
    assert not np.array_equal(got[0], (iv_nz // jv).astype(got[0].dtype))      # it is not the truncating division
    q, r = th.function([i, j], list(divmod(i, j)))(iv, jv)
    wq, wr = np.divmod(iv, jv)
    assert q.dtype == r.dtype == np.int32 and np.array_equal(q, wq) and np.array_equal(r, wr)


def test_round_defaults_to_half_to_even_like_numpy():
    """``theano/tensor/basic.py:2175-2192``: `round(a)` and `a.round()` round halves to even."""
    x = T.fvector("x")
    xv = np.array([-2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 3.5, 0.49999997, 8388609.0, 1.25, -7.75], "float32")
    got = th.function([x], [T.round(x), x.round(), T.iround(x)])(xv)
    assert np.array_equal(got[0], np.round(xv)) and np.array_equal(got[1], np.round(xv))
    assert got[2].dtype == np.int64 and np.array_equal(got[2], np.round(xv).astype("int64"))


def test_round_half_away_from_zero_is_c_round_on_the_device():
    """theano/scalar/basic.py:2686 emits C round(): halves away from zero, and nothing like
    floor(x + 0.5) at 0.49999997 or at odd integers from 2**23 up.  Bit-exact against the oracle
    (itself pinned against the host's libm) over the finite range, float32 and float64."""
    from test_oracle_scalar import ROUND_PINS, finite_float32_sweep
    x, d = T.fvector("x"), T.dvector("d")
    f = th.function([x, d], [T.round_half_away_from_zero(x), T.round_half_away_from_zero(d),
                             T.round(x, mode="half_away_from_zero")])
    pins = np.array([p for p, _ in ROUND_PINS], "float64")
    got32, got64, got_front = f(pins.astype("float32"), pins)
    for (p, want), g in zip(ROUND_PINS, got32):
        if want is not None:
            assert float(g) == want and np.signbit(g) == np.signbit(np.float32(want)), (p, g)
    assert got64[-1] == 4503599627370497.0 and np.array_equal(got_front, got32)
    xv = np.concatenate([finite_float32_sweep(), np.array([np.inf, -np.inf, np.nan], "float32")])
    dv = xv.astype("float64") * 1.0000001
    got, ref = run_both([x, d], [T.round_half_away_from_zero(x), T.round_half_away_from_zero(d)], [xv, dv])
    for g, r in zip(got, ref):
        assert g.dtype == r.dtype and np.array_equal(g, r, equal_nan=True)
        assert np.array_equal(np.signbit(g), np.signbit(r))


def test_exp_sigmoid_softplus_over_the_whole_finite_float32_range():
    """The default float32 exp is one hardware exp2 of x * log2(e) (relative error up to |x| * 4e-8) and
    the sigmoid core one exp2 and one rcp: checked against the oracle at the float32 bar (rtol 1e-5,
    atol 1e-6) over every exponent of the finite range and around each saturation threshold."""
    from test_oracle_scalar import finite_float32_sweep
    x = T.fvector("x")
    xv = finite_float32_sweep()
    outs = [T.exp(x), T.sigmoid(x), T.softplus(x), T.expm1(x), T.tanh(x), T.exp(-x) * 2]
    with np.errstate(all="ignore"):
        got, ref = run_both([x], outs, [xv])
    for k, (g, r) in enumerate(zip(got, ref)):
        assert_parity(g, r, "output %d" % k)            # float32: rtol 1e-5, atol 1e-6; inf / nan must coincide
    # the same through a float64 graph at the float64 bar
    d = T.dvector("d")
    dv = xv.astype("float64") * 7.0
    with np.errstate(all="ignore"):
        got, ref = run_both([d], [T.exp(d), T.sigmoid(d), T.softplus(d)], [dv])
    for k, (g, r) in enumerate(zip(got, ref)):
        assert_parity(g, r, "float64 output %d" % k, tol=dict(rtol=1e-12, atol=1e-300))


def test_weird_strides_five_dims():
    # theano/tensor/tests/test_elemwise.py:305-318
    rng = np.random.default_rng(11)
    x = T.TensorType("float32", (False,) * 5)("x")
    y = T.TensorType("float32", (False,) * 5)("y")
    xv = rng.standard_normal((2, 3, 4, 5, 6)).astype("float32")
    yv = rng.standard_normal((6, 5, 4, 3, 2)).astype("float32")
    got, ref = run_both([x, y], [x + y.dimshuffle(4, 3, 2, 1, 0), (x * 2).dimshuffle(1, 0, 4, 3, 2)], [xv, yv])
    for g, r in zip(got, ref):
        assert_parity(g, r, "5-d transposed")


def test_same_input_twice_and_many_inputs():
    rng = np.random.default_rng(12)
    x = T.fmatrix("x")
    xv = rng.standard_normal((17, 33)).astype("float32")
    got, ref = run_both([x], [x * x + x], [xv])
    assert_parity(got[0], ref[0], "same input")
    # theano/gpuarray/tests/test_opt.py:531-572: a sum of many inputs, more than one kernel's argument budget
    ins = [T.fmatrix("i%d" % k) for k in range(40)]
    vals = [rng.standard_normal((5, 9)).astype("float32") for _ in ins]
    out = ins[0]
    for i in ins[1:]:
        out = out + i
    got, ref = run_both(ins, [out], vals)
    assert_parity(got[0], ref[0], "40 inputs", tol=dict(rtol=1e-5, atol=1e-5))


def test_mixed_dtypes_follow_c_promotion():
    rng = np.random.default_rng(13)
    i, f, d, h = T.ivector("i"), T.fvector("f"), T.dvector("d"), T.TensorType("float16", (False,))("h")
    vals = [rand(rng, (300,), "int32"), rand(rng, (300,), "float32"), rand(rng, (300,), "float64"),
            rand(rng, (300,), "float16")]
    got, ref = run_both([i, f, d, h], [i * f, i + d, f * d, h * f, h + h, i / 7, T.cast(f, "float16")], vals)
    for k, (g, r) in enumerate(zip(got, ref)):
        assert_parity(g, r, "mixed %d" % k)


def test_large_contiguous_and_unaligned_views():
    rng = np.random.default_rng(14)
    x = T.fvector("x")
    xv = rng.standard_normal(3 * 1024 * 1024 + 5).astype("float32")
    f = th.function([x], T.exp(x) * 0.5)
    assert_parity(f(xv), G.evaluate([x], [T.exp(x) * 0.5], [xv])[0], "large vector")
    m = T.fmatrix("m")
    mv = rng.standard_normal((64, 259)).astype("float32")
    got, ref = run_both([m], [m.T * 2 + 1], [mv])
    assert_parity(got[0], ref[0], "transposed output order")


def test_host_scalar_operands_travel_by_value():
    x = T.fmatrix("x")
    s = T.TensorType("float32", (True, True))("s")
    f = th.function([x, s], x * s + s)
    xv = np.arange(12, dtype="float32").reshape(3, 4)
    assert_parity(f(xv, np.float32([[2.5]])), xv * np.float32(2.5) + np.float32(2.5), "immediate")
    assert "m0,3,0" in hip.last_plan() or ",3" in hip.last_plan()


def test_inplace_elementwise_matches_out_of_place():
    rng = np.random.default_rng(15)
    x, y = T.fmatrix("x"), T.fmatrix("y")
    xv, yv = rng.standard_normal((257, 130)).astype("float32"), rng.standard_normal((257, 130)).astype("float32")
    out = (T.exp(x) * y + 1.0) * T.tanh(y)
    f_in = th.function([x, y], out, fuse=False)
    f_out = th.function([x, y], out, fuse=False, inplace=False)
    assert any(n.op.inplace_pattern for n in f_in.toposort() if hasattr(n.op, "inplace_pattern"))
    a, b = f_in(xv, yv), f_out(xv, yv)
    assert np.array_equal(a, b)
    assert_parity(a, G.evaluate([x, y], [out], [xv, yv])[0], "unfused in-place chain")
    assert np.array_equal(f_in(xv, yv), a)            # the inputs were not overwritten by the first call


@pytest.mark.gpu
def test_column_major_inputs_give_column_major_outputs():
    """All inputs that are not broadcast along every dimension column-major (and not also
    row-major): the output is allocated column-major too (theano/tensor/elemwise.py:928-937),
    so the kernel streams; one row-major input, here also a (1, n) row, switches it back."""
    from theano_amd.hip import HipArray
    rng = np.random.default_rng(21)
    a = np.asfortranarray(rng.standard_normal((130, 70)).astype("float32"))
    b = np.asfortranarray(rng.standard_normal((130, 70)).astype("float32"))
    row = rng.standard_normal((1, 70)).astype("float32")
    x, y = T.fmatrix("x"), T.fmatrix("y")
    r = T.TensorType("float32", (True, False))("r")
    s = T.TensorType("float32", (True, True))("s")
    f = th.function([x, y, s], [th.Out(T.exp(x) * y + s, device=True)])
    one = np.full((1, 1), 0.5, "float32")
    out = f(HipArray.from_numpy(a), HipArray.from_numpy(b), one)[0]
    assert out.is_fortran and out.strides == (4, 130 * 4)
    assert np.allclose(out.to_numpy(), np.exp(a) * b + one, rtol=1e-5, atol=1e-6)
    out = f(HipArray.from_numpy(a), HipArray.from_numpy(np.ascontiguousarray(b)), one)[0]
    assert out.c_contiguous
    assert np.allclose(out.to_numpy(), np.exp(a) * b + one, rtol=1e-5, atol=1e-6)
    g = th.function([x, y, r], [th.Out(T.exp(x) * y + r, device=True)])
    out = g(HipArray.from_numpy(a), HipArray.from_numpy(b), row)[0]
    assert out.c_contiguous
    assert np.allclose(out.to_numpy(), np.exp(a) * b + row, rtol=1e-5, atol=1e-6)
    # through the host boundary
    got = th.function([x, y, s], [T.exp(x) * y + s])(a, b, one)[0]
    assert np.allclose(got, np.exp(a) * b + one, rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_special_functions_against_scipy(dtype):
    """erf / erfc / erfcx / erfinv / erfcinv / gamma / gammaln / psi / tri_gamma
    (theano/scalar/basic_scipy.py:29-470) against scipy.special, which is what the
    reference's own impl calls, and their gradients against the oracle's evaluation of
    the same gradient graphs."""
    rng = np.random.default_rng(17)
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == "float32" else dict(rtol=1e-11, atol=1e-12)
    x = T.TensorType(dtype, (False,))("x")
    wide = np.concatenate([rng.uniform(-4, 4, 3000), rng.uniform(0.05, 30, 3000)]).astype(dtype)
    unit = rng.uniform(-0.999, 0.999, 6000).astype(dtype)
    pos = np.concatenate([rng.uniform(0.05, 30, 5000), rng.uniform(-5.9, -0.1, 1000)]).astype(dtype)
    pos = pos[np.abs(pos - np.round(pos)) > 0.05]      # stay away from the poles
    cases = [("erf", wide), ("erfc", wide), ("erfcx", wide), ("erfinv", unit), ("erfcinv", (1 + unit).astype(dtype)),
             ("gamma", pos), ("gammaln", pos), ("psi", pos), ("tri_gamma", pos)]
    for name, vals in cases:
        op = getattr(T, name)
        outs = [op(x)] if name == "tri_gamma" else [op(x), th.grad(T.sum(op(x)), x)]
        got = th.function([x], outs)(vals)
        ref = G.evaluate([x], outs, [vals])
        for k, (g, r) in enumerate(zip(got, ref)):
            assert_parity(g, r, "%s output %d" % (name, k), tol=tol)


@pytest.mark.gpu
def test_float_floor_division_is_exact_at_integer_quotients():
    """x // y and x % y on float32 where x is an exact multiple of y: the quotient handed
    to floor must be the correctly rounded one (an ulp low would lose a whole unit),
    whatever division the kernels are built with; also int64 // float32, which C evaluates
    in float32 (theano/scalar/basic.py:1985-2025)."""
    rng = np.random.default_rng(77)
    k = rng.integers(-200, 200, 20000).astype("float32")
    y = (rng.integers(1, 64, 20000) / 8.0).astype("float32") * rng.choice([-1, 1], 20000).astype("float32")
    x = (k * y).astype("float32")                       # exact: small integers times eighths
    a, b = T.fvector("a"), T.fvector("b")
    q, r = th.function([a, b], [a // b, a % b])(x, y)
    assert np.array_equal(q, k) and np.array_equal(r, np.zeros_like(r))
    ref = G.evaluate([a, b], [a // b, a % b], [x + 0.25, y])
    got = th.function([a, b], [a // b, a % b])(x + np.float32(0.25), y)
    assert np.array_equal(got[0], ref[0]) and np.allclose(got[1], ref[1], rtol=1e-6, atol=1e-6)
    i, f = T.lvector("i"), T.fvector("f")
    iv = rng.integers(-1000, 1000, 5000)
    fv = rng.uniform(0.5, 3.0, 5000).astype("float32")
    fv[:3], iv[:3] = np.float32(1.96), 49              # 49 / 1.96f rounds to 25.0f
    got = th.function([i, f], i // f)(iv, fv)
    assert got.dtype == np.float64 and got[0] == 25.0
    assert np.array_equal(got, G.evaluate([i, f], [i // f], [iv, fv])[0])


@pytest.mark.gpu
def test_multi_output_kernels_from_merged_siblings():
    """Adam-style updates in one kernel with three results (float32 and float16 storage,
    a transposed operand), against the oracle; plus an integer pair with different dtypes."""
    rng = np.random.default_rng(31)
    p, g, m, v = [T.fmatrix(n) for n in "pgmv"]
    m2 = 0.9 * m + 0.1 * g
    v2 = 0.999 * v + 0.001 * T.sqr(g)
    p2 = p - 0.01 * m2 / (T.sqrt(v2) + 1e-8)
    outs = [m2, v2, p2, T.cast(p2, "float16"), p2.T * g.T]
    f = th.function([p, g, m, v], outs)
    assert sum(1 for n in f.toposort() if type(n.op).__name__ == "HipElemwise") <= 2
    vals = [rng.standard_normal((257, 129)).astype("float32") for _ in range(3)] + [rng.uniform(0.1, 1, (257, 129)).astype("float32")]
    for k, (a, b) in enumerate(zip(f(*vals), G.evaluate([p, g, m, v], outs, vals))):
        assert_parity(a, b, "adam output %d" % k, tol=dict(rtol=2e-3, atol=2e-3) if b.dtype == np.float16 else None)
    i, j = T.imatrix("i"), T.imatrix("j")
    outs = [(i & j) + 1, T.cast(i, "int8") ^ T.cast(j, "int8"), T.gt(i, j), i.astype("int64") * j]
    vals = [rng.integers(-2 ** 20, 2 ** 20, (65, 33)).astype("int32") for _ in range(2)]
    f = th.function([i, j], outs)
    assert sum(1 for n in f.toposort() if type(n.op).__name__ == "HipElemwise") == 1
    for a, b in zip(f(*vals), G.evaluate([i, j], outs, vals)):
        assert_parity(a, b, "integer siblings")


@pytest.mark.gpu
def test_user_written_composite_with_several_results():
    """An Elemwise over a Composite with more than one result, as a user writes it: every result on its own (the
    results nothing reads leave the Composite first: theano/tensor/tests/test_opt.py:1364-1382), all results
    together, and results that feed further elementwise work and a reduction."""
    from theano_amd import scalar as scal
    from theano_amd.tensor.elemwise import Elemwise
    sx = scal.float32()
    pair = Elemwise(scalar_op=scal.Composite([sx], [sx + 1, sx - 1]))
    X = T.fmatrix("X")
    o = pair(X)
    for k, want in ((0, [[2.0]]), (1, [[0.0]])):
        f = th.function([X], o[k])
        kernels = [n for n in f.toposort() if isinstance(n.op, hip.HipElemwise)]
        assert len(kernels) == 1 and len(kernels[0].outputs) == 1
        assert np.array_equal(f(np.array([[1.0]], "float32")), np.array(want, "float32"))
    rng = np.random.default_rng(17)
    sy = scal.float32()
    three = Elemwise(scalar_op=scal.Composite([sx, sy], [sx + sy, sx * sy, scal.exp(sx) - sy]))
    Y = T.frow("Y")
    r = three(X, Y)
    xv = rng.standard_normal((301, 77)).astype("float32")
    yv = rng.standard_normal((1, 77)).astype("float32")
    got = th.function([X, Y], r)(xv, yv)
    assert np.array_equal(got[0], xv + yv) and np.array_equal(got[1], xv * yv)
    assert_parity(got[2], G.evaluate([X, Y], [r[2]], [xv, yv])[0])
    outs = [r[0] * 2 + r[2], T.sum(r[1], axis=0), T.tanh(r[0]), T.max(r[2])]
    got = th.function([X, Y], outs)(xv, yv)
    ref = G.evaluate([X, Y], outs, [xv, yv])
    for g, w in zip(got, ref):
        assert_parity(g, w)
    # the same Composite over integers, exact
    ix, iy = scal.int32(), scal.int32()
    both = Elemwise(scalar_op=scal.Composite([ix, iy], [ix // iy, ix % iy]))
    A, B = T.imatrix("A"), T.imatrix("B")
    av = rng.integers(-1000, 1000, (50, 60)).astype("int32")
    bv = rng.integers(1, 30, (50, 60)).astype("int32") * rng.choice([-1, 1], (50, 60)).astype("int32")
    q, m = th.function([A, B], both(A, B))(av, bv)
    assert np.array_equal(q, av // bv) and np.array_equal(m, av % bv)


def test_fast_division_over_the_whole_float32_range():
    """The default float32 division (one hardware reciprocal of the divisor's mantissa, the exponent applied in two
    halves) over random bit patterns of the whole finite range on both sides - denormal operands, quotients that
    overflow, underflow or land among the denormals - and the special values: within 2.5 ulp of the exact quotient
    (1.5 units of the smallest denormal where the quotient is denormal), infinities, zeros with their signs and NaN
    exactly where IEEE division has them.  Once with a divisor per element and once with one divisor per row (the
    form whose divisor half the compiler computes once)."""
    rng = np.random.default_rng(2024)
    n = 400000

    def patterns(k):
        bits = rng.integers(0, 0x7f800000, k, dtype=np.uint32) | (rng.integers(0, 2, k, dtype=np.uint32) << 31)
        return bits.view("float32")

    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 1e-45, -1e-45, 1.1754944e-38, 3.4028235e38,
                        -3.4028235e38, 2.0 ** -126, 2.0 ** 127, 2.0 ** -149, 3.0, 1.0 / 3.0], "float32")
    av = np.concatenate([patterns(n), np.repeat(special, len(special)), rng.uniform(-4, 4, n).astype("float32")])
    bv = np.concatenate([patterns(n), np.tile(special, len(special)), rng.uniform(-4, 4, n).astype("float32")])
    a, b = T.fvector("a"), T.fvector("b")
    got = th.function([a, b], a / b)(av, bv)
    assert "|fd" in hip.last_plan()

    def check(g, x, y, what):
        with np.errstate(all="ignore"):
            exact = x.astype("float64") / y.astype("float64")
            want = exact.astype("float32")
        special_case = ~np.isfinite(want) | (want == 0) | ~np.isfinite(exact)
        # where IEEE gives infinity, zero or NaN: the same, sign included - except at the two edges of the range,
        # where a quotient within 2.5 ulp of the largest finite value / of the smallest denormal may round either way
        near_top = np.isfinite(exact) & (np.abs(exact) > 3.4028e38)
        near_zero = np.isfinite(exact) & (np.abs(exact) < 3e-45)
        strict = special_case & ~near_top & ~near_zero
        assert np.array_equal(g[strict], want[strict], equal_nan=True), what
        assert np.array_equal(np.signbit(g[strict & ~np.isnan(want)]), np.signbit(want[strict & ~np.isnan(want)])), what
        rest = ~special_case
        with np.errstate(over="ignore"):
            ulp = np.maximum(np.spacing(np.abs(want[rest]).astype("float32")).astype("float64"), 2.0 ** -149)
        ulp[~np.isfinite(ulp)] = 2.0 ** 104              # the spacing above the largest finite value
        err = np.abs(g[rest].astype("float64") - exact[rest]) / ulp
        assert err.max() <= 2.5, (what, float(err.max()), x[rest][err.argmax()], y[rest][err.argmax()])
        edge = near_top | near_zero
        assert np.all(np.isinf(g[near_top]) | (np.abs(g[near_top]) >= 3.4028e38)) and np.all(np.abs(g[near_zero]) <= 4.5e-45), what
        return float(err.max())

    worst = check(got, av, bv, "divisor per element")
    # one divisor per row
    m = T.fmatrix("m")
    c = T.fcol("c")
    rows = np.concatenate([patterns(3000), special])
    mv = np.concatenate([patterns(len(rows) * 64), ]).reshape(len(rows), 64)
    mv[:, :len(special)] = special
    got2 = th.function([m, c], m / c)(mv, rows.reshape(-1, 1))
    check(got2.reshape(-1), mv.reshape(-1), np.repeat(rows, 64), "divisor per row")
    assert worst > 0.5          # it is the approximate form that ran


def test_exact_float32_math_when_the_fast_forms_are_switched_off(monkeypatch):
    """THX_FAST_DIV=0: float32 division and square root correctly rounded (bit-equal to
    NumPy's), exp / sigmoid from the math library (within 2 ulp of the double result); the
    default build stays inside rtol 1e-5 on the same inputs."""
    rng = np.random.default_rng(5)
    a, b = T.fvector("a"), T.fvector("b")
    av = np.concatenate([rng.uniform(-87, 87, 50000), rng.uniform(-2, 2, 50000)]).astype("float32")
    bv = rng.uniform(0.01, 50, av.size).astype("float32")
    outs = [a / b, T.sqrt(b), T.exp(a), T.sigmoid(a)]
    fast = th.function([a, b], outs)(av, bv)
    monkeypatch.setenv("THX_FAST_DIV", "0")
    exact = th.function([a, b], outs)(av, bv)
    assert "|fd" not in hip.last_plan()
    assert np.array_equal(exact[0], av / bv) and np.array_equal(exact[1], np.sqrt(bv))
    e64 = np.exp(av.astype("float64"))
    assert np.max(np.abs(exact[2] - e64) / e64) < 2.5e-7
    s64 = 1.0 / (1.0 + np.exp(-av.astype("float64")))
    ok = av > -80                                      # below, results are denormal
    assert np.max(np.abs(exact[3][ok] - s64[ok]) / s64[ok]) < 4e-7
    for f, e in zip(fast, exact):
        assert np.allclose(f, e, rtol=1e-5, atol=1e-37)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_bessel_and_incomplete_gamma_functions_against_scipy(dtype):
    """j0 / j1 / i0 / i1 and gammainc / gammaincc / gammau / gammal / chi2sf
    (theano/scalar/basic_scipy.py:482-857) against scipy, which the reference's impl calls."""
    import scipy.special
    import scipy.stats
    rng = np.random.default_rng(23)
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == "float32" else dict(rtol=1e-10, atol=1e-13)
    x = T.TensorType(dtype, (False,))("x")
    k = T.TensorType(dtype, (False,))("k")
    xv = np.concatenate([rng.uniform(-12, 12, 4000), [0.0]]).astype(dtype)
    got = th.function([x], [T.j0(x), T.j1(x), T.i0(x), T.i1(x), th.grad(T.sum(T.j1(x)), x), th.grad(T.sum(T.i1(x)), x)])(xv)
    x64 = xv.astype("float64")
    want = [scipy.special.j0(x64), scipy.special.j1(x64), scipy.special.i0(x64), scipy.special.i1(x64),
            scipy.special.jvp(1, x64), scipy.special.ivp(1, x64)]
    for g, w in zip(got, want):
        assert g.dtype == np.dtype(dtype) and np.allclose(g, w, **tol)
    kv = rng.uniform(0.1, 40, 6000).astype(dtype)
    pv = np.concatenate([rng.uniform(0.01, 80, 5998), [0.0, 1e-3]]).astype(dtype)
    outs = [T.gammainc(k, x), T.gammaincc(k, x), T.gammal(k, x), T.gammau(k, x), T.chi2sf(x, k)]
    got = th.function([k, x], outs)(kv, pv)
    k64, p64 = kv.astype("float64"), pv.astype("float64")
    want = [scipy.special.gammainc(k64, p64), scipy.special.gammaincc(k64, p64),
            scipy.special.gammainc(k64, p64) * scipy.special.gamma(k64),
            scipy.special.gammaincc(k64, p64) * scipy.special.gamma(k64), scipy.stats.chi2.sf(p64, k64)]
    for j, (g, w) in enumerate(zip(got, want)):
        assert g.dtype == np.dtype("float64" if j == 4 else dtype), j
        with np.errstate(over="ignore"):             # gamma(k) leaves float32's range for k > 35: inf on both sides
            assert np.allclose(g, w.astype(g.dtype), rtol=tol["rtol"] * 5, atol=tol["atol"]), j
    ref = G.evaluate([k, x], outs, [kv, pv])
    for g, r in zip(got, ref):
        assert np.allclose(g, r, rtol=tol["rtol"] * 5, atol=tol["atol"])


@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_bessel_functions_of_real_order_against_scipy(dtype):
    """jv / iv (theano/scalar/basic_scipy.py:698-726, 786-811; scipy.special.jv / iv in the reference): orders of
    either sign, whole and fractional, arguments from the series' range through the transition to the oscillating /
    growing one, whole orders at negative arguments, the special points, and the gradient with respect to the
    argument, (f(v - 1, x) -+ f(v + 1, x)) / 2."""
    import scipy.special
    rng = np.random.default_rng(29)
    v, x = T.TensorType(dtype, (False,))("v"), T.TensorType(dtype, (False,))("x")
    n = 6000
    vv = np.concatenate([rng.uniform(0, 5, n), rng.uniform(-6, 0, n), rng.uniform(0, 60, n),
                         rng.integers(-8, 9, n).astype("float64")]).astype(dtype)
    xv = np.concatenate([rng.uniform(0, 2, n), rng.uniform(0.05, 40, n), rng.uniform(0, 120, n),
                         rng.uniform(-30, 30, n)]).astype(dtype)
    outs = [T.jv(v, x), T.iv(v, x)]
    got = th.function([v, x], outs)(vv, xv)
    v64, x64 = vv.astype("float64"), xv.astype("float64")
    with np.errstate(all="ignore"):
        want = [scipy.special.jv(v64, x64), scipy.special.iv(v64, x64)]
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == "float32" else dict(rtol=2e-10, atol=1e-12)
    for name, g, w in zip(("jv", "iv"), got, want):
        assert g.dtype == np.dtype(dtype)
        with np.errstate(all="ignore"):
            w = w.astype(dtype)                     # values beyond float32's range are infinite on both sides
        ok = np.isclose(g, w, equal_nan=True, **tol)
        assert ok.all(), "%s: %d values differ, first at v=%r x=%r: got %r, scipy %r" % (
            name, (~ok).sum(), vv[~ok][0], xv[~ok][0], g[~ok][0], w[~ok][0])
    ref = G.evaluate([v, x], outs, [vv, xv])
    for g, r in zip(got, ref):
        assert np.isclose(g, r, equal_nan=True, **tol).all()
    # special points: x = 0 for every kind of order, NaN operands, fractional orders left of zero
    pv = np.array([0, 1, 2.5, -1, -0.5, -1.5, -2.5, 0.5, np.nan, 1, 2], dtype)
    px = np.array([0, 0, 0, 0, 0, 0, 0, -1.0, 1, np.nan, 1e-30], dtype)
    got = th.function([v, x], outs)(pv, px)
    with np.errstate(all="ignore"):
        assert np.isclose(got[0], scipy.special.jv(pv, px).astype(dtype), rtol=tol["rtol"], atol=0, equal_nan=True).all()
        assert np.isclose(got[1], scipy.special.iv(pv, px).astype(dtype), rtol=tol["rtol"], atol=0, equal_nan=True).all()
    if dtype == "float64":
        # large arguments (Hankel's expansion): against a 40-digit evaluation, SciPy itself drifts there
        mpmath = pytest.importorskip("mpmath")
        mpmath.mp.dps = 40
        bx = rng.uniform(1e3, 1e7, 60)
        bv = rng.uniform(-1, 1, 60) * np.sqrt(bx)
        truth = np.array([float(mpmath.besselj(mpmath.mpf(float(a)), mpmath.mpf(float(b)))) for a, b in zip(bv, bx)])
        big = th.function([v, x], T.jv(v, x))(bv, bx)
        assert (np.abs(big - truth) / np.sqrt(2 / (np.pi * bx))).max() < 1e-12
    # gradient with respect to the argument; none with respect to the order
    gv = rng.uniform(0.2, 6, 2000).astype(dtype)
    gx = rng.uniform(0.2, 15, 2000).astype(dtype)
    dj, di = th.function([v, x], [th.grad(T.sum(T.jv(v, x)), x), th.grad(T.sum(T.iv(v, x)), x)])(gv, gx)
    assert np.allclose(dj, scipy.special.jvp(gv.astype("float64"), gx.astype("float64")), **tol)
    assert np.allclose(di, scipy.special.ivp(gv.astype("float64"), gx.astype("float64")), rtol=tol["rtol"] * 5, atol=tol["atol"])
    with pytest.raises(th.gradient.NullTypeGradError):
        th.grad(T.sum(T.jv(v, x)), v)


@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_sigmoid_family_and_stabilised_forms(dtype):
    """Activations of theano/tensor/nnet (sigm.py, nnet.py:2008-2050, 2437-2516) against closed forms in float64,
    with arguments far enough out that the unstabilised formulas overflow; approximate sigmoids against the
    oracle's restatement of their C text."""
    from theano_amd.tensor import nnet
    rng = np.random.default_rng(31)
    x = T.TensorType(dtype, (False, False))("x")
    t = T.TensorType(dtype, (False, False))("t")
    big = 80.0 if dtype == "float32" else 700.0
    xv = np.concatenate([rng.uniform(-big, big, (37, 50)), rng.uniform(-3, 3, (37, 50)), [[0.0] * 50]]).astype(dtype)
    tv = rng.uniform(0, 1, xv.shape).astype(dtype)
    x64, t64 = xv.astype("float64"), tv.astype("float64")
    sp = np.logaddexp(0, x64)                                    # softplus
    sg = np.exp(-np.logaddexp(0, -x64))                          # sigmoid
    outs = [T.log(nnet.sigmoid(x)), T.log(1 - nnet.sigmoid(x)), T.log1p(T.exp(x)), T.exp(x) / (1 + T.exp(x)),
            1.0 / (1.0 + T.exp(-x)), nnet.sigmoid(x) * T.exp(-x), nnet.binary_crossentropy(nnet.sigmoid(x), t),
            nnet.sigmoid_binary_crossentropy(x, t), nnet.elu(x), nnet.selu(x), nnet.hard_sigmoid(x),
            th.grad(T.sum(nnet.sigmoid_binary_crossentropy(x, t)), x), th.grad(T.sum(nnet.softsign(x)), x),
            th.grad(T.sum(nnet.elu(x, 0.5)), x)]
    bce = t64 * (sp - x64) + (1 - t64) * sp
    elu = np.where(x64 > 0, x64, np.expm1(np.minimum(x64, 0)))
    # Python floats become constants of dtype floatX (theano/scalar/basic.py:309-312): rounded to float32 by default
    scale, alpha = (float(np.dtype(th.config.floatX).type(c)) for c in (1.0507009873554804934193349852946,
                                                                       1.6732632423543772848170429916717))
    want = [x64 - sp, -sp, sp, sg, sg, np.exp(-sp), bce, bce, elu,
            scale * np.where(x64 > 0, x64, alpha * np.expm1(np.minimum(x64, 0))),
            np.clip(0.2 * x64 + 0.5, 0, 1), sg - t64, 1 / (1 + np.abs(x64)) ** 2,
            np.where(x64 > 0, 1.0, 0.5 * np.exp(np.minimum(x64, 0)))]
    got = th.function([x, t], outs)(xv, tv)
    # the reference's softplus returns x itself beyond 16 (float64), dropping log1p(exp(-16)) = 1.1e-7 of 16: 7e-9
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == "float32" else dict(rtol=1e-8, atol=1e-13)
    for j, (g, w) in enumerate(zip(got, want)):
        assert g.dtype == np.dtype(dtype) and np.all(np.isfinite(g)), j
        assert np.allclose(g, w, **tol), (j, np.abs(g - w).max())
    approx = [nnet.ultra_fast_sigmoid(x), nnet.softsign(x)]
    got, ref = run_both([x], approx, [xv])
    for g, r in zip(got, ref):
        assert_parity(g, r, "approximate sigmoid / softsign")
    assert np.abs(got[0] - sg).max() < 0.028


def test_gradient_of_log_one_minus_sigmoid_reference_values():
    """The literal answers of test_grad_useless_sum (theano/tensor/tests/test_elemwise.py:1281-1297)."""
    x = T.TensorType("float32", (True,))("x")
    f = th.function([x], th.grad(T.log(1.0 - T.nnet.sigmoid(x))[0], x))
    got = [f(np.array([v], "float32")) for v in (-100, -1, 0, 1, 100)]
    assert np.allclose(got, [[-3.72007598e-44], [-0.26894142], [-0.5], [-0.73105858], [-1.]])


def test_pow_over_every_pair_of_integer_and_float_dtypes():
    """test_elemwise_pow, theano/gpuarray/tests/test_elemwise.py:43-70: base ** exponent for every pair of
    (u)int8-64 and float16/32/64 dtypes gives NumPy's dtype and values (small exact integers)."""
    dtypes = ["uint8", "uint16", "uint32", "uint64", "int8", "int16", "int32", "int64", "float16", "float32", "float64"]
    rng = np.random.RandomState(0)
    for db in dtypes:
        base = T.TensorType(db, (False,))("b")
        exps = [T.TensorType(de, (False,))("e_" + de) for de in dtypes]
        bv = rng.randint(0, 5, size=10).astype(db)
        evs = [rng.randint(0, 3, size=10).astype(de) for de in dtypes]
        got = th.function([base] + exps, [base ** e for e in exps])(bv, *evs)
        for de, ev, g in zip(dtypes, evs, got):
            want = bv ** ev
            assert g.dtype == want.dtype, (db, de, g.dtype, want.dtype)
            if g.dtype.kind in "iu":
                assert np.array_equal(g, want), (db, de, g, want)
            else:                                # the device's pow is within a place of the host's, not identical
                tol = {"float16": 2e-3, "float32": 1e-6, "float64": 1e-12}[str(g.dtype)]
                assert np.allclose(g, want, rtol=tol, atol=0), (db, de, g, want)


@pytest.mark.parametrize("nd", [2, 8])
def test_add_and_mul_of_64_operands(nd):
    """test_many_arg_elemwise, theano/gpuarray/tests/test_opt.py:531-572: more operands than one kernel
    takes are split over several kernels, in 2 and in 8 dimensions."""
    from theano_amd.hip import HipElemwise
    rng = np.random.RandomState([1, 2, 3])
    shape = [rng.randint(1, 5) for _ in range(nd)]
    args = [rng.randn(*shape).astype("float32") for _ in range(64)]
    sym = [T.TensorType("float32", (False,) * nd)() for _ in range(64)]
    for op, npop in ((T.add, np.add), (T.mul, np.multiply)):
        f = th.function(sym, op(*sym))
        kernels = [n for n in f.toposort() if isinstance(n.op, HipElemwise)]
        assert len(kernels) > 1 and all(len(n.inputs) <= th.config.max_fused_inputs for n in kernels)
        want = args[0].astype("float64")
        for a in args[1:]:
            want = npop(want, a)
        # 63 float32 additions of N(0, 1) terms: rounding of partial sums near 8 in magnitude, against float64
        assert np.allclose(f(*args), want, rtol=1e-5, atol=3e-5 if op is T.add else 1e-30)


def test_float16_composites_and_casts():
    """test_composite_elemwise_float16 and test_cast_float16, theano/gpuarray/tests/test_elemwise.py:152-207:
    mixed float16 / integer / float32 expressions fuse and run, and every cast to and from float16 gives
    NumPy's ``astype`` (the reference only compiles the first two graphs; here they are also checked
    against the oracle)."""
    rng = np.random.default_rng(51)
    w, x, y = T.bvector("w"), T.TensorType("float16", (False,))("x"), T.fvector("y")
    cz = T.tanh(x + T.cast(y, "float16"))
    o = cz - cz ** 2 + T.cast(x, "int16") + T.cast(x, "float32") + T.cast(w, "float16") - T.constant(np.float16(1.0))
    vals = [rng.integers(-5, 5, 300).astype("int8"), rng.uniform(-4, 4, 300).astype("float16"),
            rng.uniform(-2, 2, 300).astype("float32")]
    got, ref = run_both([w, x, y], [o], vals)
    assert got[0].dtype == ref[0].dtype == np.float32
    assert_parity(got[0], ref[0], "float16 composite", tol=dict(rtol=2e-3, atol=2e-3))
    v = T.TensorType("uint8", (False,))("v")
    hs = [T.TensorType("float16", (False,))(n) for n in "abcd"]
    o2 = T.switch(v, T.mul(hs[0], hs[1], hs[2]), hs[3])
    vals2 = [rng.integers(0, 2, 300).astype("uint8")] + [rng.uniform(-2, 2, 300).astype("float16") for _ in hs]
    got, ref = run_both([v] + hs, [o2], vals2)
    assert got[0].dtype == np.float16
    assert_parity(got[0], ref[0], "float16 switch", tol=dict(rtol=2e-3, atol=2e-3))
    f16, f32, i8 = T.TensorType("float16", (False,))("h"), T.fvector("f"), T.bvector("i")
    outs = [f16.astype("float32"), f32.astype("float16"), f32.astype("float64"), f16.astype("int8"),
            f32.astype("int8"), i8.astype("float16"), i8.astype("float32")]
    d1 = (rng.random(4) * 10).astype("float16")
    d2 = (rng.random(5) * 10).astype("float32")
    d3 = (rng.random(6) * 10).astype("int8")
    res = th.function([f16, f32, i8], outs)(d1, d2, d3)
    srcs = [d1, d2, d2, d1, d2, d3, d3]
    for r, o, d in zip(res, outs, srcs):
        assert r.dtype == np.dtype(o.type.dtype) and np.array_equal(r, d.astype(o.type.dtype))


def test_inplace_operations_overwrite_their_first_argument():
    """theano/tensor/inplace.py through function(accept_inplace=True): results equal the out-of-place
    operation's converted to the first operand's type, and the first argument holds the result after
    the call (theano/tensor/tests/test_basic.py:653-657) - a host array, a device array, a strided
    device view; an argument that had to be converted is left alone."""
    from theano_amd.hip.runtime import HipArray
    from theano_amd.tensor import inplace as I
    rng = np.random.default_rng(21)
    x, y = T.fmatrix("x"), T.fmatrix("y")
    cases = [(I.add_inplace, np.add), (I.sub_inplace, np.subtract), (I.mul_inplace, np.multiply),
             (I.true_div_inplace, np.true_divide), (I.maximum_inplace, np.maximum), (I.minimum_inplace, np.minimum),
             (I.pow_inplace, lambda a, b: np.abs(a) ** b)]
    for op, npf in cases:
        xv = rng.uniform(0.5, 2.0, (33, 65)).astype("float32")
        yv = rng.uniform(0.5, 2.0, (33, 65)).astype("float32")
        want = npf(xv, yv).astype("float32")
        f = th.function([x, y], op(x, y), accept_inplace=True)
        got = f(xv, yv)
        np.testing.assert_allclose(got, want, rtol=1e-6)
        assert np.array_equal(xv, got), op
    for op, npf in [(I.exp_inplace, np.exp), (I.neg_inplace, np.negative), (I.sqr_inplace, np.square),
                    (I.abs__inplace, np.abs), (I.floor_inplace, np.floor), (I.tanh_inplace, np.tanh),
                    (I.deg2rad_inplace, np.deg2rad)]:
        xv = rng.uniform(-2.0, 2.0, (17, 129)).astype("float32")
        want = npf(xv)
        got = th.function([x], op(x), accept_inplace=True)(xv)
        np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-7)
        assert np.array_equal(xv, got), op
    # mixed types: the result is converted to the first operand's type (transfer_type(0))
    i, d = T.imatrix("i"), T.dmatrix("d")
    iv = rng.integers(-50, 50, (9, 40)).astype("int32")
    dv = rng.uniform(-3, 3, (9, 40))
    want = (iv.astype("float64") * dv).astype("int32")          # C conversion: truncation toward zero
    got = th.function([i, d], I.mul_inplace(i, d), accept_inplace=True)(iv, dv)
    assert got.dtype == np.int32 and np.array_equal(got, want) and np.array_equal(iv, want)
    # a chain over one buffer, and another reader of the old value
    f = th.function([x, y], [I.mul_inplace(I.exp_inplace(x), y), x * 2], accept_inplace=True)
    xv = rng.standard_normal((20, 30)).astype("float32")
    yv = rng.standard_normal((20, 30)).astype("float32")
    old = xv.copy()
    r0, r1 = f(xv, yv)
    np.testing.assert_allclose(r0, np.exp(old) * yv, rtol=2e-6)
    assert np.array_equal(r1, old * 2) and np.array_equal(xv, r0)
    # device arguments: overwritten on the device, also through a strided view
    f = th.function([x, y], I.add_inplace(x, y), accept_inplace=True)
    xv = rng.standard_normal((40, 50)).astype("float32")
    yv = rng.standard_normal((40, 50)).astype("float32")
    xd = HipArray.from_numpy(xv)
    got = f(xd, yv)
    assert np.array_equal(got, xv + yv) and np.array_equal(xd.to_numpy(), xv + yv)
    big = HipArray.from_numpy(np.zeros((50, 80), "float32"))
    view = big.view((40, 50), (4, 320))        # big.T[0:40, 0:50]
    from theano_amd.hip.views import copy_into
    copy_into(HipArray.from_numpy(xv), view)
    got = f(view, yv)
    back = big.to_numpy()
    assert np.array_equal(got, xv + yv) and np.array_equal(back.T[0:40, 0:50], xv + yv)
    assert not back.T[40:].any() and not back.T[:, 50:].any()
    # an argument that is converted on the way in was copied: nothing to overwrite
    lst = [[1.0, 2.0], [3.0, 4.0]]
    got = f(lst, np.ones((2, 2), "float32"))
    assert np.array_equal(got, [[2, 3], [4, 5]]) and lst == [[1.0, 2.0], [3.0, 4.0]]
    ro = np.ones((2, 2), "float32")
    ro.flags.writeable = False
    assert np.array_equal(f(ro, ro), np.full((2, 2), 2, "float32")) and np.array_equal(ro, np.ones((2, 2)))


def test_verify_grad_and_gradient_only_operations():
    """verify_grad (theano/gradient.py:1625-1800) accepts right gradients and names a wrong one; grad_clip's
    documented example (:2208-2215): d/dx grad_clip(x, -1, 1)**2 at 2.0 is 1.0 where d/dx x**2 is 4.0."""
    from theano_amd import gradient as G, scalar as scal
    from theano_amd.tensor.elemwise import Elemwise
    rng = np.random.RandomState(7)
    pts = [rng.uniform(0.5, 1.5, (3, 4)), rng.uniform(0.5, 1.5, (1, 4))]
    G.verify_grad(lambda a, b: T.tanh(a * b) + T.log(a) / b, pts, rng=rng)
    G.verify_grad(lambda a: T.sum(T.exp(a), axis=0), [pts[0].astype("float32")], rng=rng)
    G.verify_grad(lambda a: T.max(a, axis=1), [pts[0]], rng=rng)
    G.verify_grad(lambda a: T.prod(a, axis=1) * T.sum(T.sqr(a)), [pts[0]], rng=rng)
    e = T.exp
    G.verify_grad(lambda a: e(a - T.max(a, axis=1, keepdims=True)) / T.sum(e(a - T.max(a, axis=1, keepdims=True)), axis=1,
                                                                           keepdims=True), [pts[0]], rng=rng)
    with pytest.raises(TypeError, match="rng"):
        G.verify_grad(T.exp, [pts[0]])
    G.verify_grad(T.tanh, [pts[0]], rng=np.random.default_rng(5), n_tests=3)     # a Generator serves as well
    with pytest.raises(TypeError, match="floating point"):
        G.verify_grad(T.exp, [np.arange(4)], rng=rng)

    class WrongSqr(scal.Sqr):                       # the gradient of x**2 claimed to be x
        def L_op(self, inputs, outputs, gout):
            return [gout[0] * inputs[0]]
    wrong = Elemwise(WrongSqr(scal.same_out, name="wrong_sqr"))
    with pytest.raises(G.GradientError) as info:
        G.verify_grad(wrong, [pts[0]], rng=rng)
    assert info.value.abs_err > info.value.abs_tol and "exceed tolerance" in str(info.value)
    # gradient-only operations on the device
    x = T.fscalar("x")
    z, z2 = th.grad(G.grad_clip(x, -1, 1) ** 2, x), th.grad(x ** 2, x)
    got = th.function([x], [z, z2])(np.float32(2.0))
    assert got[0] == 1.0 and got[1] == 4.0
    v = T.fvector("v")
    vv = np.array([-2.0, 0.25, 3.0], "float32")
    f = th.function([v], [th.grad(T.sum(G.zero_grad(T.exp(v)) * v), v), th.grad(T.sum(G.grad_scale(T.sqr(v), 0.5)), v),
                          th.grad(T.sum(G.grad_clip(T.sqr(v), -1, 1) * 3 * v), v), G.grad_clip(v, 0, 0) + G.zero_grad(v)])
    g0, g1, g2, fwd = f(vv)
    np.testing.assert_allclose(g0, np.exp(vv), rtol=1e-6)
    np.testing.assert_allclose(g1, vv, rtol=1e-6)                       # 0.5 * 2v
    np.testing.assert_allclose(g2, 3 * vv ** 2 + np.clip(3 * vv, -1, 1) * 2 * vv, rtol=1e-6)
    assert np.array_equal(fwd, 2 * vv)


def test_fp_contract_off_gives_the_unfused_float32_arithmetic(monkeypatch):
    """$THX_FP_CONTRACT=off (read when a kernel is first compiled): a multiply followed by an add is two roundings,
    as NumPy's float32 arithmetic does them - bit for bit; the default lets the compiler fuse them into one
    (closer to the exact value, but one expression compiled into two kernels need not fuse alike).  The
    expressions carry constants no other test uses, so that their kernels are compiled here."""
    rng = np.random.default_rng(31)
    x, y, z = T.fmatrix("x"), T.fmatrix("y"), T.fmatrix("z")
    xv, yv, zv = [rng.standard_normal((97, 130)).astype("float32") for _ in range(3)]
    f32 = np.float32
    want = xv * yv + zv * f32(1.2578125) - f32(0.3720703125)
    want2 = (xv * yv + zv) * yv - xv * zv * f32(3.0791015625)
    monkeypatch.setenv("THX_FP_CONTRACT", "off")
    got, got2 = th.function([x, y, z], [x * y + z * f32(1.2578125) - f32(0.3720703125),
                                        (x * y + z) * y - x * z * f32(3.0791015625)])(xv, yv, zv)
    assert np.array_equal(got, want) and np.array_equal(got2, want2)


ARITH_DTYPES = ["int8", "uint8", "int16", "int32", "int64", "float16", "float32", "float64"]


@pytest.mark.parametrize("left", ARITH_DTYPES)
def test_arithmetic_over_every_pair_of_dtypes_against_numpy(left):
    """+ * / // between a `left` vector and a vector of every other dtype, values and result dtypes against NumPy's own
    arithmetic (not the oracle's walk over this package's graph): the value side of test_arithmetic_cast
    (theano/tensor/tests/test_basic.py:6919-7060).  `/` of two integer operands is floatX (float32 here) holding the
    float64 quotient rounded once (``TrueDiv.c_code``, theano/scalar/basic.py:1899-1915)."""
    from conftest import TOL
    rng = np.random.default_rng(abs(hash(left)) % 1000)

    def values(dt, n=517):
        if np.dtype(dt).kind == "u":
            return rng.integers(1, 12, n).astype(dt)
        if np.dtype(dt).kind == "i":
            v = rng.integers(-11, 12, n)
            v[v == 0] = 7
            return v.astype(dt)
        return (rng.uniform(0.5, 4.0, n) * rng.choice([-1.0, 1.0], n)).astype(dt)

    x = T.TensorType(left, (False,))("x")
    ys = [T.TensorType(dt, (False,))("y_" + dt) for dt in ARITH_DTYPES]
    outs = []
    for y in ys:
        outs += [x + y, x * y, x / y, x // y]
    f = th.function([x] + ys, outs)
    xv, yvs = values(left), [values(dt) for dt in ARITH_DTYPES]
    got = f(xv, *yvs)
    k = 0
    for dt, yv in zip(ARITH_DTYPES, yvs):
        up = np.result_type(left, dt)
        both_int = np.dtype(left).kind in "iu" and np.dtype(dt).kind in "iu"
        # The type the arithmetic happens in is C's, as in the reference's generated code: double if an operand is
        # double, else float if an operand is floating (float16 storage computes in float32), whatever type the
        # result is then stored in - float32 + int32 is a float32 sum stored as float64.
        if "float64" in (left, dt):
            ct = "float64"
        elif both_int:
            ct = None
        else:
            ct = "float32"
        if both_int:
            want = [xv.astype(up) + yv.astype(up), xv.astype(up) * yv.astype(up),
                    (xv.astype("float64") / yv.astype("float64")).astype("float32"),
                    np.floor_divide(xv.astype(up), yv.astype(up))]
        else:
            xc, yc = xv.astype(ct), yv.astype(ct)
            want = [(xc + yc).astype(up), (xc * yc).astype(up), (xc / yc).astype(up), np.floor(xc / yc).astype(up)]
        for name, g, w in zip(("add", "mul", "true_div", "int_div"), got[k:k + 4], want):
            what = "%s %s %s" % (left, name, dt)
            assert g.dtype == w.dtype, (what, g.dtype, w.dtype)
            if w.dtype.kind in "iu" or name == "int_div":
                assert np.array_equal(g, w), what                 # integers, and floors (whole numbers): exact
            else:
                bar = TOL["float16" if w.dtype == np.float16 else (ct or "float32")]
                assert_parity(g, w, what, tol=bar)
        k += 4


_INT_TYPES = ("bool", "int8", "uint8", "int16", "uint16", "int32", "uint32", "int64", "uint64")


def _int_grid(dtype, avoid_min):
    if dtype == "bool":
        return np.array([False, True])
    info = np.iinfo(dtype)
    vals = {info.min + 1, info.min + 2, info.max, info.max - 1, 0, 1, 2, 3, 5, 7, 100}
    if info.min < 0:
        vals |= {-1, -2, -3, -5, -7, -100}
    if not avoid_min:
        vals.add(info.min)
    return np.array(sorted(vals), dtype=dtype)


@pytest.mark.parametrize("opname", ["add", "sub", "mul", "maximum", "minimum", "int_div", "mod"])
def test_binary_integer_ops_over_every_pair_of_integer_types(opname):
    """Every pair of integer operand types, values at the ends of each range and small ones of either sign:
    + - * wrap, maximum / minimum compare in C's common type and keep the winner's own value, // and % test each
    operand's sign in its own type and divide in the common one (the oracle's restatements of these are pinned
    against gcc).  The most negative int32 / int64 stay out of // and %: their negation is undefined in C."""
    op = getattr(T, opname)
    divides = opname in ("int_div", "mod")
    problems = []                       # collected, so that one pair's failure does not hide the others
    for tx in _INT_TYPES:
        for ty in _INT_TYPES:
            x, y = T.vector("x", dtype=tx), T.vector("y", dtype=ty)
            try:
                out = op(x, y)
            except TypeError:
                assert opname == "sub" and tx == ty == "bool"
                continue
            gx, gy = _int_grid(tx, divides), _int_grid(ty, divides)
            xv, yv = np.repeat(gx, len(gy)), np.tile(gy, len(gx))
            if divides:
                keep = yv != 0
                xv, yv = xv[keep], yv[keep]
            with np.errstate(all="ignore"):
                ref = G.evaluate([x, y], [out], [xv, yv])[0]
            got = th.function([x, y], out)(xv, yv)
            assert got.dtype == ref.dtype, (opname, tx, ty)
            if ref.dtype.kind == "f":
                ok = (got == ref) | (np.isnan(got) & np.isnan(ref))
            else:
                ok = got == ref
            bad = np.flatnonzero(~ok)
            if bad.size:
                problems.append("%s(%s, %s): x=%s y=%s gives %s, the oracle %s" % (
                    opname, tx, ty, xv[bad[0]], yv[bad[0]], got[bad[0]], ref[bad[0]]))
    assert not problems, "\n".join(problems[:10])


def test_clip_and_switch_over_integer_type_combinations():
    """``clip`` over a fixed sample of 60 triples of integer types and ``switch`` over every pair, on values at the
    ends of each range: the conditionals convert as C's do (the oracle's restatements of both are pinned against
    gcc) - an int8 -128 clipped against a uint32 maximum comes out as 4294967168."""
    import itertools
    types = [t for t in _INT_TYPES if t != "bool"]
    small = lambda t: np.array(sorted({np.iinfo(t).min, np.iinfo(t).min + 1, 0, 1, 3, np.iinfo(t).max} |        # noqa: E731
                                      ({-1, -3} if np.iinfo(t).min < 0 else set())), dtype=t)
    rng = np.random.default_rng(8)
    triples = [tuple(types[i] for i in rng.integers(0, len(types), 3)) for _ in range(60)] + [("int8", "int64", "uint32")]
    problems = []
    for tx, tl, th_ in triples:
        x, lo, hi = T.vector("x", dtype=tx), T.vector("lo", dtype=tl), T.vector("hi", dtype=th_)
        out = T.clip(x, lo, hi)
        vals = [np.ascontiguousarray(a.reshape(-1)) for a in np.meshgrid(small(tx), small(tl), small(th_), indexing="ij")]
        with np.errstate(all="ignore"):
            ref = G.evaluate([x, lo, hi], [out], vals)[0]
        got = th.function([x, lo, hi], out)(*vals)
        if not (got.dtype == ref.dtype and np.array_equal(got, ref, equal_nan=True)):
            problems.append(("clip", tx, tl, th_))
    for ta, tb in itertools.product(types, repeat=2):
        c, a, b = T.vector("c", dtype="int8"), T.vector("a", dtype=ta), T.vector("b", dtype=tb)
        out = T.switch(c, a, b)
        vals = [np.ascontiguousarray(v.reshape(-1)) for v in
                np.meshgrid(np.array([0, 1, -1], "int8"), small(ta), small(tb), indexing="ij")]
        with np.errstate(all="ignore"):
            ref = G.evaluate([c, a, b], [out], vals)[0]
        got = th.function([c, a, b], out)(*vals)
        if not (got.dtype == ref.dtype and np.array_equal(got, ref, equal_nan=True)):
            problems.append(("switch", ta, tb))
    assert not problems, problems[:10]


@pytest.mark.gpu
@pytest.mark.parametrize("shape,perm", [((257, 129), (1, 0)), ((33, 65, 17), (2, 1, 0)), ((33, 65, 17), (1, 2, 0)),
                                        ((9, 1, 31, 7), (3, 2, 1, 0)), ((5, 6, 7, 8, 3), (4, 2, 0, 3, 1))])
def test_transposed_operands_and_results_walk_memory_in_order(shape, perm):
    """Operands that are all transposed the same way give a result laid out like them only in the column-major
    case (theano/tensor/elemwise.py:928-937); whatever the layout, the kernel walks the dimensions in the order
    of the result's strides and the values are those of the reference."""
    from theano_amd.hip import HipArray
    rng = np.random.default_rng(5)
    a = rng.standard_normal(shape).astype("float32")
    b = rng.standard_normal(shape).astype("float32")
    tt = T.TensorType("float32", (False,) * len(shape))
    x, y = tt("x"), tt("y")
    out = T.exp(x) * y + x
    ref = G.evaluate([x, y], [out], [a.transpose(perm), b.transpose(perm)])[0]
    xt, yt = tt("xt"), tt("yt")
    g = th.function([xt, yt], T.exp(xt.dimshuffle(*perm)) * yt.dimshuffle(*perm) + xt.dimshuffle(*perm))
    assert_parity(g(a, b), ref, "transposed inside the graph %s %s [%s]" % (shape, perm, hip.last_plan()))
    h = th.function([x, y], [th.Out(out, device=True)])
    da, db = HipArray.from_numpy(a), HipArray.from_numpy(b)
    got = h(da.transpose(*perm), db.transpose(*perm))[0]
    assert_parity(got.to_numpy(), ref, "transposed device views %s %s [%s]" % (shape, perm, hip.last_plan()))
    # one operand transposed, the other not: the result is row-major and still right
    c = rng.standard_normal(tuple(shape[p] for p in perm)).astype("float32")
    k = th.function([xt, y], T.exp(xt.dimshuffle(*perm)) * y + y)
    assert_parity(k(a, c), G.evaluate([x, y], [T.exp(x) * y + y], [a.transpose(perm), c])[0],
                  "mixed layouts %s %s [%s]" % (shape, perm, hip.last_plan()))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["int8", "float16", "float32", "float64"])
def test_operands_that_start_off_a_vector_boundary(dtype):
    """Views that drop leading elements or columns keep full-width accesses through element-aligned pointers
    (plans marked `|ua`): every alignment of two inputs and of the result written in place, odd lengths, rows of a
    matrix whose pitch is odd.  Values are those of Elemwise.perform (theano/tensor/elemwise.py:790)."""
    from theano_amd.hip import HipArray
    rng = np.random.default_rng(44)
    kind = np.dtype(dtype).kind
    draw = (lambda shape: rng.integers(-50, 50, shape).astype(dtype)) if kind == "i" else \
           (lambda shape: (rng.integers(-64, 65, shape) / 16.0).astype(dtype))
    tol = {"float16": {"rtol": 2e-3, "atol": 2e-3}}.get(dtype)
    vec, mat = T.TensorType(dtype, (False,)), T.TensorType(dtype, (False, False))
    x, y, m, w = vec("x"), vec("y"), mat("m"), mat("w")
    out = x * 2 + y
    f = th.function([x, y], [th.Out(out, device=True)])
    a, b = draw(50100), draw(50100)
    da, db = HipArray.from_numpy(a), HipArray.from_numpy(b)
    size = a.itemsize
    marked = 0
    for lo_a in (0, 1, 2, 3, 5, 8, 15):
        for lo_b in (0, 1, 7):
            for n in (50000, 49999, 40003):
                va = da.view([n], [size], da.offset + lo_a * size)
                vb = db.view([n], [size], db.offset + lo_b * size)
                got = f(va, vb)[0].to_numpy()
                marked += "|ua|" in hip.last_plan()
                ref = G.evaluate([x, y], [out], [a[lo_a:lo_a + n], b[lo_b:lo_b + n]])[0]
                assert_parity(got, ref, "[%d:], [%d:] of %d %s [%s]" % (lo_a, lo_b, n, dtype, hip.last_plan()), tol=tol)
    assert marked >= 40, marked
    # through the graph: shifted views of one array, and the same with the result written over an operand
    g = th.function([x], x[1:] - x[:-1])
    assert_parity(g(a), G.evaluate([x], [x[1:] - x[:-1]], [a])[0], "difference of neighbours %s [%s]" % (dtype, hip.last_plan()), tol=tol)
    # matrices: columns dropped on the left, a pitch that is odd
    big, other = draw((300, 1031)), draw((300, 1024))
    out2 = m[:, 7:] + w
    got = th.function([m, w], out2)(big, other)
    assert "|ua|" in hip.last_plan(), hip.last_plan()
    assert_parity(got, G.evaluate([m, w], [out2], [big, other])[0], "columns dropped %s [%s]" % (dtype, hip.last_plan()), tol=tol)
    # rows that are no whole number of vectors, next to a row and a column that broadcast
    row = T.TensorType(dtype, (True, False))("row")
    col = T.TensorType(dtype, (False, True))("col")
    for shape in ((300, 1031), (7, 100003), (513, 129), (64, 33)):       # the last one: rows too short to bother
        a2, r2, c2 = draw(shape), draw((1, shape[1])), draw((shape[0], 1))
        out3 = [m * 2 + row, m - col]
        got = th.function([m, row, col], out3)(a2, r2, c2)
        if shape[1] >= 16 * (16 // a2.itemsize):
            assert "|rg|" in hip.last_plan(), hip.last_plan()
        ref = G.evaluate([m, row, col], out3, [a2, r2, c2])
        for g_, r_ in zip(got, ref):
            assert_parity(g_, r_, "ragged rows %s %s [%s]" % (shape, dtype, hip.last_plan()), tol=tol)
    cube = T.TensorType(dtype, (False, False, False))("cube")
    plane = T.TensorType(dtype, (False, True, False))("plane")
    a3, p3 = draw((9, 11, 1001)), draw((9, 1, 1001))
    out4 = cube + plane
    got = th.function([cube, plane], out4)(a3, p3)
    assert_parity(got, G.evaluate([cube, plane], [out4], [a3, p3])[0], "ragged rows of a cube %s [%s]" % (dtype, hip.last_plan()), tol=tol)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "float16", "int64"])
def test_permuted_reads_with_wide_tiles(dtype):
    """A permuted operand beside operands in the result's layout goes through 32 x 128 tiles when those are the
    majority, or when odd extents leave single-element accesses (4-byte elements and wider); square tiles otherwise.
    Extents that are no multiples of either tile side; values as in Elemwise.perform
    (theano/tensor/elemwise.py:790), integers and the floats' small integers bit for bit."""
    rng = np.random.default_rng(8)
    draw = lambda shape: rng.integers(-20, 21, shape).astype(dtype)
    # the result's rows are 511, 383, 255 and 300 long: the last would leave a quarter of its wide tiles empty
    cases = [((511, 300), (1, 0)), ((31, 383, 129), (0, 2, 1)), ((127, 255, 33), (2, 0, 1)), ((300, 513), (1, 0))]
    wide = 0
    for shape, perm in cases:
        tt = T.TensorType(dtype, (False,) * len(shape))
        x, y = tt("x"), tt("y")
        a, b = draw(shape), draw(tuple(shape[p] for p in perm))
        for out, ins, vals in ((x.dimshuffle(*perm) * 2 + y, [x, y], [a, b]), (x.dimshuffle(*perm) + y.dimshuffle(*np.argsort(perm)).dimshuffle(*perm) * 3, [x, y], [a, b])):
            got = th.function(ins, out)(*vals)
            wide += "|t32x128|" in hip.last_plan()
            ref = G.evaluate(ins, [out], vals)[0]
            assert got.dtype == ref.dtype and np.array_equal(got, ref), "%s %s %s [%s]" % (dtype, shape, perm, hip.last_plan())
    assert wide >= 3, wide
