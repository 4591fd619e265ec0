"""GPU parity of complex64 / complex128 elementwise work and sums against the oracle (NumPy's complex arithmetic,
which is what the reference runs for these types): the operand patterns and value ranges of the reference's
testers (theano/tensor/tests/test_basic.py:664-684 complex1 / complex2, :909-911, :1113, :1372, :1443, :1498, :1556,
:1643, :2127-2145), its complex-number tests (theano/tensor/tests/test_complex.py) and CAReduce over complex
(theano/tensor/tests/test_elemwise.py:340-347)."""
import numpy as np
import pytest

import theano_amd as th
from theano_amd import hip, tensor as T
from oracle import graph_ref as G
from conftest import assert_parity

pytestmark = pytest.mark.gpu

CTYPES = {"complex64": T.cmatrix, "complex128": T.zmatrix}


def crand(rng, shape, dtype, lo=-1.0, hi=1.0):
    return (rng.uniform(lo, hi, shape) + 1j * rng.uniform(lo, hi, shape)).astype(dtype)


def conftest_tol(dtype):
    from conftest import TOL
    return TOL[dtype]


def check(ins, outs, vals, tol=None):
    got = th.function(ins, outs)(*vals)
    ref = G.evaluate(ins, outs, vals)
    for k, (g, r) in enumerate(zip(got, ref)):
        assert_parity(g, r, "output %d [%s]" % (k, hip.last_plan()), tol)
    return got


@pytest.mark.parametrize("dtype", ["complex64", "complex128"])
def test_arithmetic_over_operand_patterns(dtype):
    rng = np.random.default_rng(51)
    z, w = CTYPES[dtype]("z"), CTYPES[dtype]("w")
    x = T.fmatrix("x") if dtype == "complex64" else T.dmatrix("x")
    zv, wv = crand(rng, (23, 37), dtype), crand(rng, (23, 37), dtype)
    xv = rng.uniform(-1, 1, (23, 37)).astype(x.type.dtype)
    nz = wv + np.where(np.abs(wv) < 0.1, 1, 0).astype(dtype)              # divisors away from 0
    nx = np.where(np.abs(xv) < 0.1, 1, xv).astype(xv.dtype)
    check([z, w], [z + w, z - w, z * w, z / w, -z, T.sqr(z), T.inv(w)], [zv, nz])       # complex1
    check([z, x], [z + x, z - x, z * x, z / x, x - z, x / z], [nz, nx])                  # complex2 and its mirror
    # broadcasting: rows, columns and one-element operands of both kinds
    r, c = T.TensorType(dtype, (True, False))("r"), T.TensorType(dtype, (False, True))("c")
    check([z, r, c], [z * r + c, r * c, z / r - c], [zv, nz[:1], wv[:, :1]])
    s = T.TensorType(dtype, ())("s")
    check([z, s], [z * s + s, s / z], [nz, np.asarray(0.5 - 2j, dtype)])
    # literals and a real array against complex scalars
    check([z, x], [z * (1 + 2j) + 3, x * (2 - 1j), (z + 1) * 2.5], [zv, xv])


def test_mixed_precision_and_integer_operands_widen_first():
    """complex64 with float64 / int32 gives complex128 and the operation runs there (NumPy converts the operands
    before its loop; precision of the wide operand is not lost on the way)."""
    rng = np.random.default_rng(52)
    z, d, i, b = T.cmatrix("z"), T.dmatrix("d"), T.imatrix("i"), T.bmatrix("b")
    zv = crand(rng, (17, 29), "complex64")
    dv = rng.uniform(1, 2, (17, 29)) + 1e-12
    iv = rng.integers(-2 ** 30, 2 ** 30, (17, 29)).astype("int32")
    bv = rng.integers(-100, 100, (17, 29)).astype("int8")
    outs = [z + d, z * i, z - b, d / (z + 2), T.cast(z, "complex128") * d, T.cast(i, "complex64"), T.cast(d, "complex128")]
    got = check([z, d, i, b], outs, [zv, dv, iv, bv])
    assert [g.dtype.name for g in got] == ["complex128", "complex128", "complex64", "complex128", "complex128",
                                           "complex64", "complex128"]
    assert np.array_equal(got[0].real, zv.real.astype("float64") + dv)     # exact: float64 addition of the parts
    with pytest.raises(TypeError):                                          # theano/tensor/tests/test_basic.py:2809-2814
        T.cast(z, "float32")


@pytest.mark.parametrize("dtype", ["complex64", "complex128"])
def test_unary_math_on_the_reference_ranges(dtype):
    rng = np.random.default_rng(53)
    z = CTYPES[dtype]("z")
    tol = dict(rtol=2e-5, atol=2e-6) if dtype == "complex64" else dict(rtol=1e-11, atol=1e-12)
    cases = [((-1, 1), [T.exp(z), T.expm1(z), T.sin(z), T.cos(z), T.sinh(z), T.cosh(z), T.tanh(z), T.sqrt(z), T.sqr(z),
                        T.tan(z), T.log1p(z)]),
             ((1, 5), [T.log(z), T.log2(z), T.log10(z), T.sqrt(z), T.inv(z)]),
             ((-3.14, 3.14), [T.sin(z), T.cos(z), T.tan(z), T.tanh(z)]),
             ((-30, 30), [T.tanh(z), T.sqrt(z), T.log(z)])]
    for (lo, hi), outs in cases:
        check([z], outs, [crand(rng, (64, 65), dtype, lo, hi)], tol)
    # values with a zero part, zeros, and both signs of an axis
    pts = np.array([[0, 1, -1, 1j, -1j, 2 + 0j, -2 + 0j, 0.5j, 1e-8, 1e-8j, -1e-8, 1 + 1e-8j, -1 + 1e-8j, -1 - 1e-8j]], dtype)
    check([z], [T.exp(z), T.sqrt(z), T.sin(z), T.cos(z), T.sinh(z), T.cosh(z), T.tanh(z), T.expm1(z), abs(z)], [pts], tol)
    check([z], [T.angle(z)], [pts], tol)
    check([z], [T.log(z), T.log1p(z)], [pts[:, 1:] + 0.25], tol)


@pytest.mark.parametrize("dtype", ["complex64", "complex128"])
def test_parts_modulus_argument_and_construction(dtype):
    """theano/tensor/tests/test_complex.py: real, imag, conj, abs, angle of complex values; complex(re, im) and
    complex_from_polar(r, theta) build them (test_basic.py:2127-2145)."""
    rng = np.random.default_rng(54)
    z = CTYPES[dtype]("z")
    part = "float32" if dtype == "complex64" else "float64"
    x, y = T.TensorType(part, (False, False))("x"), T.TensorType(part, (False, False))("y")
    zv = crand(rng, (31, 33), dtype, -4, 4)
    got = check([z], [T.real(z), T.imag(z), T.conj(z), abs(z), z.real + z.imag, z.conj() * z], [zv])
    assert np.array_equal(got[0], zv.real) and np.array_equal(got[1], zv.imag) and np.array_equal(got[2], zv.conj())
    assert got[3].dtype == part
    # the argument is declared float64 whatever the input (theano/scalar/basic.py:3693) but is computed in the
    # precision of the input, by NumPy as here: the bar is that precision's
    (ang,) = check([z], [T.angle(z)], [zv], conftest_tol(part))
    assert ang.dtype == "float64"
    xv, yv = rng.uniform(-2, 2, (31, 33)).astype(part), rng.uniform(-2, 2, (31, 33)).astype(part)
    got = check([x, y], [T.complex(x, y), T.complex_from_polar(abs(x), y), T.real(T.complex(x, y)) - x], [xv, yv])
    assert got[0].dtype == dtype and np.array_equal(got[0], xv + 1j * yv) and not got[2].any()
    # parts of real values: real(x) = x, imag(x) = 0, angle(x) = 0 or pi
    got = check([x], [T.real(x), T.imag(x), T.angle(x), T.conj(x)], [xv])
    assert np.array_equal(got[0], xv) and not got[1].any() and len(np.unique(got[2])) == 2


def test_comparisons_selection_and_tests_for_nan():
    rng = np.random.default_rng(55)
    z, w, x = T.cmatrix("z"), T.zmatrix("w"), T.fmatrix("x")
    zv = crand(rng, (19, 21), "complex64").round(1)
    wv = zv.astype("complex128")
    wv[::3] += 1e-3j
    xv = zv.real.copy()
    zv[5, 5] = np.nan + 1j
    zv[6, 6] = complex(1, np.inf)
    got = check([z, w, x], [T.eq(z, w), T.neq(z, w), T.eq(z, x), T.isnan(z), T.isinf(z), T.switch(x > 0, z, w),
                            T.switch(T.eq(z, w), 1.0, z), T.second(x, z)], [zv, wv, xv])
    assert got[3].sum() == 1 and got[4].sum() == 1 and got[5].dtype == "complex128"
    for bad in (lambda: z < w, lambda: T.maximum(z, w), lambda: T.sgn(z), lambda: z // w, lambda: z % w,
                lambda: T.floor(z), lambda: T.clip(z, 0, 1)):
        with pytest.raises((TypeError, NotImplementedError)):      # as the reference: no order, no sign, no floor
            th.function([z, w], bad())(zv, wv)


@pytest.mark.parametrize("dtype", ["complex64", "complex128"])
def test_powers(dtype):
    rng = np.random.default_rng(56)
    z, w = CTYPES[dtype]("z"), CTYPES[dtype]("w")
    x = T.TensorType("float32" if dtype == "complex64" else "float64", (False, False))("x")
    zv, wv = crand(rng, (40, 41), dtype, -2, 2), crand(rng, (40, 41), dtype, -1.5, 1.5)
    xv = rng.uniform(-3, 3, (40, 41)).astype(x.type.dtype)
    tol = dict(rtol=5e-5, atol=5e-6) if dtype == "complex64" else dict(rtol=1e-10, atol=1e-12)
    check([z, w, x], [z ** w, z ** x, x ** w, z ** 2, z ** 3.0, z ** -1, z ** 0.5], [zv, wv, xv], tol)
    pts = np.array([[0, 0, 0, 1, -1, 2]], dtype)
    exps = np.array([[0, 2, 0.5, 5, 3, 10]], dtype)
    check([z, w], [z ** w], [pts, exps], tol)


@pytest.mark.parametrize("dtype", ["complex64", "complex128"])
def test_sums_and_products(dtype):
    """CAReduce{add, mul} over complex (theano/tensor/tests/test_elemwise.py:340-347, 352-366): every axis pattern,
    accumulated in complex128; long rows and columns (split reductions), transposed and strided inputs, fused
    elementwise work before and after."""
    rng = np.random.default_rng(57)
    t3 = T.TensorType(dtype, (False,) * 3)("t3")
    v3 = crand(rng, (13, 17, 19), dtype)
    axes = [None, (0,), (1,), (2,), (0, 1), (0, 2), (1, 2)]
    check([t3], [T.sum(t3, axis=a) for a in axes], [v3])
    small = (crand(rng, (5, 4, 3), dtype) * 0.5 + 1).astype(dtype)
    check([t3], [T.prod(t3, axis=a) for a in axes], [small])
    z = CTYPES[dtype]("z")
    wide, tall = crand(rng, (3, 300001), dtype), crand(rng, (200003, 5), dtype)
    for val in (wide, tall):
        got = check([z], [T.sum(z, axis=0), T.sum(z, axis=1), T.sum(z), T.sum(abs(z)), T.sum(z * z.conj()).real], [val])
        assert np.allclose(got[2], val.astype("complex128").sum(), rtol=1e-5 if dtype == "complex64" else 1e-12)
    check([z], [T.sum(z.dimshuffle(1, 0), axis=1), T.sum(z[::2, 1::3], axis=0), T.mean(z, axis=0) if hasattr(T, "mean") else T.sum(z)],
          [crand(rng, (1234, 77), dtype)])
    zero = np.zeros((0, 7), dtype)
    got = th.function([z], [T.sum(z, axis=0), T.prod(z, axis=0)])(zero)
    assert np.array_equal(got[0], np.zeros(7, dtype)) and np.array_equal(got[1], np.ones(7, dtype))
    with pytest.raises((TypeError, NotImplementedError)):
        th.function([z], T.max(z, axis=0))(wide)


def test_gradient_through_parts_of_a_complex_value():
    """d/dx, d/dy of functions of complex(x, y) taken through abs, real, imag and angle."""
    rng = np.random.default_rng(58)
    x, y = T.dmatrix("x"), T.dmatrix("y")
    c = T.complex(x, y)
    cost = T.sum(abs(c) * 2 + T.real(c) * 3 - T.imag(c) * T.imag(c) + T.angle(c))
    gx, gy = th.grad(cost, [x, y])
    xv, yv = rng.uniform(0.5, 2, (9, 11)), rng.uniform(-2, 2, (9, 11))
    got = th.function([x, y], [gx, gy])(xv, yv)
    r = np.hypot(xv, yv)
    assert np.allclose(got[0], 2 * xv / r + 3 - yv / r ** 2, rtol=1e-10)
    assert np.allclose(got[1], 2 * yv / r - 2 * yv + xv / r ** 2, rtol=1e-10)
    z = T.zmatrix("z")
    with pytest.raises(NotImplementedError):        # no gradient through complex results, as in the reference
        th.grad(T.sum(abs(T.exp(z))), z)
