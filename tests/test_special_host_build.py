"""The device helpers for complex numbers and Bessel functions of real order, compiled for the host with g++
(the header is plain C++ once the device qualifiers are defined away) and compared with NumPy / SciPy, which is
what the reference evaluates these ops with (theano/scalar/basic.py:3623-3761 through NumPy's complex loops,
theano/scalar/basic_scipy.py:698-726, 786-811 through scipy.special)."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NAMES = ["exp", "log", "sqrt", "sin", "cos", "tan", "sinh", "cosh", "tanh", "expm1", "log1p", "div", "pow", "mul", "log2",
         "log10", "conj", "abs_angle", "polar"]


@pytest.fixture(scope="module")
def host(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("special") / "libspecial_host.so")
    cmd = ["g++", "-O2", "-shared", "-fPIC", "-I", os.path.join(ROOT, "theano_amd", "csrc", "kernels"),
           os.path.join(ROOT, "tests", "native", "special_host.cpp"), "-o", out]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    return ctypes.CDLL(out)


def _bessel(host, fn, v, x):
    v, x = np.ascontiguousarray(v, "float64"), np.ascontiguousarray(x, "float64")
    out = np.empty_like(v)
    getattr(host, fn)(ctypes.c_void_p(v.ctypes.data), ctypes.c_void_p(x.ctypes.data), ctypes.c_void_p(out.ctypes.data),
                      ctypes.c_int(v.size))
    return out


@pytest.mark.parametrize("name", ["jv", "iv"])
def test_bessel_of_real_order(host, name):
    import scipy.special
    ref = getattr(scipy.special, name)
    rng = np.random.default_rng(5)
    n = 20000
    for (vlo, vhi), (xlo, xhi) in (((0, 5), (0, 2)), ((0, 5), (2, 30)), ((0, 50), (0, 100)), ((-5, 0), (0, 30)),
                                   ((0, 3), (30, 500)), ((0, 200), (0, 50))):
        v, x = rng.uniform(vlo, vhi, n), rng.uniform(xlo, xhi, n)
        got, want = _bessel(host, "host_" + name, v, x), ref(v, x)
        # errors against the size of the function's envelope: J oscillates through zero
        scale = np.abs(want) + (np.sqrt(2 / (np.pi * np.maximum(x, 1))) if name == "jv" else 1e-300)
        assert not (np.isnan(got) ^ np.isnan(want)).any()
        assert (np.abs(got - want) / scale).max() < 2e-11, ((vlo, vhi), (xlo, xhi))
    v, x = rng.integers(-6, 7, n).astype("float64"), rng.uniform(-20, 20, n)       # whole orders take any argument
    got, want = _bessel(host, "host_" + name, v, x), ref(v, x)
    assert (np.abs(got - want) / (1 + np.abs(want))).max() < 1e-13
    if name == "jv":
        # large arguments take Hankel's expansion; SciPy itself drifts there (1e-9 of the envelope at x = 1e6 and
        # nothing right beyond 1e8), so the truth is mpmath's
        mpmath = pytest.importorskip("mpmath")
        mpmath.mp.dps = 40
        for lo, hi in ((30, 100), (1e3, 1e5), (1e5, 1e7), (1e7, 1e9)):
            x = rng.uniform(lo, hi, 40)
            v = rng.uniform(-1, 1, 40) * np.sqrt(x)
            truth = np.array([float(mpmath.besselj(mpmath.mpf(float(a)), mpmath.mpf(float(b)))) for a, b in zip(v, x)])
            got = _bessel(host, "host_jv", v, x)
            assert (np.abs(got - truth) / np.sqrt(2 / (np.pi * x))).max() < 5e-14, (lo, hi)
    pv = np.array([0, 1, 2.5, -1, -0.5, -1.5, -2.5, 0.5, np.nan, 1])
    px = np.array([0, 0, 0, 0, 0, 0, 0, -1.0, 1, np.nan])
    assert np.array_equal(_bessel(host, "host_" + name, pv, px), ref(pv, px), equal_nan=True)


@pytest.mark.parametrize("dtype", ["complex128", "complex64"])
def test_complex_helpers(host, dtype):
    rng = np.random.default_rng(6)
    fn = host.host_c128 if dtype == "complex128" else host.host_c64
    refs = {"exp": np.exp, "log": np.log, "sqrt": np.sqrt, "sin": np.sin, "cos": np.cos, "tan": np.tan, "sinh": np.sinh,
            "cosh": np.cosh, "tanh": np.tanh, "expm1": np.expm1, "log2": np.log2, "log10": np.log10, "conj": np.conj}
    bar = 1e-13 if dtype == "complex128" else 1e-6
    for scale in (1e-3, 1.0, 8.0):
        n = 20000
        z = ((rng.standard_normal(n) + 1j * rng.standard_normal(n)) * scale).astype(dtype)
        w = ((rng.standard_normal(n) + 1j * rng.standard_normal(n)) * min(scale, 2.0)).astype(dtype)
        z[:6] = [0, 1, -1, 1j, -1j, -2]
        w[:6] = [1, 0.5, 2, 3, -1, 0.5]
        for k, name in enumerate(NAMES):
            out = np.empty_like(z)
            fn(ctypes.c_int(k), ctypes.c_void_p(z.ctypes.data), ctypes.c_void_p(w.ctypes.data),
               ctypes.c_void_p(out.ctypes.data), ctypes.c_int(n))
            zz, ww = z.astype("complex128"), w.astype("complex128")          # the value of the stored operands
            with np.errstate(all="ignore"):
                if name == "div":
                    want = zz / ww
                elif name == "mul":
                    want = zz * ww
                elif name == "pow":
                    want = zz ** ww
                elif name == "log1p":
                    # NumPy's own complex log1p is log(1 + z); its real part carries the rounding of 1 + z
                    want = 0.5 * np.log1p(zz.real * (2 + zz.real) + zz.imag ** 2) + 1j * np.arctan2(zz.imag, 1 + zz.real)
                elif name == "abs_angle":
                    want = np.abs(zz) + 1j * np.angle(zz)
                elif name == "polar":
                    want = zz.real * np.exp(1j * zz.imag)
                else:
                    want = refs[name](zz)
            ok = np.isfinite(want)
            assert np.array_equal(np.isfinite(out), ok), name
            err = np.abs(out[ok] - want[ok]) / np.maximum(np.abs(want[ok]), 1e-300)
            limit = bar * (30 if name == "pow" else 5)
            assert err.max() <= limit, (name, scale, float(err.max()))
