import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # the tests load the library that is built; only where none is (a fresh checkout) do they build it
    if not os.path.exists(os.path.join(ROOT, "theano_amd", "csrc", "libthx_hip.so")):
        from theano_amd.csrc import build as lib_build
        lib_build.build()


# tolerances of the parity bar, by storage dtype
TOL = {"float32": dict(rtol=1e-5, atol=1e-6), "float64": dict(rtol=1e-12, atol=1e-12),
       "float16": dict(rtol=2e-3, atol=2e-3),
       # complex values: the float bars of their parts, applied to the modulus of the difference
       "complex64": dict(rtol=1e-5, atol=1e-6), "complex128": dict(rtol=1e-12, atol=1e-12)}


def assert_parity(got, ref, what="", tol=None):
    """Bit-exact for integer / bool results, within the stated tolerance for floats."""
    got, ref = np.asarray(got), np.asarray(ref)
    assert got.shape == ref.shape, "%s: shape %s != %s" % (what, got.shape, ref.shape)
    assert got.dtype == ref.dtype, "%s: dtype %s != %s" % (what, got.dtype, ref.dtype)
    if ref.dtype.kind in "biu":
        assert np.array_equal(got, ref), "%s: integer results differ" % what
        return
    t = tol or TOL[str(ref.dtype)]
    wide = "complex128" if ref.dtype.kind == "c" else "float64"
    ok = np.isclose(got.astype(wide), ref.astype(wide), equal_nan=True, **t)
    if not ok.all():
        bad = np.argwhere(~ok)[0]
        raise AssertionError("%s: %d of %d values outside %s, first at %s: got %r, expected %r" % (
            what, (~ok).sum(), ok.size, t, tuple(bad), got[tuple(bad)], ref[tuple(bad)]))


def _neighbourhood_worst(e):
    """For every element, the smallest of the worst values over the slices it belongs to: for each axis d the
    slice is everything that shares the element's index along d (a row, a column, a channel).  Slices of fewer than
    16 elements say too little and are left out; an array without a usable axis gives its overall worst."""
    bound = np.full(e.shape, e.max() if e.size else 0.0)
    for d in range(e.ndim):
        if e.shape[d] < 2 or e.size // e.shape[d] < 16:
            continue
        others = tuple(a for a in range(e.ndim) if a != d)
        bound = np.minimum(bound, e.max(axis=others, keepdims=True))
    return bound


def assert_within_reference_error(got, ref, truth, what="", tol=None):
    """The parity bar for results where the reference's own float32 evaluation order is farther
    from the exact value than the tolerance allows (a difference of nearly equal numbers, a float32
    accumulator over many terms): `truth` is the graph's value in float64 (the oracle's wide mode)
    and errors are counted in units of the bar, |v - truth| / (atol + rtol |truth|).  `ref` is the
    reference's arithmetic (the oracle).  Three conditions, all in those units:
      * overall, the device's worst element is within the bar or no worse than the oracle's worst;
      * locally, every element is within the bar or within twice the oracle's worst error over the
        element's own row / column / channel (the smallest such slice worst): cancellation error is
        shared along the reduced axes, so a device value that is off where the oracle is exact is
        not excused by an oracle error elsewhere in the array;
      * the elements beyond the bar are not more numerous than the oracle's (half as many again, plus two,
        are allowed for two different roundings of the same quantity).
    Integer results must be equal."""
    got, ref, truth = np.asarray(got), np.asarray(ref), np.asarray(truth)
    assert got.shape == ref.shape == truth.shape, "%s: shapes %s %s %s" % (what, got.shape, ref.shape, truth.shape)
    assert got.dtype == ref.dtype, "%s: dtype %s != %s" % (what, got.dtype, ref.dtype)
    if ref.dtype.kind in "biu":
        assert np.array_equal(got, ref), "%s: integer results differ" % what
        return
    t = tol or TOL[str(ref.dtype)]
    w = truth.astype("float64")
    fin = np.isfinite(w)
    assert np.array_equal(got.astype("float64")[~fin], w[~fin], equal_nan=True), "%s: non-finite values differ" % what
    if not w.size:
        return
    unit = t["atol"] + t["rtol"] * np.abs(np.where(fin, w, 0.0))
    with np.errstate(invalid="ignore"):
        e_got = np.where(fin, np.abs(got.astype("float64") - w) / unit, 0.0)
        e_ref = np.where(fin, np.abs(ref.astype("float64") - w) / unit, 0.0)
    assert not np.isnan(e_got).any(), "%s: NaN where the float64 value is finite" % what
    worst_ref, worst_got = float(e_ref.max()), float(e_got.max())
    assert worst_got <= max(1.0, worst_ref), (
        "%s: device result is %.2f bars (%s) from the float64 value, the reference's own arithmetic %.2f"
        % (what, worst_got, t, worst_ref))
    allowed = np.maximum(1.0, 2.0 * _neighbourhood_worst(e_ref))
    over = e_got > allowed
    if over.any():
        pos = tuple(np.argwhere(over)[0])
        raise AssertionError("%s: %d elements are farther from the float64 value than the bar and than twice the "
                             "reference's error nearby; first at %s: %.2f bars, allowed %.2f" % (
                                 what, int(over.sum()), pos, e_got[pos], allowed[pos]))
    n_got, n_ref = int((e_got > 1.0).sum()), int((e_ref > 1.0).sum())
    assert n_got <= n_ref + n_ref // 2 + 2 * (n_ref > 0), (
        "%s: %d elements beyond the bar, the reference's own arithmetic has %d" % (what, n_got, n_ref))


@pytest.fixture
def dry_run():
    """Run the HIP path in dry-run mode: kernels are planned and compiled for
    gfx950, nothing executes."""
    from theano_amd import hip
    hip.set_dry_run(True)
    yield
    hip.set_dry_run(False)
