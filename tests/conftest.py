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
       "float16": dict(rtol=2e-3, atol=2e-3)}


def assert_parity(got, ref, what="", tol=None):
    """Bit-exact for integer / bool results, within the stated tolerance for floats."""
    got, ref = np.asarray(got), np.asarray(ref)
    assert got.shape == ref.shape, "%s: shape %s != %s" % (what, got.shape, ref.shape)
    assert got.dtype == ref.dtype, "%s: dtype %s != %s" % (what, got.dtype, ref.dtype)
    if ref.dtype.kind in "biu":
        assert np.array_equal(got, ref), "%s: integer results differ" % what
        return
    t = tol or TOL[str(ref.dtype)]
    ok = np.isclose(got.astype("float64"), ref.astype("float64"), equal_nan=True, **t)
    if not ok.all():
        bad = np.argwhere(~ok)[0]
        raise AssertionError("%s: %d of %d values outside %s, first at %s: got %r, expected %r" % (
            what, (~ok).sum(), ok.size, t, tuple(bad), got[tuple(bad)], ref[tuple(bad)]))


@pytest.fixture
def dry_run():
    """Run the HIP path in dry-run mode: kernels are planned and compiled for
    gfx950, nothing executes."""
    from theano_amd import hip
    hip.set_dry_run(True)
    yield
    hip.set_dry_run(False)
