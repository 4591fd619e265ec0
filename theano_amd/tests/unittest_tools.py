"""Seeding and comparison helpers for tests (``theano/tests/unittest_tools.py:43-92, 277-358``):
``fetch_seed`` / ``seed_rng`` (the seed is ``$THEANO_AMD_UNITTEST_RSEED``, default 666, or ``random``),
``verify_grad`` with NumPy's global generator seeded when none is given, ``assert_allclose`` with the
per-dtype tolerances of ``TensorType.values_eq_approx`` raising ``WrongValue``."""
import os
import sys

import numpy as np

from .. import gradient


def fetch_seed(pseed=None):
    """The seed unit tests use: ``pseed`` if given, else the configured one; None (a random seed) for 'random'
    or an invalid setting."""
    seed = pseed or os.environ.get("THEANO_AMD_UNITTEST_RSEED", 666)
    if seed == "random":
        return None
    try:
        return int(seed) if seed else None
    except ValueError:
        print("Error: THEANO_AMD_UNITTEST_RSEED contains an invalid seed, using None instead", file=sys.stderr)
        return None


def seed_rng(pseed=None):
    """Seed NumPy's global generator with ``fetch_seed(pseed)``; returns the seed."""
    seed = fetch_seed(pseed)
    np.random.seed(seed)
    return seed


def verify_grad(op, pt, n_tests=2, rng=None, *args, **kwargs):
    """``gradient.verify_grad`` with the global generator, freshly seeded, when no ``rng`` is given."""
    if rng is None:
        seed_rng()
        rng = np.random
    gradient.verify_grad(op, pt, n_tests, rng, *args, **kwargs)


class WrongValue(Exception):
    def __init__(self, expected_val, val, rtol, atol):
        Exception.__init__(self)
        self.val1, self.val2, self.rtol, self.atol = expected_val, val, rtol, atol

    def __str__(self):
        a, b = np.asarray(self.val1), np.asarray(self.val2)
        lines = ["WrongValue", "  expected: shape %s dtype %s min %s max %s" % (a.shape, a.dtype, a.min() if a.size else "-",
                                                                             a.max() if a.size else "-"),
                 "  value   : shape %s dtype %s min %s max %s" % (b.shape, b.dtype, b.min() if b.size else "-",
                                                                 b.max() if b.size else "-")]
        if a.shape == b.shape and a.size:
            err = np.abs(a.astype("float64") - b.astype("float64"))
            lines.append("  max abs error %s, max rel error %s (rtol %s, atol %s)" % (
                err.max(), (err / np.maximum(np.abs(a).astype("float64"), 1e-30)).max(), self.rtol, self.atol))
        return "\n".join(lines)


def assert_allclose(expected, value, rtol=None, atol=None):
    from ..tensor.type import TensorType
    expected, value = np.asarray(expected), np.asarray(value)
    if expected.dtype != value.dtype:           # compare in the wider of the two, as the reference's _allclose does
        wide = np.promote_types(expected.dtype, value.dtype)
        expected, value = expected.astype(wide), value.astype(wide)
    if not TensorType.values_eq_approx(expected, value, rtol, atol):
        raise WrongValue(expected, value, rtol, atol)
