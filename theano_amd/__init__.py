"""theano_amd — Theano's fused Elemwise / CAReduce path on one AMD MI355X.

Graphs are built with Theano's Op protocol (``theano_amd.tensor``), differentiated
with ``grad`` and compiled with ``function``, which lifts Elemwise / Composite /
CAReduce / DimShuffle nodes onto HIP ops backed by ``libthx_hip.so``.
"""
from .config import config  # noqa: F401
from . import gof, scalar, tensor  # noqa: F401
from .gradient import grad, Lop, Rop  # noqa: F401
from .compile import CheckModeError, NanGuardError, UnusedInputError, function, In, Out, shared  # noqa: F401
