"""The ``*_inplace`` elementwise operations of ``theano/tensor/inplace.py``: each is the Elemwise
of the scalar op of the same name whose result takes the type of the first operand
(``transfer_type(0)``) and overwrites it (``inplace_pattern {0: 0}``, ``:8-18``).

A graph that holds one compiles with ``function(..., accept_inplace=True)`` only, as in the
reference (``theano/compile/function_module.py:183-190``).  The compiled function computes the
same values out of place - every other reader of the overwritten variable sees its old value,
the order the reference's DestroyHandler enforces - and, when the overwritten variable is an
argument of the function, stores the result into that argument after the call, which is what a
caller of the reference observes (``theano/tensor/tests/test_basic.py:653-657``)."""
from .. import scalar as scal
from .elemwise import Elemwise

_NAMES = (
    # comparisons and bit operations
    "lt", "gt", "le", "ge", "eq", "neq", "and_", "or_", "xor", "invert",
    # unary arithmetic and rounding
    "abs_", "exp", "exp2", "expm1", "neg", "inv", "log", "log1p", "log2", "log10", "sgn", "ceil", "floor", "trunc",
    "round_half_to_even", "round_half_away_from_zero", "sqr", "sqrt", "deg2rad", "rad2deg",
    # circular and hyperbolic functions
    "cos", "arccos", "sin", "arcsin", "tan", "arctan", "arctan2", "cosh", "arccosh", "sinh", "arcsinh", "tanh",
    "arctanh",
    # special functions
    "erf", "erfc", "erfcx", "gamma", "gammaln", "psi", "tri_gamma", "chi2sf", "j0", "j1", "jv", "i0", "i1", "iv",
    # binary arithmetic
    "second", "maximum", "minimum", "add", "sub", "mul", "true_div", "int_div", "mod", "pow", "conj",
)


def _inplace(name):
    scalar_op = getattr(scal, name)
    full = name + "_inplace"
    return Elemwise(scalar_op.make_new_inplace(scal.transfer_type(0), name=full), {0: 0}, name=full)


for _n in _NAMES:
    globals()[_n + "_inplace"] = _inplace(_n)
del _n

__all__ = [n + "_inplace" for n in _NAMES] + ["transpose_inplace"]


def transpose_inplace(x, **kwargs):
    """The transpose as a view of ``x``'s storage (``theano/tensor/inplace.py:382-387``)."""
    from .type import as_tensor_variable
    x = as_tensor_variable(x)
    return x.dimshuffle(*reversed(range(x.type.ndim)))
