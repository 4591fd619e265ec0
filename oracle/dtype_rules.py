"""TEST INFRASTRUCTURE - not part of the product.  Only ``tests/``, the
``cpu_baseline`` leg of ``bench.py`` and ``__graft_entry__.smoke()`` may import
anything under ``oracle/``.

The output dtype every scalar op gives for given input dtypes, restated from the
reference on its own, so that a graph's dtypes are checked against something other than
the product's ``make_node``.  Keyed by the scalar op's class name.

Each op of the reference is instantiated with an output-type policy
(``theano/scalar/basic.py:1659-3761``, ``theano/scalar/basic_scipy.py:60-857``,
``theano/tensor/nnet/sigm.py:167, 233, 370``, ``theano/tensor/nnet/nnet.py:2514``,
``theano/tensor/elemwise.py:2082``) or overrides ``output_types``
(``basic.py:1228, 1260, 1513, 1524, 1536, 1891, 2422, 2472, 3699``); the policies themselves are
``basic.py:836-1019`` and the promotion they rest on is ``basic.py:59-87``.

Pinned by tests/test_oracle_dtype_rules.py against what the reference's own tests state: int8 into
a float-only op gives what float32 gives and int8 / int8 gives floatX
(``theano/scalar/tests/test_basic.py:264-362``), comparisons and isnan give bool
(``theano/tensor/tests/test_basic.py:3069-3079``), exp of int32 is float64 and of complex128 is
complex128 (``:4879-4887``), and + - * / // on every pair of dtypes give what NumPy's arrays give
(``:6923-7010``), with NumPy itself as the judge there; promotion is checked to be a lattice join.
"""
import numpy as np

DISCRETE = ("bool", "int8", "int16", "int32", "int64", "uint8", "uint16", "uint32", "uint64")
INTEGER = DISCRETE[1:]
FLOAT = ("float16", "float32", "float64")
COMPLEX = ("complex64", "complex128")
ALL = DISCRETE + FLOAT + COMPLEX


class Refused(TypeError):
    """The reference raises TypeError for these input dtypes."""


def promote(dtypes, floatX="float64", cast_policy="custom"):
    """basic.py:59-87: NumPy's promotion folded over the operands from the left (it is not
    associative: int8, uint8, float16 give float32, float16, int8, uint8 give float16), narrowed back
    to floatX under the 'numpy+floatX' policy when no operand asked for the wider float."""
    acc = np.dtype(dtypes[0])
    for d in dtypes[1:]:
        acc = np.promote_types(acc, np.dtype(d))
    out = str(acc)
    if cast_policy == "numpy+floatX":
        if floatX == "float32" and out == "float64" and "float64" not in dtypes:
            return "float32"
        if floatX == "float16" and out in ("float64", "float32") and "float64" not in dtypes \
                and (out == "float64" or "float32" not in dtypes):
            return "float16"
    return out


_TO_FLOAT = dict(bool="float32", int8="float32", int16="float32", int32="float64", int64="float64",
                 uint8="float32", uint16="float32", uint32="float64", uint64="float64")    # basic.py:861-869


def _no_complex(ts):
    if any(t in COMPLEX for t in ts):
        raise Refused("complex")


def upcast_out(ts, **kw):
    return promote(ts, **kw)


def upcast_out_nobool(ts, **kw):                      # basic.py:841
    out = promote(ts, **kw)
    if out == "bool":
        raise Refused("bool output")
    return out


def upcast_out_min8(ts, **kw):                        # basic.py:848
    out = promote(ts, **kw)
    return "int8" if out == "bool" else out


def upcast_out_no_complex(ts, **kw):                  # basic.py:897
    _no_complex(ts)
    return promote(ts, **kw)


def upgrade_to_float(ts, **kw):                       # basic.py:855
    return promote([_TO_FLOAT.get(t, t) for t in ts], **kw)


def upgrade_to_float_no_complex(ts, **kw):            # basic.py:957
    _no_complex(ts)
    return upgrade_to_float(ts, **kw)


def upgrade_to_float64(ts, **kw):                     # basic.py:874
    return "float64"


def same_out(ts, **kw):
    return ts[0]


def same_out_nobool(ts, **kw):                        # basic.py:885
    if ts[0] == "bool":
        raise Refused("bool input")
    return ts[0]


def same_out_min8(ts, **kw):                          # basic.py:891
    return "int8" if ts[0] == "bool" else ts[0]


def same_out_float_only(ts, **kw):                    # basic.py:903
    if ts[0] not in FLOAT:
        raise Refused("float only")
    return ts[0]


def real_out(ts, **kw):                               # basic.py:1013
    return {"complex64": "float32", "complex128": "float64"}.get(ts[0], ts[0])


def _bool_out(ts, **kw):                              # basic.py:1228, 1260
    return "bool"


def _second(ts, **kw):                                # transfer_type(1), basic.py:2294
    return ts[1]


def _switch(ts, **kw):                                # basic.py:1513
    return promote(ts[1:], **kw)


def _unary_bit(ts, **kw):                             # basic.py:1524
    if ts[0] not in DISCRETE:
        raise Refused("bit op on a non-integer")
    return ts[0]


def _binary_bit(ts, **kw):                            # basic.py:1536
    if ts[0] == "bool" and ts[1] == "bool":
        return "bool"
    if any(t not in INTEGER for t in ts):
        raise Refused("bit op on a non-integer or on a bool beside an integer")
    return promote(ts, **kw)


def _true_div(ts, floatX="float64", **kw):            # basic.py:1891
    if all(t in DISCRETE for t in ts):
        return floatX
    return promote(ts, floatX=floatX, **kw)


def _abs(ts, **kw):                                   # basic.py:2422
    return real_out(ts)


def _sgn(ts, **kw):                                   # basic.py:2472
    if ts[0] == "bool":
        raise Refused("bool")
    _no_complex(ts)
    return ts[0]


def _angle(ts, **kw):                                 # specific_out(float64), basic.py:3694
    return "float64"


def _complex(ts, **kw):                               # basic.py:3699, 3742
    _no_complex(ts)
    return "complex128" if promote(ts) in ("float64", "int64", "uint64", "int32", "uint32") else "complex64"


RULES = {}
for _n in "Maximum Minimum Add Mul IntDiv Mod MulWithoutZeros".split():
    RULES[_n] = upcast_out
RULES.update(Sub=upcast_out_nobool, Pow=upcast_out_min8, Clip=upcast_out_no_complex, TrueDiv=_true_div,
             Second=_second, Identity=same_out, Sqr=same_out, Abs=_abs, Sgn=_sgn, Neg=same_out_nobool,
             RoundHalfToEven=same_out_float_only, RoundHalfAwayFromZero=same_out_float_only,
             Real=real_out, Imag=real_out, Angle=_angle, Conj=same_out_min8, Complex=_complex,
             ComplexFromPolar=_complex, Switch=_switch, Invert=_unary_bit, Chi2SF=upgrade_to_float64)
for _n in "LT GT LE GE EQ NEQ IsNan IsInf InRange".split():
    RULES[_n] = _bool_out
for _n in "OR XOR AND".split():
    RULES[_n] = _binary_bit
for _n in "Ceil Floor Trunc Erfc Erfcx Erfinv Erfcinv".split():
    RULES[_n] = upgrade_to_float_no_complex
for _n in ("Inv Log Log2 Log10 Log1p Exp Exp2 Expm1 Sqrt Deg2Rad Rad2Deg Cos ArcCos Sin ArcSin Tan ArcTan ArcTan2 "
           "Cosh ArcCosh Sinh ArcSinh Tanh ArcTanh Erf Gamma GammaLn Psi TriGamma GammaInc GammaIncC GammaU GammaL "
           "Jv J1 J0 Iv I1 I0 ScalarSigmoid UltraFastScalarSigmoid ScalarSoftplus ScalarSoftsign").split():
    RULES[_n] = upgrade_to_float


def out_dtype(class_name, in_dtypes, floatX="float64", cast_policy="custom"):
    """Output dtype of the reference's op of that class for these input dtypes; raises Refused where
    the reference raises TypeError and KeyError for a class the reference does not have."""
    return RULES[class_name](list(in_dtypes), floatX=floatX, cast_policy=cast_policy)


def check_node(op, in_dtypes, out_dtypes, floatX="float64", cast_policy="custom"):
    """Assert one scalar application's output dtype (Cast states its own target; classes the
    reference does not have are skipped)."""
    name = type(op).__name__
    if name == "Cast" or name not in RULES:
        return
    want = out_dtype(name, in_dtypes, floatX, cast_policy)
    assert list(out_dtypes) == [want], "%s%s gives %s, the reference gives %s" % (
        name, tuple(in_dtypes), list(out_dtypes), want)
