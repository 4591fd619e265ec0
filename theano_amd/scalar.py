"""Scalar type system and per-element operations.

Mirrors ``theano/scalar/basic.py``: dtype algebra (``upcast`` :59-87, output
type policies :836-1019), the ScalarOps with their C semantics (:1214-3100),
``Composite`` (:3764-4127) and the thresholded sigmoid / softplus of
``theano/tensor/nnet/sigm.py:29-88, 330-372``.  ``c_code`` returns the statement
executed per element inside a device functor; its text is the normative
definition of each op here exactly as the C snippets are in the reference.
float16 values are computed in float32 (what ``Compositef32``
:4130-4208 arranges for the reference's device code).
"""
import builtins
import hashlib
import math

import numpy as np

from . import gof
from .config import config
from .gof import Apply, Constant, MethodNotDefined, Op, Type, Variable

float_dtypes = ("float16", "float32", "float64")
int_dtypes = ("int8", "int16", "int32", "int64")
uint_dtypes = ("uint8", "uint16", "uint32", "uint64")
integer_dtypes = int_dtypes + uint_dtypes
discrete_dtypes = ("bool",) + integer_dtypes
complex_dtypes = ("complex64", "complex128")
continuous_dtypes = float_dtypes + complex_dtypes
all_dtypes = discrete_dtypes + float_dtypes + complex_dtypes

# dtype -> (ABI code, storage C type, compute C type)
_DTYPE_INFO = {
    "bool": (0, "thx_bool", "thx_bool"), "int8": (1, "thx_i8", "thx_i8"), "uint8": (2, "thx_u8", "thx_u8"),
    "int16": (3, "thx_i16", "thx_i16"), "uint16": (4, "thx_u16", "thx_u16"), "int32": (5, "thx_i32", "thx_i32"),
    "uint32": (6, "thx_u32", "thx_u32"), "int64": (7, "thx_i64", "thx_i64"), "uint64": (8, "thx_u64", "thx_u64"),
    "float16": (9, "thx_f16", "thx_f32"), "float32": (10, "thx_f32", "thx_f32"), "float64": (11, "thx_f64", "thx_f64"),
    "complex64": (12, "thx_c64", "thx_c64"), "complex128": (13, "thx_c128", "thx_c128"),
}


def dtype_code(dtype):
    return _DTYPE_INFO[str(dtype)][0]


def storage_ctype(dtype):
    return _DTYPE_INFO[str(dtype)][1]


def compute_ctype(dtype):
    return _DTYPE_INFO[str(dtype)][2]


def upcast(dtype, *dtypes):
    """Result dtype of mixing the given dtypes: NumPy array promotion.  Under cast_policy
    'numpy+floatX' a float64 (float32) that NumPy's promotion alone produced - no operand was that
    wide - is narrowed to a float32 (float16) floatX (``theano/scalar/basic.py:59-87``)."""
    names = [str(np.dtype(dt)) for dt in (dtype,) + dtypes]
    z = np.zeros((), dtype=names[0])
    for dt in names[1:]:
        z = z + np.zeros((), dtype=dt)
    rval = str(z.dtype)
    if config.cast_policy == "numpy+floatX":
        if config.floatX == "float32" and rval == "float64" and "float64" not in names:
            return "float32"
        if (config.floatX == "float16" and rval in ("float64", "float32") and "float64" not in names and
                "float32" not in names):
            return "float16"
    return rval


class IntegerDivisionError(Exception):
    pass


class ComplexError(NotImplementedError):
    """An operation that complex numbers do not have (``theano/scalar/basic.py:43-48``)."""


# --------------------------------------------------------------------------
class Scalar(Type):
    """Type of one number of a given dtype (``theano/scalar/basic.py:293-416``)."""

    def __init__(self, dtype):
        if dtype == "floatX":
            dtype = config.floatX
        dtype = str(np.dtype(dtype)) if dtype != "bool" else "bool"
        if dtype not in _DTYPE_INFO:
            raise TypeError("unsupported dtype for a Scalar: %s" % dtype)
        self.dtype = dtype

    def filter(self, data, strict=False, allow_downcast=None):
        return np.asarray(data, dtype=self.dtype)[()]

    def __eq__(self, other):
        return type(self) is type(other) and self.dtype == other.dtype

    def __hash__(self):
        return hash(("Scalar", self.dtype))

    def __str__(self):
        return self.dtype

    __repr__ = __str__

    @staticmethod
    def upcast(*types):
        return upcast(*[getattr(t, "dtype", t) for t in types])


def get_scalar_type(dtype):
    return Scalar(dtype)


bool_ = Scalar("bool")
int8, int16, int32, int64 = Scalar("int8"), Scalar("int16"), Scalar("int32"), Scalar("int64")
uint8, uint16, uint32, uint64 = Scalar("uint8"), Scalar("uint16"), Scalar("uint32"), Scalar("uint64")
float16, float32, float64 = Scalar("float16"), Scalar("float32"), Scalar("float64")
complex64, complex128 = Scalar("complex64"), Scalar("complex128")


# the type tuples and constructors of theano/scalar/basic.py:679-687, 818-833
int_types, uint_types = (int8, int16, int32, int64), (uint8, uint16, uint32, uint64)
float_types, complex_types = (float16, float32, float64), (complex64, complex128)
integer_types = int_types + uint_types
discrete_types = (bool_,) + integer_types
continuous_types = float_types + complex_types
all_types = discrete_types + continuous_types


def _multi(scalar_type):
    """``ints("a b")``-style constructors: one variable for one name, a list for several."""
    def make(*names):
        if len(names) == 1 and isinstance(names[0], str) and " " in names[0]:
            names = tuple(names[0].split())
        made = [scalar_type(n) for n in names]
        return made[0] if len(made) == 1 else made
    return make


ints, floats = _multi(int64), _multi(float64)
complexs = complexs128 = _multi(complex128)
complexs64 = _multi(complex64)


def as_common_dtype(*vars):
    """The variables (scalar or tensor) cast to the upcast of their dtypes (``theano/scalar/basic.py:90-95``)."""
    dtype = upcast(*[v.type.dtype for v in vars])
    return tuple(v.astype(dtype) for v in vars)


class _scalar_py_operators(object):
    """Operator overloads so that gradient formulas read like arithmetic."""

    dtype = property(lambda self: self.type.dtype)

    def __abs__(self): return abs_(self)
    def __neg__(self): return neg(self)
    def __invert__(self): return invert(self)
    def __and__(self, o): return and_(self, o)
    def __or__(self, o): return or_(self, o)
    def __xor__(self, o): return xor(self, o)
    def __rand__(self, o): return and_(o, self)
    def __ror__(self, o): return or_(o, self)
    def __rxor__(self, o): return xor(o, self)
    def __lt__(self, o): return lt(self, o)
    def __gt__(self, o): return gt(self, o)
    def __le__(self, o): return le(self, o)
    def __ge__(self, o): return ge(self, o)
    def __add__(self, o): return add(self, o)
    def __sub__(self, o): return sub(self, o)
    def __mul__(self, o): return mul(self, o)
    def __truediv__(self, o): return div_proxy(self, o)
    __div__ = __truediv__
    def __floordiv__(self, o): return int_div(self, o)
    def __mod__(self, o): return mod_check(self, o)
    def __pow__(self, o): return pow(self, o)
    def __radd__(self, o): return add(o, self)
    def __rsub__(self, o): return sub(o, self)
    def __rmul__(self, o): return mul(o, self)
    def __rtruediv__(self, o): return div_proxy(o, self)
    __rdiv__ = __rtruediv__
    def __rfloordiv__(self, o): return int_div(o, self)
    def __rmod__(self, o): return mod(o, self)
    def __rpow__(self, o): return pow(o, self)

    def zeros_like(self, dtype=None):
        # a zero that still depends on self, as theano/scalar/basic.py:789-799
        if dtype is None:
            dtype = self.type.dtype
        return second(self, ScalarConstant(Scalar(dtype), np.asarray(0, dtype=dtype)[()]))

    def ones_like(self, dtype=None):
        if dtype is None:
            dtype = self.type.dtype
        return second(self, ScalarConstant(Scalar(dtype), np.asarray(1, dtype=dtype)[()]))

    def astype(self, dtype):
        return cast(self, dtype)


class ScalarVariable(_scalar_py_operators, Variable):
    pass


class ScalarConstant(_scalar_py_operators, Constant):
    def signature(self):
        return (self.type, np.asarray(self.data).tobytes())


Scalar.Variable = ScalarVariable
Scalar.Constant = ScalarConstant


def _autocast(x):
    """dtype chosen for a Python literal (``NumpyAutocaster``,
    ``theano/scalar/basic.py:132-214``).  cast_policy 'numpy' takes NumPy's choice, 'numpy+floatX' too except
    that a Python float becomes floatX; the rest of the function is the 'custom' policy."""
    if isinstance(x, (bool, np.bool_)):
        return np.asarray(x, dtype="bool")
    if config.cast_policy in ("numpy", "numpy+floatX"):
        if config.cast_policy == "numpy+floatX" and isinstance(x, float) and not hasattr(x, "dtype"):
            return np.asarray(x, dtype=config.floatX)
        return np.asarray(x)
    if isinstance(x, (int, np.integer)) and not hasattr(x, "dtype"):
        for dt in int_dtypes:
            try:
                x_ = np.asarray(x, dtype=dt)
            except OverflowError:
                continue
            if x_ == x:
                return x_
        return np.asarray(x, dtype="uint64")
    if isinstance(x, float):
        if config.floatX != "float64":
            return np.asarray(x, dtype=config.floatX)
        x_ = None
        for dt in ("float32", "float64"):
            x_ = np.asarray(x, dtype=dt)
            if x_ == x or (x != x):
                break
        return x_
    return np.asarray(x)


def convert(x, dtype=None):
    """Typed NumPy value of ``x`` under the casting policy
    (``theano/scalar/basic.py:252-290``)."""
    if dtype is not None:
        return np.asarray(x, dtype=config.floatX if dtype == "floatX" else dtype)
    if isinstance(x, (bool, int, float, np.bool_)) and not isinstance(x, np.generic):
        return _autocast(x)
    if isinstance(x, np.generic):
        return np.asarray(x)
    if isinstance(x, np.ndarray):
        return x
    x_ = np.asarray(x)
    if x_.size == 0 and not hasattr(x, "dtype"):
        x_ = np.asarray(x, dtype=config.floatX)
    elif x_.dtype == np.float64 and config.floatX != "float64" and not hasattr(x, "dtype"):
        pass  # lists of Python floats keep NumPy's float64, as in the reference
    return x_


def constant(x, name=None, dtype=None):
    x = convert(x, dtype=dtype)
    if x.ndim != 0:
        raise TypeError("scalar.constant needs a 0-d value")
    return ScalarConstant(Scalar(str(x.dtype)), x[()], name=name)


def as_scalar(x, name=None):
    if isinstance(x, Apply):
        x = x.default_output()
    if isinstance(x, Variable):
        if isinstance(x.type, Scalar):
            return x
        raise TypeError("not a scalar variable: %s" % (x,))
    return constant(x, name=name)


# --------------------------------------------------------------------------
# output type policies (theano/scalar/basic.py:836-1019)
def upcast_out(*types):
    return (Scalar(Scalar.upcast(*types)),)


def upcast_out_nobool(*types):
    t = upcast_out(*types)
    if t[0] == bool_:
        raise TypeError("bool output not supported")
    return t


def upcast_out_min8(*types):
    t = upcast_out(*types)
    return (int8,) if t[0] == bool_ else t


_TO_FLOAT = {"bool": "float32", "int8": "float32", "int16": "float32", "int32": "float64", "int64": "float64",
             "uint8": "float32", "uint16": "float32", "uint32": "float64", "uint64": "float64"}


def upgrade_to_float(*types):
    return (Scalar(upcast(*[_TO_FLOAT.get(t.dtype, t.dtype) for t in types])),)


def same_out(t):
    return (t,)


def _no_complex(types, what="complex argument not supported"):
    if any(t.dtype in complex_dtypes for t in types):
        raise TypeError(what)


def upcast_out_no_complex(*types):
    _no_complex(types, "complex type are not supported")
    return upcast_out(*types)


def upgrade_to_float_no_complex(*types):
    _no_complex(types)
    return upgrade_to_float(*types)


def real_out(t):
    """The type of one component: float32 for complex64, float64 for complex128, the type itself
    otherwise (``theano/scalar/basic.py:1008-1019``)."""
    return ({"complex64": float32, "complex128": float64}.get(t.dtype, t),)


def int_out(*types):
    return (int64,)


def float_out(*types):
    return (float64,)


def same_out_nocomplex(t):
    _no_complex([t])
    return (t,)


def int_out_nocomplex(*types):
    _no_complex(types)
    return (int64,)


def float_out_nocomplex(*types):
    _no_complex(types)
    return (float64,)


def same_out_nobool(t):
    if t == bool_:
        raise TypeError("bool input not supported")
    return (t,)


def same_out_min8(t):
    return (int8,) if t == bool_ else (t,)


def same_out_float_only(t):
    if t.dtype not in float_dtypes:
        raise TypeError("only float type are supported")
    return (t,)


class transfer_type(object):
    """Output i takes the type of input ``transfer[i]`` (None: the upcast)."""

    def __init__(self, *transfer):
        self.transfer = transfer

    def __eq__(self, other):
        return type(self) is type(other) and self.transfer == other.transfer

    def __hash__(self):
        return hash(("transfer_type", self.transfer))

    def __call__(self, *types):
        up = upcast_out(*types)[0]
        return [up if i is None else (Scalar(i) if isinstance(i, str) else types[i]) for i in self.transfer]


class specific_out(object):
    def __init__(self, *spec):
        self.spec = spec

    def __eq__(self, other):
        return type(self) is type(other) and self.spec == other.spec

    def __hash__(self):
        return hash(("specific_out", self.spec))

    def __call__(self, *types):
        return self.spec


# --------------------------------------------------------------------------
def _fn(name, dtype):
    """libm-style function name for the compute type of ``dtype``; helpers of
    the kernel prelude (``thx_*``) are overloaded instead."""
    return name if compute_ctype(dtype) == "thx_f64" or name.startswith("thx_") else name + "f"


def c_literal(value, dtype):
    """Device source text of a constant of the given dtype."""
    dtype = str(dtype)
    if dtype == "bool":
        return "((thx_bool)%d)" % (1 if value else 0)
    if dtype in complex_dtypes:
        v = builtins.complex(np.asarray(value, dtype=dtype))
        part = "float32" if dtype == "complex64" else "float64"
        return "%s(%s, %s)" % (compute_ctype(dtype), c_literal(v.real, part), c_literal(v.imag, part))
    if dtype in float_dtypes:
        v = float(np.asarray(value, dtype=dtype))
        ct = compute_ctype(dtype)
        if math.isnan(v):
            return "((%s)NAN)" % ct
        if math.isinf(v):
            return "((%s)%sINFINITY)" % (ct, "-" if v < 0 else "")
        if ct == "thx_f64":
            return "(%r)" % v
        return "(%rf)" % v
    v = int(value)
    if dtype == "int64":
        if v == -(1 << 63):
            return "(-9223372036854775807LL - 1)"
        return "(%dLL)" % v
    if dtype == "uint64":
        return "(%dULL)" % v
    if dtype == "uint32":
        return "(%dU)" % v
    if dtype == "int32":
        if v == -(1 << 31):
            return "(-2147483647 - 1)"
        return "(%d)" % v
    return "((%s)%d)" % (storage_ctype(dtype), v)


class ScalarOp(Op):
    """Base of per-element operations (``theano/scalar/basic.py:1022-1198``)."""

    nin = -1
    nout = 1
    identity = None
    commutative = False
    associative = False
    __props__ = ("output_types_preference",)

    def __init__(self, output_types_preference=None, name=None):
        self.name = name
        if output_types_preference is not None:
            self.output_types_preference = output_types_preference
        elif not hasattr(self, "output_types_preference"):
            self.output_types_preference = None

    def _props(self):
        return (self.output_types_preference,)

    def __str__(self):
        return self.name if getattr(self, "name", None) else type(self).__name__

    __repr__ = __str__

    def output_types(self, types):
        pref = self.output_types_preference
        if pref is None:
            raise MethodNotDefined("output_types", type(self))
        variables = pref(*types)
        if len(variables) != self.nout:
            raise TypeError("%s: expected %d outputs, policy gave %d" % (self, self.nout, len(variables)))
        return list(variables)

    def make_node(self, *inputs):
        if self.nin >= 0 and len(inputs) != self.nin:
            raise TypeError("%s takes %d inputs, got %d" % (self, self.nin, len(inputs)))
        inputs = [as_scalar(i) for i in inputs]
        outputs = [t() for t in self.output_types([i.type for i in inputs])]
        if len(outputs) != self.nout:
            raise TypeError("wrong number of outputs")
        return Apply(self, inputs, outputs)

    def c_code(self, node, inputs, outputs):
        """Statement computing ``outputs`` (names) from ``inputs`` (expressions)."""
        raise MethodNotDefined("c_code", type(self))

    def supports_c_code(self, inputs, outputs):
        try:
            node = Apply(self, inputs, [o.clone() for o in outputs])
            self.c_code(node, ["x"] * len(inputs), ["z"] * len(outputs))
        except (MethodNotDefined, NotImplementedError):
            return False
        return True

    def make_new_inplace(self, output_types_preference=None, name=None):
        return type(self)(output_types_preference, name)


class UnaryScalarOp(ScalarOp):
    nin = 1


class BinaryScalarOp(ScalarOp):
    nin = 2


def _zero_grads(inputs):
    return [i.zeros_like(dtype=config.floatX) if i.type.dtype in discrete_dtypes else i.zeros_like() for i in inputs]


# ---- comparisons (theano/scalar/basic.py:1214-1431) ---------------------------
class LogicalComparison(BinaryScalarOp):
    def output_types(self, types):
        return [bool_]

    def L_op(self, inputs, outputs, gout):
        return [i.zeros_like(dtype=config.floatX) for i in inputs]


def _cmp(name, sym):
    class _C(LogicalComparison):
        def c_code(self, node, inputs, outputs):
            if any(i.type.dtype in complex_dtypes for i in node.inputs):
                if sym not in ("==", "!="):
                    raise NotImplementedError("complex numbers have no order (theano/scalar/basic.py:1280-1350)")
                ct = compute_ctype(upcast(*[i.type.dtype for i in node.inputs]))
                return "%s = ((%s)%s %s (%s)%s);" % (outputs[0], ct, inputs[0], sym, ct, inputs[1])
            return "%s = (%s %s %s);" % (outputs[0], inputs[0], sym, inputs[1])
    _C.__name__ = _C.__qualname__ = name      # instances pickle by reference to the module-level name
    _C.commutative = sym in ("==", "!=")
    return _C


LT, GT, LE, GE, EQ, NEQ = (_cmp("LT", "<"), _cmp("GT", ">"), _cmp("LE", "<="), _cmp("GE", ">="),
                           _cmp("EQ", "=="), _cmp("NEQ", "!="))
lt, gt, le, ge, eq, neq = LT(name="lt"), GT(name="gt"), LE(name="le"), GE(name="ge"), EQ(name="eq"), NEQ(name="neq")


class FixedLogicalComparison(UnaryScalarOp):
    def output_types(self, types):
        return [bool_]

    def L_op(self, inputs, outputs, gout):
        return [inputs[0].zeros_like(dtype=config.floatX)]


class IsNan(FixedLogicalComparison):
    def c_code(self, node, inputs, outputs):
        if node.inputs[0].type.dtype in discrete_dtypes:
            return "%s = 0;" % outputs[0]
        if node.inputs[0].type.dtype in complex_dtypes:
            return "%s = (isnan(%s.re) || isnan(%s.im)) ? 1 : 0;" % (outputs[0], inputs[0], inputs[0])
        return "%s = isnan(%s) ? 1 : 0;" % (outputs[0], inputs[0])


class IsInf(FixedLogicalComparison):
    def c_code(self, node, inputs, outputs):
        if node.inputs[0].type.dtype in discrete_dtypes:
            return "%s = 0;" % outputs[0]
        if node.inputs[0].type.dtype in complex_dtypes:
            return "%s = (isinf(%s.re) || isinf(%s.im)) ? 1 : 0;" % (outputs[0], inputs[0], inputs[0])
        return "%s = isinf(%s) ? 1 : 0;" % (outputs[0], inputs[0])


isnan, isinf = IsNan(name="isnan"), IsInf(name="isinf")


class InRange(ScalarOp):
    """``low < x < hi`` with either end open or closed (``theano/scalar/basic.py:1434-1481``)."""
    nin = 3
    __props__ = ("openlow", "openhi")

    def __init__(self, openlow, openhi, name=None):
        ScalarOp.__init__(self, None, name)
        self.openlow, self.openhi = bool(openlow), bool(openhi)

    def _props(self):
        return (self.openlow, self.openhi)

    def output_types(self, types):
        return [bool_]

    def c_code(self, node, inputs, outputs):
        if any(i.type.dtype in complex_dtypes for i in node.inputs):
            raise NotImplementedError("complex numbers have no order (theano/scalar/basic.py:1280-1350)")
        x, low, hi = inputs
        return "%s = (%s %s %s && %s %s %s);" % (outputs[0], x, ">" if self.openlow else ">=", low,
                                                 x, "<" if self.openhi else "<=", hi)

    def L_op(self, inputs, outputs, gout):
        if any(i.type.dtype in complex_dtypes for i in inputs):
            raise NotImplementedError("no gradient of InRange for complex numbers")
        return _zero_grads(inputs)

    def make_new_inplace(self, output_types_preference=None, name=None):
        return type(self)(self.openlow, self.openhi, name)


inopenrange = InRange(True, True, name="inopenrange")
inclosedrange = InRange(False, False, name="inclosedrange")


class Switch(ScalarOp):
    nin = 3

    def output_types(self, types):
        return list(upcast_out(types[1], types[2]))

    def c_code(self, node, inputs, outputs):
        ot = node.outputs[0].type.dtype
        if node.inputs[0].type.dtype in complex_dtypes:
            raise NotImplementedError("switch on a complex condition")
        if ot in complex_dtypes:
            ct = compute_ctype(ot)
            return "%s = %s ? (%s)%s : (%s)%s;" % (outputs[0], inputs[0], ct, inputs[1], ct, inputs[2])
        return "%s = %s ? %s : %s;" % (outputs[0], inputs[0], inputs[1], inputs[2])

    def L_op(self, inputs, outputs, gout):
        cond, ift, iff = inputs
        (gz,) = gout
        if outputs[0].type.dtype in discrete_dtypes:
            first, secnd = ift.zeros_like(dtype=config.floatX), iff.zeros_like(dtype=config.floatX)
        else:
            first, secnd = switch(cond, gz, 0.0), switch(cond, 0.0, gz)
        return [cond.zeros_like(dtype=config.floatX), first, secnd]


switch = Switch(name="switch")


# ---- bit operations (theano/scalar/basic.py:1523-1617) ------------------------
class UnaryBitOp(UnaryScalarOp):
    def output_types(self, types):
        for t in types:
            if t.dtype not in discrete_dtypes:
                raise TypeError("input to a BitOp must have type (u)int8, (u)int16, (u)int32 or (u)int64 or bool "
                                "not %s" % t)
        return list(upcast_out(*types))

    def L_op(self, inputs, outputs, gout):
        return [inputs[0].zeros_like(dtype=config.floatX)]


class BinaryBitOp(BinaryScalarOp):
    commutative = True
    associative = True

    def output_types(self, types):
        t0, t1 = types
        if t0 == bool_ and t1 == bool_:
            return [bool_]
        for t in types:
            if t.dtype not in integer_dtypes:
                raise TypeError("input to a BitOp must have type (u)int8, (u)int16, (u)int32 or (u)int64 or be all "
                                "bools not %s" % t)
        return list(upcast_out(*types))

    def L_op(self, inputs, outputs, gout):
        return [i.zeros_like(dtype=config.floatX) for i in inputs]

    def c_code(self, node, inputs, outputs):
        return "%s = (%s %s %s);" % (outputs[0], inputs[0], self.symbol, inputs[1])


class OR(BinaryBitOp):
    identity = 0
    symbol = "|"


class XOR(BinaryBitOp):
    identity = 0
    symbol = "^"


class AND(BinaryBitOp):
    identity = -1
    symbol = "&"


class RightShift(BinaryBitOp):
    """Arithmetic ``x >> y``.  The reference has no shift op; for signed
    two's-complement operands this equals ``int_div(x, 2**y)``
    (``theano/scalar/basic.py:1960-2025``), which is what pins it."""
    commutative = False
    associative = False
    symbol = ">>"

    def output_types(self, types):
        for t in types:
            if t.dtype not in integer_dtypes:
                raise TypeError("shift operands must be integers, not %s" % t)
        return list(upcast_out(*types))


class LeftShift(RightShift):
    symbol = "<<"


class Invert(UnaryBitOp):
    def c_code(self, node, inputs, outputs):
        if node.outputs[0].type == bool_:
            return "%s = (!%s);" % (outputs[0], inputs[0])
        return "%s = (~%s);" % (outputs[0], inputs[0])


or_, xor, and_, invert = OR(name="or_"), XOR(name="xor"), AND(name="and_"), Invert(name="invert")
right_shift, left_shift = RightShift(name="right_shift"), LeftShift(name="left_shift")


# ---- max / min (theano/scalar/basic.py:1623-1696) ------------------------------
class Maximum(BinaryScalarOp):
    commutative = True
    associative = True

    def c_code(self, node, inputs, outputs):
        x, y = inputs
        if node.outputs[0].type.dtype in complex_dtypes:
            raise NotImplementedError("maximum / minimum of complex numbers (theano/scalar/basic.py:1635, 1674)")
        return self._pick(node, x, y, outputs[0], ">", ">=")

    @staticmethod
    def _pick(node, x, y, z, first, then):
        """``z = y OP x ? y : (x OP= y ? x : nan(""))`` (theano/scalar/basic.py:1637-1639): both comparisons, so
        that a NaN on either side gives NaN, made in C's common type of the operands.  The reference's ``nan("")``
        makes the whole expression a double, so the operand that wins arrives in ``z`` as the value it is (an int8
        of -128 beside a uint32 stays -128): each branch is converted to the result type here, which says the
        same without the detour - and without the rounding to 53 bits that the detour gives 64-bit integers."""
        out = node.outputs[0].type.dtype
        if out in float_dtypes:
            # the NaN in the result's own arithmetic type: a float NAN beside integer operands (int32 beside
            # uint64 gives a float64 node) would make the expression a float and round the operands to 24 bits
            nan = "NAN" if all(i.type.dtype in float_dtypes for i in node.inputs) else "((%s)NAN)" % compute_ctype(out)
            return "%s = ((%s) %s (%s) ? (%s) : ((%s) %s (%s) ? (%s) : %s));" % (z, y, first, x, y, x, then, y, x, nan)
        ct = storage_ctype(out) if out != "bool" else "bool"
        return "%s = ((%s) %s (%s) ? (%s)(%s) : (%s)(%s));" % (z, y, first, x, ct, y, ct, x)

    def L_op(self, inputs, outputs, gout):
        x, y = inputs
        (gz,) = gout
        if outputs[0].type.dtype in discrete_dtypes:
            return [x.zeros_like(dtype=config.floatX), y.zeros_like(dtype=config.floatX)]
        e = eq(outputs[0], x)
        return [e * gz, (constant(1, dtype=gz.type.dtype) - e) * gz]


class Minimum(Maximum):
    def c_code(self, node, inputs, outputs):
        x, y = inputs
        if node.outputs[0].type.dtype in complex_dtypes:
            raise NotImplementedError("maximum / minimum of complex numbers (theano/scalar/basic.py:1635, 1674)")
        return self._pick(node, x, y, outputs[0], "<", "<=")


maximum, minimum = Maximum(upcast_out, name="maximum"), Minimum(upcast_out, name="minimum")


# ---- arithmetic (theano/scalar/basic.py:1699-2261) ------------------------------
def _to_complex_result(node, inputs):
    """Operand expressions converted to the result type when that is complex: every operand is
    widened first and the operation runs in the result type, as NumPy's loops do (the reference's
    C mixes types through overloads, ``theano/scalar/basic.py:584-631``)."""
    ot = node.outputs[0].type.dtype
    if ot not in complex_dtypes:
        return list(inputs)
    ct = compute_ctype(ot)
    return ["(%s)%s" % (ct, i) for i in inputs]


def _wrapping(fn, operands):
    """``a op b op c`` from left to right through the library's wrapping helper: signed integer results that
    leave their range wrap as NumPy's do instead of being undefined (kernels/thx_common.h)."""
    expr = operands[0]
    for o in operands[1:]:
        expr = "%s(%s, %s)" % (fn, expr, o)
    return expr if len(operands) > 1 else "(%s)" % expr


class Add(ScalarOp):
    identity = 0
    commutative = True
    associative = True

    def c_code(self, node, inputs, outputs):
        if node.outputs[0].type.dtype in int_dtypes and inputs:
            return "%s = %s;" % (outputs[0], _wrapping("thx_wadd", inputs))
        sym = " || " if node.outputs[0].type == bool_ else " + "
        inputs = _to_complex_result(node, inputs)
        return "%s = %s;" % (outputs[0], sym.join(inputs) if inputs else "0")

    def L_op(self, inputs, outputs, gout):
        (gz,) = gout
        if outputs[0].type.dtype in discrete_dtypes:
            return [i.zeros_like(dtype=config.floatX) for i in inputs]
        return [gz for _ in inputs]


class Mul(ScalarOp):
    identity = 1
    commutative = True
    associative = True

    def c_code(self, node, inputs, outputs):
        if node.outputs[0].type.dtype in int_dtypes and inputs:
            return "%s = %s;" % (outputs[0], _wrapping("thx_wmul", inputs))
        sym = " && " if node.outputs[0].type == bool_ else " * "
        inputs = _to_complex_result(node, inputs)
        return "%s = %s;" % (outputs[0], sym.join(inputs) if inputs else "1")

    def L_op(self, inputs, outputs, gout):
        (gz,) = gout
        if outputs[0].type.dtype in discrete_dtypes:
            return [i.zeros_like(dtype=config.floatX) for i in inputs]
        return [mul(*([gz] + [o for j, o in enumerate(inputs) if j != k])) for k in range(len(inputs))]


class Sub(BinaryScalarOp):
    def c_code(self, node, inputs, outputs):
        if node.outputs[0].type.dtype in int_dtypes:
            return "%s = thx_wsub(%s, %s);" % (outputs[0], inputs[0], inputs[1])
        inputs = _to_complex_result(node, inputs)
        return "%s = %s - %s;" % (outputs[0], inputs[0], inputs[1])

    def L_op(self, inputs, outputs, gout):
        (gz,) = gout
        if outputs[0].type.dtype in discrete_dtypes:
            return [i.zeros_like(dtype=config.floatX) for i in inputs]
        return [gz, -gz]


add, mul, sub = Add(upcast_out, name="add"), Mul(upcast_out, name="mul"), Sub(upcast_out_nobool, name="sub")


class MulWithoutZeros(BinaryScalarOp):
    """Product that skips zeros: the combiner of ProdWithoutZeros, which the
    gradient of Prod uses for groups holding exactly one zero
    (``theano/tensor/elemwise.py:2054-2083``).  Its identity is 0, not 1, so
    that a group of zeros reduces to 0."""

    identity = 0
    commutative = True
    associative = True

    def c_code(self, node, inputs, outputs):
        x, y = inputs
        return "%s = ((%s == 0) ? (%s) : ((%s == 0) ? (%s) : ((%s) * (%s))));" % (outputs[0], x, y, y, x, y, x)


mul_without_zeros = MulWithoutZeros(upcast_out, name="mul_without_zeros")


def int_or_true_div(x_discrete, y_discrete):
    """Which division ``x / y`` means (``theano/scalar/basic.py:1826-1873``)."""
    if x_discrete and y_discrete:
        if config.int_division == "raise":
            raise IntegerDivisionError("dividing two integer types with '/' is forbidden by config.int_division; "
                                       "use // or cast one argument to float")
        if config.int_division == "int":
            return int_div
        return true_div
    return true_div


def div_proxy(x, y):
    x, y = as_scalar(x), as_scalar(y)
    return int_or_true_div(x.type.dtype in discrete_dtypes, y.type.dtype in discrete_dtypes)(x, y)


class TrueDiv(BinaryScalarOp):
    def output_types(self, types):
        if all(t.dtype in discrete_dtypes for t in types):
            return [Scalar(config.floatX)]
        return BinaryScalarOp.output_types(self, types)

    def c_code(self, node, inputs, outputs):
        if all(i.type.dtype in discrete_dtypes for i in node.inputs):
            return "%s = ((double)%s) / %s;" % (outputs[0], inputs[0], inputs[1])
        if node.outputs[0].type.dtype in complex_dtypes:
            x, y = _to_complex_result(node, inputs)
            return "%s = %s / %s;" % (outputs[0], x, y)
        if node.outputs[0].type.dtype in ("float16", "float32"):
            # single-precision division goes through the device helper (a plain `/` unless the
            # library was asked for the 2.5-ulp form); the reference's text is `x / y`
            return "%s = thx_fdiv(%s, %s);" % (outputs[0], inputs[0], inputs[1])
        return "%s = %s / %s;" % (outputs[0], inputs[0], inputs[1])

    def L_op(self, inputs, outputs, gout):
        x, y = inputs
        (gz,) = gout
        if all(i.type.dtype in discrete_dtypes for i in inputs):
            return [x.zeros_like(), y.zeros_like()]
        return [gz / y, -(gz * x) / (y * y)]


true_div = TrueDiv(upcast_out, name="true_div")


class IntDiv(BinaryScalarOp):
    """Floor division with Python's sign rule; the four sign cases are spelled
    out because C division truncates (``theano/scalar/basic.py:1960-2025``).
    Integer division by zero cannot raise on the device: like the reference's
    ``#ifdef KERNEL`` branch the hardware result is stored."""

    def c_code(self, node, inputs, outputs):
        x, y = inputs
        (z,) = outputs
        t = upcast(*[i.type.dtype for i in node.inputs])
        if t in complex_dtypes:
            raise ComplexError("floor division (//) is not defined for complex numbers (theano/scalar/basic.py:1947-1949)")
        if t in discrete_dtypes:
            d = lambda a, b: "(%s / %s)" % (a, b)
            m = lambda a, b: "(%s %% %s)" % (a, b)
            zero = "%s = 0;" % z
        else:
            # the quotient must be the correctly rounded one whatever division the kernels are
            # built with: floor() of a quotient that is an ulp low loses a whole unit
            fl, fm = _fn("floor", t), _fn("fmod", t)
            d = lambda a, b: "%s(thx_exact_div(%s, %s))" % (fl, a, b)
            m = lambda a, b: "%s(%s, %s)" % (fm, a, b)
            zero = "%s = %s;" % (z, d(x, y))
        # integer negations and the final subtraction wrap (the most negative value is its own negative)
        neg = (lambda a: "thx_wneg(%s)" % a) if t in discrete_dtypes else (lambda a: "(-%s)" % a)
        less = (lambda a, b: "thx_wsub(%s, %s)" % (a, b)) if t in discrete_dtypes else (lambda a, b: "%s - %s" % (a, b))
        nx, ny = neg(x), neg(y)
        return ("if (%(y)s == 0) { %(zero)s } "
                "else if (%(y)s < 0) { if (%(x)s < 0) { %(z)s = %(mm)s; } "
                "else { %(z)s = %(a)s; } } "
                "else { if (%(x)s < 0) { %(z)s = %(b)s; } "
                "else { %(z)s = %(pp)s; } }") % dict(
                    x=x, y=y, z=z, zero=zero, mm=d(nx, ny), pp=d(x, y),
                    a=less(neg(d(x, ny)), "((%s == 0) ? 0 : 1)" % m(x, ny)),
                    b=less(neg(d(nx, y)), "((%s == 0) ? 0 : 1)" % m(nx, y)))

    def L_op(self, inputs, outputs, gout):
        return [i.zeros_like(dtype=config.floatX) for i in inputs]


int_div = IntDiv(upcast_out, name="int_div")
floor_div = int_div


class Mod(BinaryScalarOp):
    """Remainder with the sign of the divisor (``theano/scalar/basic.py:2048-2147``)."""

    def c_code(self, node, inputs, outputs):
        x, y = inputs
        (z,) = outputs
        t = upcast(*[i.type.dtype for i in node.inputs])
        if t in complex_dtypes:
            raise ComplexError("the mod operator (%) is not defined for complex numbers (theano/scalar/basic.py:2050-2052)")
        if t in discrete_dtypes:
            m = lambda a, b: "(%s %% %s)" % (a, b)
            zero = "%s = 0;" % z
        else:
            # the reference calls the double overload whatever the input type
            m = lambda a, b: "fmod((double)%s, (double)%s)" % (a, b)
            zero = "%s = %s;" % (z, m(x, y))
        integer = t in discrete_dtypes
        neg = (lambda a: "thx_wneg(%s)" % a) if integer else (lambda a: "(-%s)" % a)
        plus = (lambda a, b: "thx_wadd(%s, %s)" % (a, b)) if integer else (lambda a, b: "%s + %s" % (a, b))
        nx, ny = neg(x), neg(y)
        mm, pm, mp, pp = m(nx, ny), m(x, ny), m(nx, y), m(x, y)
        return ("if (%(y)s == 0) { %(zero)s } "
                "else if (%(y)s < 0) { if (%(x)s < 0) { %(z)s = %(a)s; } "
                "else { %(z)s = %(b)s; } } "
                "else { if (%(x)s < 0) { %(z)s = %(c)s; } "
                "else { %(z)s = %(pp)s; } }") % dict(
                    x=x, y=y, z=z, zero=zero, pp=pp, a=neg(mm),
                    b=plus("(%s)" % pm, "(%s != 0 ? %s : 0)" % (pm, y)),
                    c=plus(neg(mp), "(%s != 0 ? %s : 0)" % (mp, y)))

    def L_op(self, inputs, outputs, gout):
        x, y = inputs
        (gz,) = gout
        if outputs[0].type.dtype in discrete_dtypes:
            return [i.zeros_like(dtype=config.floatX) for i in inputs]
        return [gz, -(x // y) * gz]


mod = Mod(upcast_out, name="mod")


def mod_check(x, y):
    """``x % y`` of the operators: refuses complex operands when the graph is built
    (``theano/scalar/basic.py:2038-2045``)."""
    x, y = as_scalar(x), as_scalar(y)
    if x.type.dtype in complex_dtypes or y.type.dtype in complex_dtypes:
        raise ComplexError("the mod operator (%) is not defined for complex numbers (theano/scalar/basic.py:2050-2052)")
    return mod(x, y)


class Pow(BinaryScalarOp):
    def c_code(self, node, inputs, outputs):
        # C's pow(): arguments promote to double
        (x, y), (z,) = inputs, outputs
        if node.outputs[0].type.dtype in complex_dtypes:
            x, y = _to_complex_result(node, inputs)
            return "%s = thx_cpow(%s, %s);" % (z, x, y)
        if node.outputs[0].type.dtype in discrete_dtypes:
            # The host libm the reference runs on returns whole powers of whole numbers exactly, and the
            # conversion to the integer result truncates.  The device's pow may come out one place short
            # (pow(3, 1) = 2.9999999999999996 would truncate to 2): round powers with exponents >= 0, which
            # are whole; negative exponents give at most 1/2 in magnitude beyond |base| = 1 and still truncate.
            ct = storage_ctype(node.outputs[0].type.dtype)
            return ("{ const double thx_p = pow((double)%s, (double)%s); %s = ((double)%s < 0) ? (%s)thx_p : (%s)rint(thx_p); }"
                    % (x, y, z, y, ct, ct))
        return "%s = pow((double)%s, (double)%s);" % (z, x, y)

    def L_op(self, inputs, outputs, gout):
        x, y = inputs
        (gz,) = gout
        if outputs[0].type.dtype in discrete_dtypes:
            return [i.zeros_like(dtype=config.floatX) for i in inputs]
        first = gz * y * x ** (y - 1)
        secnd = switch(eq(x, 0), 0, gz * log(x) * x ** y)
        return [first, secnd]


pow = Pow(upcast_out_min8, name="pow")


class Clip(ScalarOp):
    nin = 3

    def output_types(self, types):
        return list(upcast_out_no_complex(*types))

    def c_code(self, node, inputs, outputs):
        x, lo, hi = inputs
        return "%s = %s < %s ? %s : %s > %s ? %s : %s;" % (outputs[0], x, lo, lo, x, hi, hi, x)

    def L_op(self, inputs, outputs, gout):
        x, mn, mx = inputs
        (gz,) = gout
        if outputs[0].type.dtype in integer_dtypes:
            return [i.zeros_like(dtype=config.floatX) for i in inputs]
        return [((x >= mn) & (x <= mx)) * gz, (x < mn) * gz, (x > mx) * gz]


clip = Clip(name="clip")


class Second(BinaryScalarOp):
    """``second(x, y) = y``; only the shape of ``x`` matters at tensor level."""

    def c_code(self, node, inputs, outputs):
        return "%s = %s;" % (outputs[0], inputs[1])

    def connection_pattern(self, node):
        return [[False], [True]]

    def L_op(self, inputs, outputs, gout):
        x, y = inputs
        (gz,) = gout
        if y.type.dtype in continuous_dtypes:
            return [DisconnectedType()(), gz]
        return [DisconnectedType()(), y.zeros_like()]


second = Second(transfer_type(1), name="second")


class Identity(UnaryScalarOp):
    def c_code(self, node, inputs, outputs):
        return "%s = %s;" % (outputs[0], inputs[0])

    def L_op(self, inputs, outputs, gout):
        if inputs[0].type.dtype in continuous_dtypes:
            return [gout[0]]
        return [inputs[0].zeros_like(dtype=config.floatX)]


identity = Identity(same_out, name="identity")


class Cast(UnaryScalarOp):
    def __init__(self, o_type, name=None):
        if not isinstance(o_type, Scalar):
            raise TypeError(o_type)
        UnaryScalarOp.__init__(self, specific_out(o_type), name=name)
        self.o_type = o_type

    def __str__(self):
        return "Cast{%s}" % self.o_type.dtype

    def make_new_inplace(self, output_types_preference=None, name=None):
        return type(self)(self.o_type, name)

    def c_code(self, node, inputs, outputs):
        if node.outputs[0].type == bool_:
            return "%s = (%s) ? 1 : 0;" % (outputs[0], inputs[0])
        return "%s = (%s)%s;" % (outputs[0], compute_ctype(node.outputs[0].type.dtype), inputs[0])

    def L_op(self, inputs, outputs, gout):
        if self.o_type.dtype in continuous_dtypes:
            return [gout[0]]
        return [inputs[0].zeros_like(dtype=config.floatX)]


_cast_mapping = dict((dt, Cast(Scalar(dt), name="convert_to_" + dt)) for dt in all_dtypes)
# convert_to_bool ... convert_to_complex128, the module-level names of theano/scalar/basic.py:2403-2417
globals().update(("convert_to_" + dt, op) for dt, op in _cast_mapping.items())


def cast(x, dtype):
    if dtype == "floatX":
        dtype = config.floatX
    x = as_scalar(x)
    dtype = str(dtype)
    if x.type.dtype == dtype:
        return x
    if x.type.dtype in complex_dtypes and dtype not in complex_dtypes:
        raise TypeError("Casting from complex to real is ambiguous: consider real(), imag(), angle() or abs()")
    return _cast_mapping[dtype](x)


class Abs(UnaryScalarOp):
    def output_types(self, types):
        # the modulus of a complex number is real (theano/scalar/basic.py:2421-2430)
        return list(real_out(types[0]))

    def c_code(self, node, inputs, outputs):
        t = node.inputs[0].type.dtype
        (x,), (z,) = inputs, outputs
        if t in complex_dtypes:
            return "%s = thx_cabs(%s);" % (z, x)
        if t in int_dtypes:
            return "%s = thx_wabs(%s);" % (z, x)        # abs of the most negative value wraps to itself
        if t in float_dtypes:
            return "%s = %s(%s);" % (z, _fn("fabs", t), x)
        return "%s = %s;" % (z, x)  # bool and unsigned

    def L_op(self, inputs, outputs, gout):
        (x,) = inputs
        if outputs[0].type.dtype in discrete_dtypes:
            return [x.zeros_like(dtype=config.floatX)]
        if x.type.dtype in complex_dtypes:
            return [gout[0] * x / abs_(x)]       # theano/scalar/basic.py:2447
        return [gout[0] * sgn(x)]


abs_ = Abs(same_out, name="abs_")


class Sgn(UnaryScalarOp):
    def output_types(self, types):
        if types[0] == bool_:
            raise TypeError(types[0])
        _no_complex(types, "complex has no sgn")
        return [types[0]]

    def c_code(self, node, inputs, outputs):
        t = node.inputs[0].type.dtype
        (x,), (z,) = inputs, outputs
        if t in float_dtypes:
            return "%s = (%s > 0) ? 1. : ((%s < 0) ? -1. : (isnan(%s) ? NAN : 0.));" % (z, x, x, x)
        if t in int_dtypes:
            return "%s = (%s >= 0) ? (%s == 0) ? 0 : 1 : -1;" % (z, x, x)
        return "%s = (%s == 0) ? 0 : 1;" % (z, x)

    def L_op(self, inputs, outputs, gout):
        return _zero_grads(inputs)


sgn = Sgn(name="sgn")


def _unary_math(cname, fname, grad_fn, policy=upgrade_to_float):
    """A libm call on the input cast to the output type, the shape every unary
    math op has in the reference (e.g. ``Exp`` ``theano/scalar/basic.py:2919-2952``)."""
    class _U(UnaryScalarOp):
        def c_code(self, node, inputs, outputs):
            ot = node.outputs[0].type.dtype
            if ot in complex_dtypes:
                if fname not in _COMPLEX_MATH:
                    raise NotImplementedError("%s has no device code for complex numbers" % fname)
                return "%s = thx_c%s((%s)%s);" % (outputs[0], fname, compute_ctype(ot), inputs[0])
            fn = _fn(fname, ot)
            if fn == "expf":
                fn = "thx_fexp"        # expf, or exp2 of x * log2(e) in the 2.5-ulp build
            elif fn == "sqrtf":
                fn = "thx_fsqrt"       # sqrtf, or one hardware sqrt in the 2.5-ulp build: the same bits in every kernel
            return "%s = %s((%s)%s);" % (outputs[0], fn, compute_ctype(ot), inputs[0])

        def L_op(self, inputs, outputs, gout):
            (x,) = inputs
            if outputs[0].type.dtype in discrete_dtypes:
                return [x.zeros_like(dtype=config.floatX)]
            if outputs[0].type.dtype in complex_dtypes:
                raise NotImplementedError("gradient of %s for complex numbers (the reference has none either)" % fname)
            if grad_fn is None:
                return _zero_grads(inputs)
            return [grad_fn(x, outputs[0], gout[0])]
    _U.__name__ = _U.__qualname__ = cname
    globals()[cname] = _U            # importable by name: instances pickle by reference to their class
    return _U(policy, name=fname if fname != "fabs" else "abs")


# the functions with a complex form among the device helpers
_COMPLEX_MATH = ("exp", "expm1", "log", "log2", "log10", "log1p", "sqrt", "sin", "cos", "tan", "sinh", "cosh", "tanh")

ceil = _unary_math("Ceil", "ceil", None, upgrade_to_float_no_complex)
floor = _unary_math("Floor", "floor", None, upgrade_to_float_no_complex)
log = _unary_math("Log", "log", lambda x, z, gz: gz / x)
log2 = _unary_math("Log2", "log2", lambda x, z, gz: gz / (x * math.log(2.0)))
log10 = _unary_math("Log10", "log10", lambda x, z, gz: gz / (x * math.log(10.0)))
log1p = _unary_math("Log1p", "log1p", lambda x, z, gz: gz / (1 + x))
exp = _unary_math("Exp", "exp", lambda x, z, gz: gz * z)
exp2 = _unary_math("Exp2", "exp2", lambda x, z, gz: gz * z * math.log(2.0))
expm1 = _unary_math("Expm1", "expm1", lambda x, z, gz: gz * exp(x))
sqrt = _unary_math("Sqrt", "sqrt", lambda x, z, gz: (gz * 0.5) / z)
cos = _unary_math("Cos", "cos", lambda x, z, gz: -gz * sin(x))
sin = _unary_math("Sin", "sin", lambda x, z, gz: gz * cos(x))
tan = _unary_math("Tan", "tan", lambda x, z, gz: gz / sqr(cos(x)))
arccos = _unary_math("ArcCos", "acos", lambda x, z, gz: -gz / sqrt(1 - sqr(x)))
arcsin = _unary_math("ArcSin", "asin", lambda x, z, gz: gz / sqrt(1 - sqr(x)))
arctan = _unary_math("ArcTan", "atan", lambda x, z, gz: gz / (1 + sqr(x)))
cosh = _unary_math("Cosh", "cosh", lambda x, z, gz: gz * sinh(x))
sinh = _unary_math("Sinh", "sinh", lambda x, z, gz: gz * cosh(x))
tanh = _unary_math("Tanh", "tanh", lambda x, z, gz: gz * (1 - sqr(z)))
arccosh = _unary_math("ArcCosh", "acosh", lambda x, z, gz: gz / sqrt(sqr(x) - 1))
arcsinh = _unary_math("ArcSinh", "asinh", lambda x, z, gz: gz / sqrt(sqr(x) + 1))
arctanh = _unary_math("ArcTanh", "atanh", lambda x, z, gz: gz / (1 - sqr(x)))

# Special functions (``theano/scalar/basic_scipy.py:29-391``): the device math library has the
# error and gamma functions; digamma and trigamma are helpers of the kernel prelude.
_TWO_OVER_SQRT_PI = 2.0 / math.sqrt(math.pi)
erf = _unary_math("Erf", "erf", lambda x, z, gz: gz * _TWO_OVER_SQRT_PI * exp(-x * x))
erfc = _unary_math("Erfc", "erfc", lambda x, z, gz: -gz * _TWO_OVER_SQRT_PI * exp(-x * x))
erfcx = _unary_math("Erfcx", "erfcx", lambda x, z, gz: gz * (-_TWO_OVER_SQRT_PI + (2.0 * x) * z))
erfinv = _unary_math("Erfinv", "erfinv", lambda x, z, gz: gz * (1.0 / _TWO_OVER_SQRT_PI) * exp(z * z))
erfcinv = _unary_math("Erfcinv", "erfcinv", lambda x, z, gz: -gz * (1.0 / _TWO_OVER_SQRT_PI) * exp(z * z))
gamma = _unary_math("Gamma", "tgamma", lambda x, z, gz: gz * z * psi(x))
gammaln = _unary_math("GammaLn", "lgamma", lambda x, z, gz: gz * psi(x))
psi = _unary_math("Psi", "thx_psi", lambda x, z, gz: gz * tri_gamma(x))
tri_gamma = _unary_math("TriGamma", "thx_trigamma", None)
# Bessel functions (``theano/scalar/basic_scipy.py:714-857``); J1' and I1' are written through the
# recurrences J1' = J0 - J1 / x and I1' = I0 - I1 / x (the reference's (J0 - J2) / 2 and (I0 + I2) / 2)
j0 = _unary_math("J0", "j0", lambda x, z, gz: -gz * j1(x))
j1 = _unary_math("J1", "j1", lambda x, z, gz: gz * switch(eq(x, 0), 0.5, j0(x) - z / x))
i0 = _unary_math("I0", "thx_i0", lambda x, z, gz: gz * i1(x))
i1 = _unary_math("I1", "thx_i1", lambda x, z, gz: gz * switch(eq(x, 0), 0.5, i0(x) - z / x))


def upgrade_to_float64(*types):
    """Always float64 (``theano/scalar/basic.py:914-920``)."""
    return (float64,)


class _IncompleteGamma(BinaryScalarOp):
    """Regularized incomplete gamma functions and their relatives
    (``theano/scalar/basic_scipy.py:482-711``), evaluated by the kernel prelude's helpers in
    double precision.  Not differentiable, as in the reference."""

    expr = None

    def c_code(self, node, inputs, outputs):
        a, b = ["((double)%s)" % i for i in inputs]
        return "%s = %s;" % (outputs[0], self.expr % dict(a=a, b=b))


class GammaInc(_IncompleteGamma):           # P(k, x)
    expr = "thx_gammainc(%(a)s, %(b)s)"


class GammaIncC(_IncompleteGamma):          # Q(k, x)
    expr = "thx_gammaincc(%(a)s, %(b)s)"


class GammaU(_IncompleteGamma):             # upper incomplete gamma: Q(k, x) * gamma(k)
    expr = "thx_gammaincc(%(a)s, %(b)s) * tgamma(%(a)s)"


class GammaL(_IncompleteGamma):             # lower incomplete gamma: P(k, x) * gamma(k)
    expr = "thx_gammainc(%(a)s, %(b)s) * tgamma(%(a)s)"


class Chi2SF(_IncompleteGamma):             # chi-square survival function of x with k degrees of freedom
    expr = "thx_gammaincc(0.5 * %(b)s, 0.5 * %(a)s)"


gammainc, gammaincc = GammaInc(upgrade_to_float, name="gammainc"), GammaIncC(upgrade_to_float, name="gammaincc")
gammau, gammal = GammaU(upgrade_to_float, name="gammau"), GammaL(upgrade_to_float, name="gammal")
chi2sf = Chi2SF(upgrade_to_float64, name="chi2sf")


class Trunc(UnaryScalarOp):
    def c_code(self, node, inputs, outputs):
        ot = node.outputs[0].type.dtype
        fl = _fn("floor", ot)
        (x,) = inputs
        return "%s = %s >= 0 ? %s(%s) : -%s(-%s);" % (outputs[0], x, fl, x, fl, x)

    def L_op(self, inputs, outputs, gout):
        return [inputs[0].zeros_like(dtype=config.floatX)]


trunc = Trunc(upgrade_to_float, name="trunc")


class _AngleUnit(UnaryScalarOp):
    """``x * factor`` with the factor a double constant, as the reference's C text has it: an
    integer or float32 operand is multiplied in double precision and rounded to the result type
    once (``theano/scalar/basic.py:3086-3150``)."""
    factor = 1.0

    def c_code(self, node, inputs, outputs):
        if node.inputs[0].type.dtype in complex_dtypes:
            raise NotImplementedError("%s of a complex number" % self)
        return "%s = %s * (%r);" % (outputs[0], inputs[0], self.factor)

    def L_op(self, inputs, outputs, gout):
        (x,) = inputs
        (gz,) = gout
        if gz.type.dtype in complex_dtypes:
            raise NotImplementedError("gradient of %s for complex numbers" % self)
        if outputs[0].type.dtype in discrete_dtypes:
            return _zero_grads(inputs)
        return [gz * self.factor]


class Deg2Rad(_AngleUnit):
    factor = math.pi / 180.0


class Rad2Deg(_AngleUnit):
    factor = 180.0 / math.pi


deg2rad = Deg2Rad(upgrade_to_float, name="deg2rad")
rad2deg = Rad2Deg(upgrade_to_float, name="rad2deg")


class RoundHalfToEven(UnaryScalarOp):
    def c_code(self, node, inputs, outputs):
        ot = node.outputs[0].type.dtype
        return "%s = %s(%s);" % (outputs[0], _fn("rint", ot), inputs[0])

    def L_op(self, inputs, outputs, gout):
        return _zero_grads(inputs)


class RoundHalfAwayFromZero(UnaryScalarOp):
    def c_code(self, node, inputs, outputs):
        ot = node.outputs[0].type.dtype
        return "%s = %s(%s);" % (outputs[0], _fn("round", ot), inputs[0])

    def L_op(self, inputs, outputs, gout):
        return _zero_grads(inputs)


round_half_to_even = RoundHalfToEven(same_out_float_only, name="round_half_to_even")
round_half_away_from_zero = RoundHalfAwayFromZero(same_out_float_only, name="round_half_away_from_zero")


class Neg(UnaryScalarOp):
    def c_code(self, node, inputs, outputs):
        if node.outputs[0].type.dtype in int_dtypes:
            return "%s = thx_wneg(%s);" % (outputs[0], inputs[0])
        return "%s = -%s;" % (outputs[0], inputs[0])

    def L_op(self, inputs, outputs, gout):
        if outputs[0].type.dtype in discrete_dtypes:
            return [inputs[0].zeros_like(dtype=config.floatX)]
        return [-gout[0]]


neg = Neg(same_out_nobool, name="neg")


class Inv(UnaryScalarOp):
    def c_code(self, node, inputs, outputs):
        if node.outputs[0].type.dtype in ("float16", "float32"):
            # the reference's `1.0 / x` is a double division rounded to float; on the device the
            # single-precision helper gives the same value to within its 2.5 ulp
            return "%s = thx_fdiv(1.0f, %s);" % (outputs[0], inputs[0])
        return "%s = 1.0 / %s;" % (outputs[0], inputs[0])

    def L_op(self, inputs, outputs, gout):
        (x,) = inputs
        if outputs[0].type.dtype in discrete_dtypes:
            return [x.zeros_like(dtype=config.floatX)]
        return [-gout[0] / (x * x)]


inv = Inv(upgrade_to_float, name="inv")


class Sqr(UnaryScalarOp):
    def c_code(self, node, inputs, outputs):
        if node.outputs[0].type.dtype in int_dtypes:
            return "%s = thx_wmul(%s, %s);" % (outputs[0], inputs[0], inputs[0])
        return "%s = %s * %s;" % (outputs[0], inputs[0], inputs[0])

    def L_op(self, inputs, outputs, gout):
        (x,) = inputs
        if outputs[0].type.dtype in discrete_dtypes:
            return [x.zeros_like(dtype=config.floatX)]
        return [gout[0] * x * 2]


sqr = Sqr(same_out, name="sqr")


class ArcTan2(BinaryScalarOp):
    def c_code(self, node, inputs, outputs):
        ot = node.outputs[0].type.dtype
        ct = compute_ctype(ot)
        return "%s = %s((%s)%s, (%s)%s);" % (outputs[0], _fn("atan2", ot), ct, inputs[0], ct, inputs[1])

    def L_op(self, inputs, outputs, gout):
        y, x = inputs
        (gz,) = gout
        if outputs[0].type.dtype in discrete_dtypes:
            return [i.zeros_like(dtype=config.floatX) for i in inputs]
        den = sqr(x) + sqr(y)
        return [gz * x / den, -gz * y / den]


arctan2 = ArcTan2(upgrade_to_float, name="arctan2")


# ---- sigmoid / softplus (theano/tensor/nnet/sigm.py:29-88, 330-372) -------------
class ScalarSigmoid(UnaryScalarOp):
    """1/(1+exp(-x)) with the reference's saturation thresholds."""

    def c_code(self, node, inputs, outputs):
        t = node.inputs[0].type.dtype
        (x,), (z,) = inputs, outputs
        if t in discrete_dtypes:
            # The reference has C code for floating-point operands only and evaluates integers through its Python
            # ``impl`` (theano/tensor/nnet/sigm.py:36-46); here they are converted to the result's float type
            # (int8 -> float32, int32 -> float64: upgrade_to_float) and take that type's formula.
            t = node.outputs[0].type.dtype
            x = "((%s)%s)" % (compute_ctype(t), x)
        if t in ("float32", "float16"):
            return "%s = %s < -88.0f ? 0.0f : %s > 15.0f ? 1.0f : thx_sigmoid_core(%s);" % (z, x, x, x)
        if t == "float64":
            return "%s = %s < -709.0 ? 0.0 : %s > 19.0 ? 1.0 : 1.0 / (1.0 + exp(-%s));" % (z, x, x, x)
        raise NotImplementedError("only floating point is implemented")

    def L_op(self, inputs, outputs, gout):
        y = scalar_sigmoid(inputs[0])
        return [gout[0] * y * (1.0 - y)]


scalar_sigmoid = ScalarSigmoid(upgrade_to_float, name="scalar_sigmoid")


class ScalarSoftplus(UnaryScalarOp):
    def c_code(self, node, inputs, outputs):
        t = node.inputs[0].type.dtype
        (x,), (z,) = inputs, outputs
        if t in discrete_dtypes:           # as for the sigmoid: integers take the result type's formula
            t = node.outputs[0].type.dtype
            x = "((%s)%s)" % (compute_ctype(t), x)
        if t in ("float32", "float16"):
            return "%s = %s < -103.0f ? 0.0f : %s > 14.0f ? %s : log1pf(expf(%s));" % (z, x, x, x, x)
        if t == "float64":
            return "%s = %s < -745.0 ? 0.0 : %s > 16.0 ? %s : log1p(exp(%s));" % (z, x, x, x, x)
        raise NotImplementedError("only floating point is implemented")

    def L_op(self, inputs, outputs, gout):
        return [gout[0] * scalar_sigmoid(inputs[0])]


scalar_softplus = ScalarSoftplus(upgrade_to_float, name="scalar_softplus")


class SigmoidBinaryCrossentropy(BinaryScalarOp):
    """``softplus(-|x|) + x * ((x > 0) - t)``: the cross-entropy of ``sigmoid(x)`` against the probability
    ``t`` in its overflow-free form, with the gradients the reference attaches to that formula,
    ``sigmoid(x) - t`` and ``-x`` (theano/tensor/nnet/nnet.py:2028-2050; the formula's own derivative
    is off by one half at x = 0, where |x| has none)."""

    def c_code(self, node, inputs, outputs):
        ot = node.outputs[0].type.dtype
        ct = compute_ctype(ot)
        (x, t), (z,) = inputs, outputs
        lo = "-745.0" if ot == "float64" else "-103.0f"
        ex = _fn("exp", ot)
        ex = "thx_fexp" if ex == "expf" else ex
        return ("{ const %(ct)s thx_x = (%(ct)s)%(x)s; const %(ct)s thx_a = -%(fabs)s(thx_x); "
                "const %(ct)s thx_sp = thx_a < %(lo)s ? (%(ct)s)0 : %(log1p)s(%(exp)s(thx_a)); "
                "%(z)s = thx_sp + thx_x * ((%(ct)s)(thx_x > 0) - (%(ct)s)%(t)s); }") % dict(
                    ct=ct, x=x, t=t, z=z, lo=lo, fabs=_fn("fabs", ot), log1p=_fn("log1p", ot), exp=ex)

    def L_op(self, inputs, outputs, gout):
        x, t = inputs
        (gz,) = gout
        if outputs[0].type.dtype in discrete_dtypes:
            return [i.zeros_like(dtype=config.floatX) for i in inputs]
        return [gz * (scalar_sigmoid(x) - t), gz * (-x)]


sigmoid_binary_crossentropy = SigmoidBinaryCrossentropy(upgrade_to_float, name="sigmoid_binary_crossentropy")


class UltraFastScalarSigmoid(UnaryScalarOp):
    """0.5 * (t(0.5 * x) + 1) with a three-piece rational / linear / constant stand-in t for tanh
    (theano/tensor/nnet/sigm.py:179-230): a speed option, within 0.028 of the sigmoid.  As in the
    reference's C text the pieces are evaluated in double and rounded to the output type where the C
    code assigns to a variable of that type."""

    def c_code(self, node, inputs, outputs):
        (x,), (z,) = inputs, outputs
        ct = compute_ctype(node.outputs[0].type.dtype)
        piece = ("(%(v)s < 1.7 ? (1.5 * %(v)s / (1 + %(v)s)) : (%(v)s < 3 ? (0.935409070603099 + "
                 "0.0458812946797165 * (%(v)s - 1.7)) : 0.99505475368673))")
        return ("{ const %(ct)s thx_h = (%(ct)s)(0.5 * (double)%(x)s); const %(ct)s thx_m = -thx_h; %(ct)s thx_t; "
                "if (thx_h >= 0) thx_t = (%(ct)s)" + piece % {"v": "(double)thx_h"} + "; else thx_t = (%(ct)s)(-" +
                piece % {"v": "(double)thx_m"} + "); %(z)s = (%(ct)s)(0.5 * ((double)thx_t + 1.)); }") % dict(ct=ct, x=x, z=z)

    def L_op(self, inputs, outputs, gout):
        raise MethodNotDefined("grad", type(self))       # as in the reference: the op is put in after the gradient


ultra_fast_scalar_sigmoid = UltraFastScalarSigmoid(upgrade_to_float, name="ultra_fast_scalar_sigmoid")


class ScalarSoftsign(UnaryScalarOp):
    """x / (1 + |x|) (theano/tensor/nnet/nnet.py:2484-2516; the constant is a double in the C text)."""

    def c_code(self, node, inputs, outputs):
        (x,), (z,) = inputs, outputs
        if node.inputs[0].type.dtype not in ("float32", "float64"):
            raise NotImplementedError("only floating point x is implemented")
        ct = compute_ctype(node.outputs[0].type.dtype)
        return "%s = (%s)((double)%s / (1.0 + fabs((double)%s)));" % (z, ct, x, x)

    def L_op(self, inputs, outputs, gout):
        (x,) = inputs
        if x.type.dtype not in float_dtypes:
            raise NotImplementedError("softsign gradient: floating point only")
        d = 1.0 + abs_(x)
        return [gout[0] / (d * d)]


scalar_softsign = ScalarSoftsign(upgrade_to_float, name="scalar_softsign")


# --------------------------------------------------------------------------
class DisconnectedType(Type):
    """Type of the placeholder gradient for an input the cost does not depend
    on (``theano/gradient.py``)."""

    def filter(self, data, strict=False, allow_downcast=None):
        raise AssertionError("a disconnected gradient has no value")

    def __eq__(self, other):
        return type(self) is type(other)

    def __hash__(self):
        return hash("DisconnectedType")

    def __str__(self):
        return "DisconnectedType"


# ---- complex numbers (theano/scalar/basic.py:3623-3761) -----------------------------------
# The reference runs these five through NumPy on the host (none has C code there); here they are
# device code like every other op.
class Real(UnaryScalarOp):
    def c_code(self, node, inputs, outputs):
        if node.inputs[0].type.dtype in complex_dtypes:
            return "%s = %s.re;" % (outputs[0], inputs[0])
        return "%s = %s;" % (outputs[0], inputs[0])

    def L_op(self, inputs, outputs, gout):
        if inputs[0].type.dtype in complex_dtypes:
            return [complex(gout[0], 0)]
        return [gout[0]] if inputs[0].type.dtype in float_dtypes else _zero_grads(inputs)


class Imag(UnaryScalarOp):
    def c_code(self, node, inputs, outputs):
        if node.inputs[0].type.dtype in complex_dtypes:
            return "%s = %s.im;" % (outputs[0], inputs[0])
        return "%s = 0;" % outputs[0]

    def L_op(self, inputs, outputs, gout):
        (x,) = inputs
        if x.type.dtype in complex_dtypes:
            return [complex(0, gout[0])]
        return [second(x, 0)] if x.type.dtype in float_dtypes else _zero_grads(inputs)


class Angle(UnaryScalarOp):
    """Argument of a complex number, always float64 as in the reference
    (``theano/scalar/basic.py:3660-3693``; NumPy computes it in the precision of the input)."""

    def c_code(self, node, inputs, outputs):
        t = node.inputs[0].type.dtype
        if t in complex_dtypes:
            return "%s = thx_cangle(%s);" % (outputs[0], inputs[0])
        # np.angle of a real: 0 or pi (NaN stays), in the precision of the input
        if t in ("float16", "float32"):
            return "%s = atan2f(0.0f, (float)%s);" % (outputs[0], inputs[0])
        return "%s = atan2(0.0, (double)%s);" % (outputs[0], inputs[0])

    def L_op(self, inputs, outputs, gout):
        (c,) = inputs
        if c.type.dtype not in complex_dtypes:
            return [second(c, 0)] if c.type.dtype in float_dtypes else _zero_grads(inputs)
        # d theta = (x dy - y dx) / r^2
        x, y = real(c), imag(c)
        r2 = x * x + y * y
        return [cast(complex(-gout[0] * y / r2, gout[0] * x / r2), c.type.dtype)]


class Complex(BinaryScalarOp):
    def output_types(self, types):
        for t in types:
            if t.dtype in complex_dtypes:
                raise TypeError(t)
        up = upcast(*[t.dtype for t in types])
        return [complex128 if up in ("float64", "int64", "uint64", "int32", "uint32") else complex64]

    def c_code(self, node, inputs, outputs):
        ot = node.outputs[0].type.dtype
        part = "thx_f32" if ot == "complex64" else "thx_f64"
        return "%s = %s((%s)%s, (%s)%s);" % (outputs[0], compute_ctype(ot), part, inputs[0], part, inputs[1])

    def L_op(self, inputs, outputs, gout):
        x, y = inputs
        (gz,) = gout
        return [g if i.type.dtype in float_dtypes else i.zeros_like(dtype=config.floatX)
                for i, g in ((x, cast(real(gz), x.type.dtype)), (y, cast(imag(gz), y.type.dtype)))]


class Conj(UnaryScalarOp):
    def c_code(self, node, inputs, outputs):
        if node.inputs[0].type.dtype in complex_dtypes:
            return "%s = thx_cconj(%s);" % (outputs[0], inputs[0])
        return "%s = %s;" % (outputs[0], inputs[0])


class ComplexFromPolar(BinaryScalarOp):
    """``r (cos theta + i sin theta)``.  The reference's host implementation raises ValueError for a negative
    radius (``theano/scalar/basic.py:3746-3748``); device code cannot raise and stores the value the formula
    gives."""

    def output_types(self, types):
        return Complex.output_types(self, types)

    def c_code(self, node, inputs, outputs):
        ot = node.outputs[0].type.dtype
        part = "thx_f32" if ot == "complex64" else "thx_f64"
        return "%s = thx_cpolar((%s)%s, (%s)%s);" % (outputs[0], part, inputs[0], part, inputs[1])


real, imag = Real(real_out, name="real"), Imag(real_out, name="imag")
angle = Angle(specific_out(float64), name="angle")
complex = Complex(name="complex")
conj = Conj(same_out_min8, name="conj")
complex_from_polar = ComplexFromPolar(name="complex_from_polar")


# ---- Bessel functions of real order (theano/scalar/basic_scipy.py:698-726, 786-811) ------------
class _BesselOfOrder(BinaryScalarOp):
    """``scipy.special.jv`` / ``iv`` in the reference (host only); device helpers here, evaluated in
    double precision whatever the result type.  No gradient with respect to the order."""

    fn = None
    sign = None

    def c_code(self, node, inputs, outputs):
        _no_complex([i.type for i in node.inputs])
        return "%s = %s((double)%s, (double)%s);" % (outputs[0], self.fn, inputs[0], inputs[1])

    def L_op(self, inputs, outputs, gout):
        from .gradient import grad_not_implemented
        v, x = inputs
        (gz,) = gout
        if outputs[0].type.dtype in discrete_dtypes:
            return _zero_grads(inputs)
        me = type(self)(upgrade_to_float, name=self.name)
        lower, upper = me(v - 1, x), me(v + 1, x)
        return [grad_not_implemented(self, 0, v), gz * (lower + upper if self.sign > 0 else lower - upper) / 2.]


class Jv(_BesselOfOrder):
    fn, sign = "thx_jv", -1


class Iv(_BesselOfOrder):
    fn, sign = "thx_iv", 1


jv, iv = Jv(upgrade_to_float, name="jv"), Iv(upgrade_to_float, name="iv")


# --------------------------------------------------------------------------
class Composite(ScalarOp):
    """A scalar sub-graph as one op (``theano/scalar/basic.py:3764-4127``).

    The graph is cloned, nested Composites are inlined, constants are kept
    inside as literals, and the generated code string is the op's identity
    (eq / hash), as in the reference (:4085-4112)."""

    def __init__(self, inputs, outputs, name=None):
        for i in inputs:
            if not isinstance(i.type, Scalar):
                raise TypeError("Composite inputs must be scalar variables")
        inputs, outputs = gof.clone(list(inputs), list(outputs))
        # inline nested composites
        changed = True
        while changed:
            changed = False
            for node in gof.io_toposort(inputs, outputs):
                if isinstance(node.op, Composite):
                    inner = node.op
                    memo = dict(zip(inner.inputs, node.inputs))
                    memo = gof.clone_get_equiv([], inner.outputs, copy_inputs=False, memo=memo)
                    repl = dict(zip(node.outputs, [memo[o] for o in inner.outputs]))
                    outputs = [repl.get(o, o) for o in outputs]
                    for n2 in gof.io_toposort(inputs, outputs):
                        n2.inputs = [repl.get(i, i) for i in n2.inputs]
                    changed = True
                    break
        # equal ops on the same values are computed once (the merge of theano/scalar/basic.py:3915-3925)
        first, repl = {}, {}
        for node in gof.io_toposort(inputs, outputs):
            node.inputs = [repl.get(i, i) for i in node.inputs]
            operands = [("c", str(i.type), repr(i.data)) if isinstance(i, Constant) else ("v", id(i)) for i in node.inputs]
            if isinstance(node.op, (Add, Mul)):      # a * b and b * a are one value
                operands.sort()
            key = (node.op, tuple(operands))
            prev = first.setdefault(key, node)
            if prev is not node:
                repl.update(zip(node.outputs, prev.outputs))
        outputs = [repl.get(o, o) for o in outputs]
        self.inputs = inputs
        self.outputs = outputs
        self.inputs_type = tuple(i.type for i in inputs)
        self.outputs_type = tuple(o.type for o in outputs)
        self.nin = len(inputs)
        self.nout = len(outputs)
        self.name = name
        self.output_types_preference = None
        self._code = None

    # identity ----------------------------------------------------------------
    def body(self, innames, outnames, prefix="t"):
        """Statements computing ``outnames`` from ``innames``; temporaries are
        declared in the compute type of their dtype, in topological order."""
        names = dict(zip(self.inputs, innames))
        lines = []
        nodes = gof.io_toposort(self.inputs, self.outputs)
        counter = 0
        for node in nodes:
            args = []
            for i in node.inputs:
                if i in names:
                    args.append(names[i])
                elif isinstance(i, Constant):
                    args.append(c_literal(i.data, i.type.dtype))
                else:
                    raise ValueError("Composite graph uses a variable that is not an input: %s" % i)
            outs = []
            for o in node.outputs:
                nm = "%s%d" % (prefix, counter)
                counter += 1
                names[o] = nm
                outs.append(nm)
                lines.append("%s %s;" % (compute_ctype(o.type.dtype), nm))
            lines.append(node.op.c_code(node, args, outs))
        for o, nm in zip(self.outputs, outnames):
            if o in names:
                src = names[o]
            elif isinstance(o, Constant):
                src = c_literal(o.data, o.type.dtype)
            else:
                raise ValueError("Composite output is not computed from its inputs")
            lines.append("%s = %s;" % (nm, src))
        return "\n".join(lines)

    def code_signature(self):
        if self._code is None:
            self._code = self.body(["i%d" % k for k in range(self.nin)], ["o%d" % k for k in range(self.nout)])
        return self._code

    def __eq__(self, other):
        return (type(self) is type(other) and self.inputs_type == other.inputs_type and
                self.outputs_type == other.outputs_type and self.code_signature() == other.code_signature())

    def __hash__(self):
        return hash((type(self), self.inputs_type, self.outputs_type, self.code_signature()))

    def __str__(self):
        if self.name:
            return self.name
        names = dict((i, "i%d" % k) for k, i in enumerate(self.inputs))

        def show(v):
            if v in names:
                return names[v]
            if isinstance(v, Constant):
                return str(v.data)
            return "%s(%s)" % (v.owner.op, ", ".join(show(i) for i in v.owner.inputs))
        return "Composite{%s}" % ", ".join(show(o) for o in self.outputs)

    __repr__ = __str__

    # protocol ----------------------------------------------------------------
    def output_types(self, types):
        if tuple(types) != self.inputs_type:
            raise TypeError("Wrong types for Composite. Expected %s, got %s." % (self.inputs_type, tuple(types)))
        return list(self.outputs_type)

    def make_node(self, *inputs):
        inputs = [as_scalar(i) for i in inputs]
        if tuple(i.type for i in inputs) == self.inputs_type:
            return Apply(self, inputs, [t() for t in self.outputs_type])
        # rebuild for the new input types (theano/scalar/basic.py:3998-4015)
        new_ins = [i.type() for i in inputs]
        memo = dict(zip(self.inputs, new_ins))
        for node in gof.io_toposort(self.inputs, self.outputs):
            args = [memo.get(i, i) for i in node.inputs]
            new_node = node.op.make_node(*args)
            for o, no in zip(node.outputs, new_node.outputs):
                memo[o] = no
        op = Composite(new_ins, [memo.get(o, o) for o in self.outputs])
        return Apply(op, inputs, [t() for t in op.outputs_type])

    def clone_float32(self):
        """The same Composite with every float16 value computed in float32 (``Compositef32`` and
        ``Composite.clone_float32``, ``theano/scalar/basic.py:4130-4208``, what ``GpuElemwise`` hands to its
        kernel generator): float16 inputs and constants become float32, a cast from float32 to float16 and a
        cast of a float16 value to the type it now has disappear, any other cast to float16 becomes a cast to
        float32.  (The kernels here widen float16 on load and round on store, so the generated code of a
        float16 Composite already computes this way; the method is the reference's interface to that form.)"""
        mapping = {}
        for i in self.inputs:
            mapping[i] = float32() if i.type.dtype == "float16" else i.type()
        for node in gof.io_toposort(self.inputs, self.outputs):
            for i in node.inputs:
                if i not in mapping:
                    if not isinstance(i, Constant):
                        raise ValueError("Composite graph uses a variable that is not an input: %s" % i)
                    mapping[i] = constant(np.float32(i.data)) if i.type.dtype == "float16" else i
            out = node.outputs[0]
            if isinstance(node.op, Cast):
                inp = mapping[node.inputs[0]]
                to_half = node.op.o_type.dtype == "float16"
                if to_half and node.inputs[0].type.dtype == "float32":
                    mapping[out] = inp                      # float32 -> float16: gone
                    continue
                o_type = float32 if to_half else node.op.o_type
                src_is_half = inp.type.dtype == "float16" if to_half else node.inputs[0].type.dtype == "float16"
                if (to_half or src_is_half) and o_type == inp.type:
                    mapping[out] = inp                      # a cast to the type the value already has
                    continue
                mapping[out] = cast(inp, o_type.dtype)
                continue
            new_node = node.op.make_node(*[mapping[i] for i in node.inputs])
            if any(o.type.dtype == "float16" for o in new_node.outputs):
                raise TypeError("%s still yields float16 from float32 operands" % node.op)
            for o, no in zip(node.outputs, new_node.outputs):
                mapping[o] = no
        return Composite([mapping[i] for i in self.inputs], [mapping[o] for o in self.outputs])

    def c_code(self, node, inputs, outputs):
        # The temporaries' prefix is a digest of the operand names: the same in every process, so
        # that the text (and the kernel cache key made from it) is reproducible, and different
        # between an outer Composite and one emitted inside it, whose operands are the outer's
        # temporaries.
        tag = hashlib.sha1(",".join(list(inputs) + list(outputs)).encode()).hexdigest()[:6]
        return "{\n" + self.body(list(inputs), list(outputs), prefix="c%s_" % tag) + "\n}"

    def L_op(self, inputs, outputs, gout):
        raise NotImplementedError("grad is not implemented for Composite")

    def __getstate__(self):
        d = dict(self.__dict__)
        d["_code"] = None
        return d
