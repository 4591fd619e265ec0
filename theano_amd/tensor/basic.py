"""User-level tensor functions: one Elemwise instance per ScalarOp, casts,
fills and the reduction front-ends.

Mirrors the on-path parts of ``theano/tensor/basic.py``: ``_scal_elemwise``
:975-1020, ``makeKeepDims`` :1613-1647, ``max``/``min`` :1682-1775,
``sum``/``prod`` :3190-3244, ``mean`` :3291-3382, ``var``/``std`` :3386-3480,
``any``/``all`` :6353-6366, and ``sigmoid``/``softplus`` of
``theano/tensor/nnet/sigm.py:167-168, 372``.
"""
import numpy as np

from .. import scalar as scal
from ..config import config
from ..gof import Apply, Op
from .elemwise import All, Any, CAReduce, DimShuffle, Elemwise, Prod, Sum
from .type import TensorType, as_tensor_variable, constant

discrete_dtypes = scal.discrete_dtypes
continuous_dtypes = scal.continuous_dtypes
int_dtypes = scal.int_dtypes
uint_dtypes = scal.uint_dtypes


def _elemwise(scalar_op, name):
    return Elemwise(scalar_op, name="Elemwise{%s}" % name)


lt, gt, le, ge = _elemwise(scal.lt, "lt"), _elemwise(scal.gt, "gt"), _elemwise(scal.le, "le"), _elemwise(scal.ge, "ge")
eq, neq = _elemwise(scal.eq, "eq"), _elemwise(scal.neq, "neq")
isnan, isinf = _elemwise(scal.isnan, "isnan"), _elemwise(scal.isinf, "isinf")
switch = _elemwise(scal.switch, "switch")
where = switch
and_, or_, xor, invert = (_elemwise(scal.and_, "and_"), _elemwise(scal.or_, "or_"), _elemwise(scal.xor, "xor"),
                          _elemwise(scal.invert, "invert"))
bitwise_and, bitwise_or, bitwise_xor, bitwise_not = and_, or_, xor, invert
right_shift, left_shift = _elemwise(scal.right_shift, "right_shift"), _elemwise(scal.left_shift, "left_shift")
maximum, minimum = _elemwise(scal.maximum, "maximum"), _elemwise(scal.minimum, "minimum")
add, mul, sub = _elemwise(scal.add, "add"), _elemwise(scal.mul, "mul"), _elemwise(scal.sub, "sub")
true_div, int_div, mod = _elemwise(scal.true_div, "true_div"), _elemwise(scal.int_div, "int_div"), _elemwise(scal.mod, "mod")
pow, clip, second = _elemwise(scal.pow, "pow"), _elemwise(scal.clip, "clip"), _elemwise(scal.second, "second")
fill = second
tensor_copy = _elemwise(scal.identity, "identity")
abs_, sgn, neg, inv = _elemwise(scal.abs_, "abs_"), _elemwise(scal.sgn, "sgn"), _elemwise(scal.neg, "neg"), _elemwise(scal.inv, "inv")
ceil, floor, trunc = _elemwise(scal.ceil, "ceil"), _elemwise(scal.floor, "floor"), _elemwise(scal.trunc, "trunc")
round_half_to_even = _elemwise(scal.round_half_to_even, "round_half_to_even")
round_half_away_from_zero = _elemwise(scal.round_half_away_from_zero, "round_half_away_from_zero")
log, log2, log10, log1p = _elemwise(scal.log, "log"), _elemwise(scal.log2, "log2"), _elemwise(scal.log10, "log10"), _elemwise(scal.log1p, "log1p")
exp, exp2, expm1 = _elemwise(scal.exp, "exp"), _elemwise(scal.exp2, "exp2"), _elemwise(scal.expm1, "expm1")
sqr, sqrt = _elemwise(scal.sqr, "sqr"), _elemwise(scal.sqrt, "sqrt")
cos, sin, tan = _elemwise(scal.cos, "cos"), _elemwise(scal.sin, "sin"), _elemwise(scal.tan, "tan")
arccos, arcsin, arctan, arctan2 = (_elemwise(scal.arccos, "arccos"), _elemwise(scal.arcsin, "arcsin"),
                                   _elemwise(scal.arctan, "arctan"), _elemwise(scal.arctan2, "arctan2"))
cosh, sinh, tanh = _elemwise(scal.cosh, "cosh"), _elemwise(scal.sinh, "sinh"), _elemwise(scal.tanh, "tanh")
arccosh, arcsinh, arctanh = _elemwise(scal.arccosh, "arccosh"), _elemwise(scal.arcsinh, "arcsinh"), _elemwise(scal.arctanh, "arctanh")
erf, erfc, erfcx = _elemwise(scal.erf, "erf"), _elemwise(scal.erfc, "erfc"), _elemwise(scal.erfcx, "erfcx")
erfinv, erfcinv = _elemwise(scal.erfinv, "erfinv"), _elemwise(scal.erfcinv, "erfcinv")
gamma, gammaln = _elemwise(scal.gamma, "gamma"), _elemwise(scal.gammaln, "gammaln")
psi, tri_gamma = _elemwise(scal.psi, "psi"), _elemwise(scal.tri_gamma, "tri_gamma")
j0, j1, i0, i1 = _elemwise(scal.j0, "j0"), _elemwise(scal.j1, "j1"), _elemwise(scal.i0, "i0"), _elemwise(scal.i1, "i1")
jv, iv = _elemwise(scal.jv, "jv"), _elemwise(scal.iv, "iv")
gammainc, gammaincc = _elemwise(scal.gammainc, "gammainc"), _elemwise(scal.gammaincc, "gammaincc")
real, imag, angle, conj = (_elemwise(scal.real, "real"), _elemwise(scal.imag, "imag"), _elemwise(scal.angle, "angle"),
                           _elemwise(scal.conj, "conj"))
complex, complex_from_polar = _elemwise(scal.complex, "complex"), _elemwise(scal.complex_from_polar, "complex_from_polar")
gammau, gammal, chi2sf = _elemwise(scal.gammau, "gammau"), _elemwise(scal.gammal, "gammal"), _elemwise(scal.chi2sf, "chi2sf")
sigmoid = _elemwise(scal.scalar_sigmoid, "sigmoid")
softplus = _elemwise(scal.scalar_softplus, "softplus")


def div_proxy(x, y):
    """``x / y``: integer or true division by operand types
    (``theano/tensor/basic.py`` ``div_proxy``, ``theano/scalar/basic.py:1826-1885``)."""
    x, y = as_tensor_variable(x), as_tensor_variable(y)
    f = scal.int_or_true_div(x.type.dtype in discrete_dtypes, y.type.dtype in discrete_dtypes)
    return (int_div if f is scal.int_div else true_div)(x, y)


_cast_ops = dict((dt, Elemwise(scal._cast_mapping[dt], name="Elemwise{Cast{%s}}" % dt)) for dt in scal.all_dtypes)


def cast(x, dtype):
    if dtype == "floatX":
        dtype = config.floatX
    dtype = str(dtype)
    x = as_tensor_variable(x)
    if x.type.dtype == dtype:
        return x
    if x.type.dtype in scal.complex_dtypes and dtype not in scal.complex_dtypes:
        # theano/tensor/basic.py:1263-1266
        raise TypeError("Casting from complex to real is ambiguous: consider real(), imag(), angle() or abs()")
    return _cast_ops[dtype](x)


def zeros_like(model, dtype=None, opt=False):
    """``fill(model, 0)``; with ``opt`` the bare constant when it already has ``model``'s type
    (``theano/tensor/basic.py:2521-2547``)."""
    model = as_tensor_variable(model)
    if dtype is None:
        dtype = model.type.dtype
    ret = constant(0, dtype=dtype)
    if opt and ret.type == model.type:
        return ret
    return fill(model, ret)


def ones_like(model, dtype=None, opt=False):
    """``fill(model, 1)`` (``theano/tensor/basic.py:2493-2518``)."""
    model = as_tensor_variable(model)
    if dtype is None:
        dtype = model.type.dtype
    ret = constant(1, dtype=dtype)
    if opt and ret.type == model.type:
        return ret
    return fill(model, ret)


def iround(a, mode=None):
    """``cast(round(a, mode), 'int64')`` (``theano/tensor/basic.py:2168-2171``)."""
    return cast(round(a, mode), "int64")


def round(a, mode=None):
    """Rounding of halves to even (the default, NumPy's) or away from zero (``theano/tensor/basic.py:2175-2192``)."""
    if mode is None:
        mode = "half_to_even"
    if mode == "half_away_from_zero":
        return round_half_away_from_zero(a)
    if mode == "half_to_even":
        return round_half_to_even(a)
    raise Exception("round mode %s is not implemented." % mode)


def tensor_from_scalar(s):
    raise NotImplementedError("scalar variables cannot be turned into tensors here; use a 0-d tensor")


# --------------------------------------------------------------------------
class ShapeFloat(Op):
    """Extent of dimension ``i`` of the input as a 0-d tensor of ``dtype``.

    With a floating dtype it stands for ``cast(shape(x)[i], dtype)`` in ``mean`` /
    ``var`` (``theano/tensor/basic.py:3352-3373``), with int64 for ``Shape_i``
    (``theano/compile/ops.py:377-470``), what ``x.shape[i]`` is.  It runs on the host
    and reads only array metadata, whichever memory the array lives in; fused
    consumers take its value as a kernel argument."""

    __props__ = ("i", "dtype")

    def __init__(self, i, dtype):
        self.i = int(i)
        self.dtype = str(dtype)

    def make_node(self, x):
        x = x if hasattr(x.type, "ndim") else as_tensor_variable(x)
        if self.i >= x.type.ndim:
            raise TypeError("x has too few dimensions for ShapeFloat", (x, self.i))
        return Apply(self, [x], [TensorType(self.dtype, ())()])

    def perform(self, node, inputs, output_storage):
        output_storage[0][0] = np.asarray(inputs[0].shape[self.i], dtype=self.dtype)

    def infer_shape(self, node, shapes):
        return [()]

    def connection_pattern(self, node):
        return [[False]]

    def grad(self, inp, grads):
        return [scal.DisconnectedType()()]

    def R_op(self, inputs, eval_points):
        return [None]           # an extent does not move with the values (``Shape.R_op``, theano/compile/ops.py:279-280)


# --------------------------------------------------------------------------
def _axis_list(axis, ndim):
    if axis is None:
        return list(range(ndim))
    if isinstance(axis, (int, np.integer)):
        axis = [int(axis)]
    elif isinstance(axis, np.ndarray) and axis.ndim == 0:
        axis = [int(axis)]
    else:
        axis = [int(a) for a in axis]
    return axis


def makeKeepDims(x, y, axis):
    """Re-insert, with length one, the axes of ``x`` that a reduction dropped."""
    x, y = as_tensor_variable(x), as_tensor_variable(y)
    newaxis = [a + x.type.ndim if a < 0 else a for a in _axis_list(axis, x.type.ndim)]
    i, new_dims = 0, []
    for j in range(x.type.ndim):
        if j in newaxis:
            new_dims.append("x")
        else:
            new_dims.append(i)
            i += 1
    return DimShuffle(y.type.broadcastable, new_dims)(y)


def sum(input, axis=None, dtype=None, keepdims=False, acc_dtype=None):
    out = Sum(axis=axis, dtype=dtype, acc_dtype=acc_dtype)(input)
    if keepdims:
        out = makeKeepDims(input, out, axis)
    return out


def prod(input, axis=None, dtype=None, keepdims=False, acc_dtype=None, no_zeros_in_input=False):
    out = Prod(axis, dtype=dtype, acc_dtype=acc_dtype, no_zeros_in_input=no_zeros_in_input)(input)
    if keepdims:
        out = makeKeepDims(input, out, axis)
    return out


class Max(CAReduce):
    """``CAReduce{maximum}`` carrying the gradient of the reference's
    ``MaxAndArgmax`` (``theano/tensor/basic.py:1429-1483``), which is what
    ``tensor.max`` becomes once ``local_max_and_argmax``
    (``theano/tensor/opt_uncanonicalize.py:51-68``) has run."""

    __props__ = ("axis",)

    def __init__(self, axis=None):
        CAReduce.__init__(self, scal.maximum, axis)

    def _props(self):
        return (self.axis,)

    def __str__(self):
        return "Max" if self.axis is None else "Max{%s}" % ", ".join(map(str, self.axis))

    def L_op(self, inp, out, grads):
        (x,) = inp
        (g_max,) = grads
        if x.type.dtype in discrete_dtypes:
            return [x.zeros_like(dtype=config.floatX)]
        axis = self.axis if self.axis is not None else tuple(range(x.type.ndim))
        pattern, k = [], 0
        for i in range(x.type.ndim):
            if i in axis:
                pattern.append("x")
            else:
                pattern.append(k)
                k += 1
        g_max_pad = DimShuffle(g_max.type.broadcastable, pattern)(g_max)
        xmax_pad = DimShuffle(out[0].type.broadcastable, pattern)(out[0])
        return [eq(xmax_pad, x) * g_max_pad]


class Min(CAReduce):
    """``CAReduce{minimum}`` (what ``local_max_to_min`` produces,
    ``theano/tensor/opt_uncanonicalize.py:71-94``)."""

    __props__ = ("axis",)

    def __init__(self, axis=None):
        CAReduce.__init__(self, scal.minimum, axis)

    def _props(self):
        return (self.axis,)

    def __str__(self):
        return "Min" if self.axis is None else "Min{%s}" % ", ".join(map(str, self.axis))

    L_op = Max.L_op


class MaxAndArgmax(Op):
    """Maximum and the position of its first occurrence over ``axis`` (a sorted
    tuple of axes) - ``theano/tensor/basic.py:1273-1483``.  The second output is
    int64: the index ``numpy.argmax`` gives once the reduced axes are moved to the
    end, in their original order, and flattened (``perform``, :1311-1330).  A NaN
    is the maximum and its position the argmax, as with NumPy."""

    __props__ = ("axis",)

    def __init__(self, axis):
        self.axis = tuple(sorted(int(a) for a in axis))

    def _props(self):
        return (self.axis,)

    def __str__(self):
        return "MaxAndArgmax{%s}" % ", ".join(map(str, self.axis))

    def make_node(self, x):
        x = as_tensor_variable(x)
        for a in self.axis:
            if a < 0 or a >= x.type.ndim:
                raise ValueError("MaxAndArgmax: bad axis argument")
        if not self.axis:
            raise ValueError("MaxAndArgmax needs at least one axis")
        b = [bb for i, bb in enumerate(x.type.broadcastable) if i not in self.axis]
        return Apply(self, [x], [TensorType(x.type.dtype, b)(), TensorType("int64", b)()])

    def infer_shape(self, node, shapes):
        kept = tuple(s for i, s in enumerate(shapes[0]) if i not in self.axis)
        return [kept, kept]

    def perform(self, node, inputs, output_storage):
        raise NotImplementedError("MaxAndArgmax runs on the device only; compile the graph with function()")

    def connection_pattern(self, node):
        return [[True, False]]

    def L_op(self, inp, out, grads):
        # theano/tensor/basic.py:1429-1483: the gradient flows to the positions that equal the maximum
        (x,) = inp
        g_max = grads[0]
        if g_max is None or isinstance(getattr(g_max, "type", None), scal.DisconnectedType):
            return [x.zeros_like()]
        if x.type.dtype in discrete_dtypes:
            return [x.zeros_like(dtype=config.floatX)]
        pattern, k = [], 0
        for i in range(x.type.ndim):
            if i in self.axis:
                pattern.append("x")
            else:
                pattern.append(k)
                k += 1
        g_max_pad = DimShuffle(g_max.type.broadcastable, pattern)(g_max)
        xmax_pad = DimShuffle(out[0].type.broadcastable, pattern)(out[0])
        return [eq(xmax_pad, x) * g_max_pad]


def max_and_argmax(a, axis=None, keepdims=False):
    """``[max, argmax]`` over ``axis`` (None: all axes) -
    ``theano/tensor/basic.py:1651-1680``."""
    a = as_tensor_variable(a)
    if a.type.ndim == 0:                      # nothing to reduce: the value itself, at position 0
        return [a, constant(0, dtype="int64")]
    ax = sorted(set(d + a.type.ndim if d < 0 else d for d in _axis_list(axis, a.type.ndim)))
    if not ax:
        ax = list(range(a.type.ndim))
    out, argout = MaxAndArgmax(ax)(a)
    if keepdims:
        out = makeKeepDims(a, out, ax)
        argout = makeKeepDims(a, argout, ax)
    return [out, argout]


def argmax(x, axis=None, keepdims=False):
    return max_and_argmax(x, axis, keepdims)[1]


def argmin(x, axis=None, keepdims=False):
    """``argmax`` of the order-reversed values, as the reference does
    (``theano/tensor/basic.py:1779-1803``): ``-x``, ``max - x`` for unsigned
    integers, ``~x`` for bool."""
    x = as_tensor_variable(x)
    dt = x.type.dtype
    if dt in scal.float_dtypes or dt in scal.int_dtypes:
        return argmax(-x, axis=axis, keepdims=keepdims)
    if dt in scal.uint_dtypes:
        return argmax(np.array(np.iinfo(dt).max, dtype=dt) - x, axis=axis, keepdims=keepdims)
    if dt == "bool":
        return argmax(~x, axis=axis, keepdims=keepdims)
    raise NotImplementedError(dt)


def max(x, axis=None, keepdims=False):
    x = as_tensor_variable(x)
    out = Max(axis)(x)
    if keepdims:
        out = makeKeepDims(x, out, axis)
    return out


def min(x, axis=None, keepdims=False):
    x = as_tensor_variable(x)
    out = Min(axis)(x)
    if keepdims:
        out = makeKeepDims(x, out, axis)
    return out


def shape_i(x, i):
    """``x.shape[i]`` as a 0-d int64 variable."""
    x = as_tensor_variable(x)
    if x.type.broadcastable[i]:
        return constant(np.int64(1))
    return ShapeFloat(i, "int64")(x)


def Shape_i(i):
    return ShapeFloat(i, "int64")


def mod_check(x, y):
    """``x % y`` of the operators: complex operands are refused when the graph is built
    (``theano/tensor/basic.py:3622-3629``)."""
    if as_tensor_variable(x).type.dtype in scal.complex_dtypes or as_tensor_variable(y).type.dtype in scal.complex_dtypes:
        raise scal.ComplexError("the mod operator (%) is not defined for complex numbers "
                                "(theano/scalar/basic.py:2050-2052)")
    return mod(x, y)


def divmod(x, y):
    """Elementwise ``(x // y, x % y)`` (``theano/tensor/basic.py:3562-3564``)."""
    return int_div(x, y), mod_check(x, y)


def squeeze(x):
    """``x`` without its broadcastable dimensions: a view (``theano/tensor/extra_ops.py:556-579``)."""
    x = as_tensor_variable(x)
    return x.dimshuffle([i for i in range(x.type.ndim) if not x.type.broadcastable[i]])


def mean(input, axis=None, dtype=None, op=False, keepdims=False, acc_dtype=None):
    """Sum divided by the extent of every reduced axis in turn; float16 inputs
    are summed in float32 and the result is cast back.  ``op=True`` asks the reference for its
    host-only ``Mean`` op (``theano/tensor/basic.py:3246-3288, 3328-3344``), which has no device form."""
    input = as_tensor_variable(input)
    if op:
        raise NotImplementedError("mean(op=True): the Mean op computes on the host in float64; call "
                                  "mean(..., op=False), which sums and divides on the device")
    if dtype is not None:
        sum_dtype = dtype
    else:
        sum_dtype = "float32" if input.type.dtype == "float16" else None
    s = sum(input, axis=axis, dtype=sum_dtype, keepdims=keepdims, acc_dtype=acc_dtype)
    shp_dtype = "float32" if s.type.dtype in ("float16", "float32", "complex64") else "float64"
    for i in _axis_list(axis, input.type.ndim):
        s = true_div(s, ShapeFloat(i if i >= 0 else i + input.type.ndim, shp_dtype)(input))
    if s.type.dtype in discrete_dtypes:
        s = cast(s, shp_dtype)
    if dtype == "float16" or (dtype is None and input.type.dtype == "float16"):
        s = cast(s, "float16")
    s.name = "mean"
    return s


def var(input, axis=None, ddof=0, keepdims=False, corrected=False):
    """Two-pass variance: mean of the squared deviations from the mean."""
    if isinstance(ddof, bool):
        raise ValueError("Parameter keepdims is now at index 3: (input, axis=None, ddof=0, keepdims=False, "
                         "corrected=False)")
    input = as_tensor_variable(input)
    axis = _axis_list(axis, input.type.ndim)
    mean_input = mean(input, axis, keepdims=True)
    centered = input - mean_input
    two = constant(2, dtype=centered.type.dtype)
    if ddof == 0:
        v = mean(centered ** two, axis, keepdims=keepdims)
    else:
        v = sum(centered ** two, axis=axis, keepdims=keepdims)
        for i in axis:
            v = true_div(v, ShapeFloat(i, "float64")(input) - ddof)
    if corrected:
        if ddof == 0:
            error = mean(centered, axis, keepdims=keepdims) ** 2
        else:
            error = sum(centered, axis=axis, keepdims=keepdims) ** 2
            for i in axis:
                n = ShapeFloat(i, "float64")(input)
                error = true_div(error, (n - ddof) * n)
        v = v - error
    v.name = "var"
    return v


def std(input, axis=None, ddof=0, keepdims=False, corrected=False):
    ret = sqrt(var(input, axis=axis, ddof=ddof, keepdims=keepdims, corrected=corrected))
    ret.name = "std"
    return ret


def any(x, axis=None, keepdims=False):
    out = Any(axis)(x)
    if keepdims:
        out = makeKeepDims(x, out, axis)
    return out


def all(x, axis=None, keepdims=False):
    out = All(axis)(x)
    if keepdims:
        out = makeKeepDims(x, out, axis)
    return out


def softmax(x):
    """Row softmax written with Elemwise and CAReduce nodes, the graph the
    reference's ``softmax_simplifier`` recognises (``theano/tensor/nnet/nnet.py:888-925``)."""
    x = as_tensor_variable(x)
    e = exp(x - max(x, axis=-1, keepdims=True))
    return e / sum(e, axis=-1, keepdims=True)


# ---- further front ends of theano/tensor/basic.py, all compositions of the ops above ---------------
floor_div, power, square, absolute, sign = int_div, pow, sqr, abs_, sgn
rint = round_half_to_even


# ``x * (pi / 180)`` and ``x * (180 / pi)`` as the reference's scalar ops compute them: the product in
# double precision, rounded to the result type once (``theano/tensor/basic.py:2280-2288``)
deg2rad, rad2deg = _elemwise(scal.deg2rad, "deg2rad"), _elemwise(scal.rad2deg, "rad2deg")


def smallest(*args):
    """Elementwise smallest of the arguments (``theano/tensor/basic.py:1809-1820``)."""
    if len(args) == 2:
        a, b = args
        return switch(lt(a, b), a, b)
    from .views import stack
    return min(stack(list(args)), axis=0)


def largest(*args):
    """Elementwise largest of the arguments (``theano/tensor/basic.py:1824-1835``)."""
    if len(args) == 2:
        a, b = args
        return switch(gt(a, b), a, b)
    from .views import stack
    return max(stack(list(args)), axis=0)


def ceil_intdiv(a, b):
    """``ceil(a / b)`` without leaving the integers (``theano/tensor/basic.py:3601-3620``)."""
    div = int_div(a, b)
    return cast(neq(mod(a, b), 0), div.type.dtype) + div


def isclose(a, b, rtol=1.e-5, atol=1.e-8, equal_nan=False):
    """``numpy.isclose`` as a graph (``theano/tensor/basic.py:1942-2030``): within tolerance and
    neither NaN nor infinite, or infinities of the same sign, or (``equal_nan``) both NaN."""
    a, b = as_tensor_variable(a), as_tensor_variable(b)
    close_prelim = le(abs_(a - b), atol + rtol * abs_(b))
    a_nan, b_nan = isnan(a), isnan(b)
    a_inf, b_inf = isinf(a), isinf(b)
    nans_or_infs = or_(or_(a_nan, b_nan), or_(a_inf, b_inf))
    close = and_(close_prelim, invert(nans_or_infs))
    inf_eq = and_(and_(a_inf, b_inf), eq(a_inf * sgn(a), b_inf * sgn(b)))
    close_with_infs = or_(close, inf_eq)
    if equal_nan:
        return or_(close_with_infs, and_(a_nan, b_nan))
    return close_with_infs


def allclose(a, b, rtol=1.e-5, atol=1.e-8, equal_nan=False):
    """``all(isclose(a, b))`` (``theano/tensor/basic.py:1908-1939``)."""
    return all(isclose(a, b, rtol, atol, equal_nan))


def ptp(a, axis=None):
    """Range of values, ``max - min`` along an axis (``theano/tensor/basic.py:6722-6746``)."""
    a = as_tensor_variable(a)
    return max(a, axis) - min(a, axis)


def shape_padleft(t, n_ones=1):
    """``theano/tensor/basic.py:4559-4573``"""
    t = as_tensor_variable(t)
    return t.dimshuffle(*(["x"] * n_ones + list(range(t.type.ndim))))


def shape_padright(t, n_ones=1):
    """``theano/tensor/basic.py:4576-4590``"""
    t = as_tensor_variable(t)
    return t.dimshuffle(*(list(range(t.type.ndim)) + ["x"] * n_ones))


def shape_padaxis(t, axis):
    """A broadcastable dimension inserted at ``axis`` (``theano/tensor/basic.py:4593-4630``)."""
    t = as_tensor_variable(t)
    nd = t.type.ndim + 1
    if not -nd <= axis < nd:
        raise IndexError("axis {0} is out of bounds [-{1}, {1})".format(axis, nd))
    axis = axis + nd if axis < 0 else axis
    pattern = list(range(t.type.ndim))
    pattern.insert(axis, "x")
    return t.dimshuffle(*pattern)


def transpose(x, axes=None):
    """``theano/tensor/basic.py:3701-3716``"""
    x = as_tensor_variable(x)
    axes = list(range(x.type.ndim - 1, -1, -1)) if axes is None else list(axes)
    return x.dimshuffle(*axes)


def swapaxes(y, axis1, axis2):
    """``theano/tensor/basic.py:6753-6760``"""
    y = as_tensor_variable(y)
    order = list(range(y.type.ndim))
    order[axis1], order[axis2] = order[axis2], order[axis1]
    return y.dimshuffle(*order)


def zeros(shape, dtype=None):
    """``alloc(0, *shape)`` (``theano/tensor/basic.py:2550-2558``); entries: ints or ``v.shape[d]``."""
    from .views import alloc
    shape = list(shape) if isinstance(shape, (list, tuple)) else [shape]
    return alloc(np.array(0, dtype=dtype or config.floatX), *shape)


def ones(shape, dtype=None):
    """``alloc(1, *shape)`` (``theano/tensor/basic.py:2561-2569``)."""
    from .views import alloc
    shape = list(shape) if isinstance(shape, (list, tuple)) else [shape]
    return alloc(np.array(1, dtype=dtype or config.floatX), *shape)
