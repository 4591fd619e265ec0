"""TensorType, tensor variables and constants.

Mirrors ``theano/tensor/type.py:15-610`` (dtype + broadcastable pattern,
``filter``) and the operator overloads of ``theano/tensor/var.py:38-830``.
"""
import numpy as np

from .. import scalar as scal
from ..config import config
from ..gof import Apply, Constant, Type, Variable


class TensorType(Type):
    """dtype plus, per dimension, whether its extent is known to be 1."""

    def __init__(self, dtype, broadcastable, name=None, sparse_grad=False):
        self.sparse_grad = sparse_grad        # a hint for gradients of indexing ops; nothing here reads it
        if dtype == "floatX":
            dtype = config.floatX
        self.dtype = str(dtype)
        if self.dtype not in scal.all_dtypes:
            raise TypeError("Unsupported dtype for TensorType: %s" % self.dtype)
        self.broadcastable = tuple(bool(b) for b in broadcastable)
        self.ndim = len(self.broadcastable)
        self.name = name
        self.numpy_dtype = np.dtype(self.dtype)

    def clone(self, dtype=None, broadcastable=None):
        return type(self)(self.dtype if dtype is None else dtype,
                          self.broadcastable if broadcastable is None else broadcastable)

    def filter(self, data, strict=False, allow_downcast=None):
        """Convert ``data`` to an ndarray of this type or raise TypeError
        (``theano/tensor/type.py:95-236``)."""
        if isinstance(data, np.ndarray) and data.dtype == self.numpy_dtype:
            pass
        elif strict:
            raise TypeError("%s expected a ndarray object with dtype = %s (got %s)." %
                            (self, self.numpy_dtype, getattr(data, "dtype", type(data))))
        else:
            arr = np.asarray(data)
            if allow_downcast or arr.dtype == self.numpy_dtype:
                data = np.asarray(arr, dtype=self.dtype)
            else:
                up = scal.upcast(self.dtype, str(arr.dtype)) if str(arr.dtype) in scal.all_dtypes else None
                python_number = isinstance(data, (int, float, bool)) or (
                    isinstance(data, (list, tuple)) and arr.dtype in (np.float64, np.int64))
                if up == self.dtype or python_number:
                    data = np.asarray(arr, dtype=self.dtype)
                else:
                    raise TypeError("%s cannot store a value of dtype %s without risking loss of precision." %
                                    (self, arr.dtype))
        if data.ndim != self.ndim:
            raise TypeError("Wrong number of dimensions: expected %s, got %s with shape %s." %
                            (self.ndim, data.ndim, data.shape))
        for i, b in enumerate(self.broadcastable):
            if b and data.shape[i] != 1:
                raise TypeError("Non-unit value on shape on a broadcastable dimension.", data.shape,
                                self.broadcastable)
        return data

    def __eq__(self, other):
        return (type(self) is type(other) and self.dtype == other.dtype and
                self.broadcastable == other.broadcastable)

    def __hash__(self):
        return hash((type(self), self.dtype, self.broadcastable))

    def __str__(self):
        if self.name:
            return self.name
        names = {(): "scalar", (False,): "vector", (False, True): "col", (True, False): "row",
                 (False, False): "matrix"}
        b = self.broadcastable
        bcast = names.get(b, "%dD" % len(b) if not any(b) else str(b))
        return "TensorType(%s, %s)" % (self.dtype, bcast)

    __repr__ = __str__

    @staticmethod
    def values_eq_approx(a, b, rtol=None, atol=None):
        if a.shape != b.shape or a.dtype != b.dtype:
            return False
        if a.dtype.kind in "biu":
            return bool(np.array_equal(a, b))
        tol = {"float16": 1e-3, "float32": 1e-5, "float64": 1e-8}[str(a.dtype)]
        return bool(np.allclose(a, b, rtol=rtol or 1e-5, atol=atol or tol, equal_nan=True))


    # -- the value-level helpers of theano/tensor/type.py:202-310, 552-610
    @staticmethod
    def values_eq(a, b, force_same_dtype=True):
        """Exact equality of two values, NaNs and infinities in the same places counting as equal."""
        a, b = np.asarray(a), np.asarray(b)
        if a.shape != b.shape or (force_same_dtype and a.dtype != b.dtype):
            return False
        return bool(np.array_equal(a, b, equal_nan=a.dtype.kind in "fc" and b.dtype.kind in "fc"))

    @staticmethod
    def may_share_memory(a, b):
        return bool(isinstance(a, np.ndarray) and isinstance(b, np.ndarray) and np.may_share_memory(a, b))

    def value_zeros(self, shape):
        return np.zeros(shape, dtype=self.dtype)

    def value_validity_msg(self, a):
        try:
            self.filter(a, strict=True)
        except Exception as e:
            return str(e)
        return "value is valid"

    def to_scalar_type(self):
        return scal.Scalar(self.dtype)

    def get_shape_info(self, obj):
        return obj.shape

    def get_size(self, shape_info):
        n = self.numpy_dtype.itemsize
        for s in shape_info:
            n *= int(s)
        return n

    def convert_variable(self, var):
        """``var`` under this type's broadcast pattern when it has the same dtype and rank and is at least as
        broadcastable wherever this type is; None otherwise."""
        vt = var.type
        if (type(self) is type(vt) and self.dtype == vt.dtype and self.ndim == vt.ndim and
                all(sb == ob or ob for sb, ob in zip(self.broadcastable, vt.broadcastable))):
            from .views import patternbroadcast
            return patternbroadcast(var, self.broadcastable)
        return None

    def filter_variable(self, other, allow_convert=True):
        """A symbolic variable (or a value, made a constant) as a variable of this type, or TypeError."""
        if not isinstance(other, Variable):
            other = constant(self.filter(other))
        if other.type == self:
            return other
        if allow_convert:
            conv = self.convert_variable(other)
            if conv is not None and conv.type == self:
                return conv
        raise TypeError("Cannot convert Type %s (of Variable %s) into Type %s. You can try to manually convert %s "
                        "into a %s." % (other.type, other, self, other, self))


class _tensor_py_operators(object):
    """Arithmetic, comparison and reduction sugar on tensor variables."""

    dtype = property(lambda self: self.type.dtype)
    ndim = property(lambda self: self.type.ndim)
    broadcastable = property(lambda self: self.type.broadcastable)
    # `numpy_value * variable` reaches __rmul__ instead of NumPy trying to broadcast over the variable
    # (theano/tensor/var.py:733)
    __array_priority__ = 1000

    def _b(self):
        from . import basic
        return basic

    def __abs__(self): return self._b().abs_(self)
    def __neg__(self): return self._b().neg(self)
    def __invert__(self): return self._b().invert(self)
    # Results of the ordering operators refuse to be truth-tested, so that `a < b < c` (Python's
    # `(a < b) and (b < c)`) fails loudly instead of silently dropping `a < b`
    # (theano/tensor/var.py:52-95); every other variable is truthy.
    _is_nonzero = True

    def _comparison(self, rval):
        rval._is_nonzero = False
        return rval

    def __lt__(self, o): return self._comparison(self._b().lt(self, o))
    def __le__(self, o): return self._comparison(self._b().le(self, o))
    def __gt__(self, o): return self._comparison(self._b().gt(self, o))
    def __ge__(self, o): return self._comparison(self._b().ge(self, o))

    def __bool__(self):
        if self._is_nonzero:
            return True
        raise TypeError("Variables do not support boolean operations.")

    __nonzero__ = __bool__          # its Python 2 name, theano/tensor/var.py:98-105

    def __and__(self, o): return self._b().and_(self, o)
    def __or__(self, o): return self._b().or_(self, o)
    def __xor__(self, o): return self._b().xor(self, o)
    def __rand__(self, o): return self._b().and_(o, self)
    def __ror__(self, o): return self._b().or_(o, self)
    def __rxor__(self, o): return self._b().xor(o, self)
    def __rshift__(self, o): return self._b().right_shift(self, o)
    def __lshift__(self, o): return self._b().left_shift(self, o)
    def __add__(self, o): return self._b().add(self, o)
    def __sub__(self, o): return self._b().sub(self, o)
    def __mul__(self, o): return self._b().mul(self, o)
    # `/` is true division whatever the operand types; only Python 2's `__div__` chose between the
    # two divisions by type (theano/tensor/var.py:162-174, 199-209)
    def __truediv__(self, o): return self._b().true_div(self, o)
    def __div__(self, o): return self._b().div_proxy(self, o)
    def __floordiv__(self, o): return self._b().int_div(self, o)
    def __mod__(self, o): return self._b().mod_check(self, o)
    def __pow__(self, o): return self._b().pow(self, o)
    def __radd__(self, o): return self._b().add(o, self)
    def __rsub__(self, o): return self._b().sub(o, self)
    def __rmul__(self, o): return self._b().mul(o, self)
    def __rtruediv__(self, o): return self._b().true_div(o, self)
    def __rdiv__(self, o): return self._b().div_proxy(o, self)
    def __rfloordiv__(self, o): return self._b().int_div(o, self)
    def __rmod__(self, o): return self._b().mod(o, self)
    def __rpow__(self, o): return self._b().pow(o, self)

    # -- views and casts
    def dimshuffle(self, *pattern):
        from .elemwise import DimShuffle
        if len(pattern) == 1 and isinstance(pattern[0], (list, tuple)):
            pattern = pattern[0]
        return DimShuffle(self.type.broadcastable, pattern)(self)

    @property
    def T(self):
        return self.dimshuffle(*reversed(range(self.ndim)))

    def __getitem__(self, idx):
        from . import views
        return views.subtensor(self, idx)

    def __iter__(self):
        # without this Python would iterate through __getitem__ forever
        raise TypeError("a symbolic tensor cannot be iterated over; index it explicitly")

    @property
    def shape(self):
        """The extents as a tuple of 0-d int64 variables (``Shape_i``,
        ``theano/compile/ops.py:377-470``): metadata read on the host when the function runs.
        They take part in arithmetic as host scalars, and ``reshape`` / ``alloc`` accept them
        as "the extent of dimension d of that tensor"."""
        return tuple(self._b().shape_i(self, d) for d in range(self.ndim))

    @property
    def size(self):
        """The number of elements, the product of the extents (``theano/tensor/var.py:289-290``): a 0-d
        int64 host value like the extents themselves."""
        n = None
        for d in self.shape:
            n = d if n is None else n * d
        return n if n is not None else self._b().constant(np.int64(1))

    def reshape(self, *shape, **kw):
        """``x.reshape((a, b))``, ``x.reshape(a, b)`` or ``x.reshape(shape_vector, ndim=n)``
        (``theano/tensor/var.py:297-330``)."""
        from . import views
        ndim = kw.pop("ndim", None)
        if kw:
            raise TypeError("reshape() got unexpected keyword arguments %s" % sorted(kw))
        if ndim is not None and not isinstance(ndim, (int, np.integer)):
            raise ValueError("Expected ndim to be an integer, is " + str(type(ndim)))
        if len(shape) == 1 and hasattr(shape[0], "owner") and getattr(shape[0].type, "ndim", 0) == 1:
            return views.reshape(self, shape[0], ndim=ndim)
        one = shape[0] if len(shape) == 1 else None
        is_pair = (isinstance(one, (list, tuple)) and len(one) == 2 and hasattr(one[0], "type") and
                   isinstance(one[1], (int, np.integer)) and
                   0 <= one[1] < getattr(one[0].type, "ndim", 0))   # x.reshape((v, d)): the extent of v along d
        if isinstance(one, (list, tuple)) and not is_pair:
            shape = tuple(one)
        return views.reshape(self, shape, ndim=ndim)

    def fill(self, value):
        """A tensor of this one's shape filled with ``value`` (``theano/tensor/var.py:_tensor_py_operators.fill``)."""
        from . import basic
        return basic.fill(self, value)

    def flatten(self, ndim=1):
        from . import views
        return views.flatten(self, ndim)

    def astype(self, dtype):
        return self._b().cast(self, dtype)

    # -- complex numbers (theano/tensor/var.py: real, imag, conj)
    real = property(lambda self: self._b().real(self))
    imag = property(lambda self: self._b().imag(self))

    def conj(self):
        return self._b().conj(self)

    conjugate = conj

    def zeros_like(self, dtype=None):
        return self._b().zeros_like(self, dtype=dtype)

    def ones_like(self, dtype=None):
        return self._b().ones_like(self, dtype=dtype)

    # -- reductions
    def sum(self, axis=None, dtype=None, keepdims=False, acc_dtype=None):
        return self._b().sum(self, axis=axis, dtype=dtype, keepdims=keepdims, acc_dtype=acc_dtype)

    def prod(self, axis=None, dtype=None, keepdims=False, acc_dtype=None):
        return self._b().prod(self, axis=axis, dtype=dtype, keepdims=keepdims, acc_dtype=acc_dtype)

    def mean(self, axis=None, dtype=None, keepdims=False, acc_dtype=None):
        return self._b().mean(self, axis=axis, dtype=dtype, keepdims=keepdims, acc_dtype=acc_dtype)

    def var(self, axis=None, ddof=0, keepdims=False, corrected=False):
        return self._b().var(self, axis=axis, ddof=ddof, keepdims=keepdims, corrected=corrected)

    def std(self, axis=None, ddof=0, keepdims=False, corrected=False):
        return self._b().std(self, axis=axis, ddof=ddof, keepdims=keepdims, corrected=corrected)

    def max(self, axis=None, keepdims=False):
        return self._b().max(self, axis=axis, keepdims=keepdims)

    def min(self, axis=None, keepdims=False):
        return self._b().min(self, axis=axis, keepdims=keepdims)

    def any(self, axis=None, keepdims=False):
        return self._b().any(self, axis=axis, keepdims=keepdims)

    def all(self, axis=None, keepdims=False):
        return self._b().all(self, axis=axis, keepdims=keepdims)

    def argmax(self, axis=None, keepdims=False):
        return self._b().argmax(self, axis=axis, keepdims=keepdims)

    def argmin(self, axis=None, keepdims=False):
        return self._b().argmin(self, axis=axis, keepdims=keepdims)

    def norm(self, L, axis=None, keepdims=False):
        """``(sum |x|^L)^(1/L)`` (``theano/tensor/var.py:686-698``); L = 0 and infinity are not implemented
        there either."""
        if L == 0 or np.isinf(L):
            raise NotImplementedError()
        b = self._b()
        y = b.pow(b.pow(abs(self), L).sum(axis=axis), 1.0 / L)
        return b.makeKeepDims(self, y, axis) if keepdims else y

    def ptp(self, axis=None):
        return self._b().ptp(self, axis)

    # -- further elementwise methods of theano/tensor/var.py
    def clip(self, a_min, a_max):
        return self._b().clip(self, a_min, a_max)

    def round(self, mode=None):
        return self._b().round(self, mode)

    def copy(self, name=None):
        out = self._b().tensor_copy(self)
        out.name = name
        return out

    def transpose(self, *axes):
        if len(axes) == 1 and isinstance(axes[0], (list, tuple)):
            axes = tuple(axes[0])
        return self._b().transpose(self, axes if axes and axes != (None,) else None)

    def swapaxes(self, axis1, axis2):
        return self._b().swapaxes(self, axis1, axis2)

    def ravel(self):
        return self.flatten()

    def squeeze(self):
        return self._b().squeeze(self)

    def __divmod__(self, o): return self._b().divmod(self, o)
    def __rdivmod__(self, o): return self._b().divmod(o, self)
    def __ceil__(self): return self._b().ceil(self)
    def __floor__(self): return self._b().floor(self)
    def __trunc__(self): return self._b().trunc(self)
    def arccos(self): return self._b().arccos(self)
    def arccosh(self): return self._b().arccosh(self)
    def arcsin(self): return self._b().arcsin(self)
    def arcsinh(self): return self._b().arcsinh(self)
    def arctan(self): return self._b().arctan(self)
    def arctanh(self): return self._b().arctanh(self)
    def ceil(self): return self._b().ceil(self)
    def cos(self): return self._b().cos(self)
    def cosh(self): return self._b().cosh(self)
    def deg2rad(self): return self._b().deg2rad(self)
    def exp(self): return self._b().exp(self)
    def exp2(self): return self._b().exp2(self)
    def expm1(self): return self._b().expm1(self)
    def floor(self): return self._b().floor(self)
    def log(self): return self._b().log(self)
    def log10(self): return self._b().log10(self)
    def log1p(self): return self._b().log1p(self)
    def log2(self): return self._b().log2(self)
    def rad2deg(self): return self._b().rad2deg(self)
    def sin(self): return self._b().sin(self)
    def sinh(self): return self._b().sinh(self)
    def sqrt(self): return self._b().sqrt(self)
    def tan(self): return self._b().tan(self)
    def tanh(self): return self._b().tanh(self)
    def trunc(self): return self._b().trunc(self)


class TensorVariable(_tensor_py_operators, Variable):
    pass


class TensorConstant(_tensor_py_operators, Constant):
    def signature(self):
        a = np.asarray(self.data)
        return (self.type, a.shape, a.tobytes())

    def __str__(self):
        if self.name is not None:
            return self.name
        a = np.asarray(self.data)
        return "TensorConstant{%s}" % (a if a.size <= 4 else "shape %s" % (a.shape,))

    __repr__ = __str__


TensorType.Variable = TensorVariable
TensorType.Constant = TensorConstant


def constant(x, name=None, ndim=None, dtype=None):
    """Tensor constant; every extent-1 dimension is broadcastable
    (``theano/tensor/basic.py:211-262``)."""
    x_ = scal.convert(x, dtype=dtype)
    if str(x_.dtype) not in scal.all_dtypes:
        raise TypeError("cannot make a tensor constant of dtype %s" % x_.dtype)
    bcast = [s == 1 for s in x_.shape]
    if ndim is not None:
        if len(bcast) < ndim:
            bcast = [True] * (ndim - len(bcast)) + bcast
            x_ = x_.reshape((1,) * (ndim - x_.ndim) + x_.shape)
        elif len(bcast) > ndim:
            raise ValueError("constant has %d dimensions, asked for %d" % (len(bcast), ndim))
    return TensorConstant(TensorType(str(x_.dtype), bcast), np.asarray(x_, order="C"), name=name)


def as_tensor_variable(x, name=None, ndim=None):
    if isinstance(x, Apply):
        x = x.default_output()
    if isinstance(x, Variable):
        if isinstance(x.type, scal.Scalar):
            from .basic import tensor_from_scalar
            x = tensor_from_scalar(x)
        if not isinstance(x.type, TensorType):
            to_tensor = getattr(x.type, "as_tensor_variable", None)
            if to_tensor is None:
                raise TypeError("Variable type field must be a TensorType.", x, x.type)
            x = to_tensor(x)
        if ndim is not None and x.type.ndim != ndim:
            if x.type.ndim < ndim:
                x = x.dimshuffle(*(["x"] * (ndim - x.type.ndim) + list(range(x.type.ndim))))
            else:
                raise ValueError("TensorType could not be cast to have %i dimensions" % ndim, x.type)
        return x
    if isinstance(x, (tuple, list)) and any(isinstance(i, Variable) for i in x):
        raise TypeError("lists of symbolic variables are not supported here")
    return constant(x, name=name, ndim=ndim)


def _mk(dtype, bcast):
    def make(name=None):
        return TensorType(dtype, bcast)(name)
    return make


for _p, _dt in (("b", "int8"), ("w", "int16"), ("i", "int32"), ("l", "int64"), ("h", "float16"),
                ("f", "float32"), ("d", "float64"), ("c", "complex64"), ("z", "complex128")):
    globals()[_p + "scalar"] = _mk(_dt, ())
    globals()[_p + "vector"] = _mk(_dt, (False,))
    globals()[_p + "matrix"] = _mk(_dt, (False, False))
    globals()[_p + "row"] = _mk(_dt, (True, False))
    globals()[_p + "col"] = _mk(_dt, (False, True))
    globals()[_p + "tensor3"] = _mk(_dt, (False,) * 3)
    globals()[_p + "tensor4"] = _mk(_dt, (False,) * 4)
    for _nd in (5, 6, 7):
        globals()[_p + "tensor%d" % _nd] = _mk(_dt, (False,) * _nd)


def scalar(name=None, dtype=None):
    return TensorType(dtype or config.floatX, ())(name)


def vector(name=None, dtype=None):
    return TensorType(dtype or config.floatX, (False,))(name)


def matrix(name=None, dtype=None):
    return TensorType(dtype or config.floatX, (False, False))(name)


def row(name=None, dtype=None):
    return TensorType(dtype or config.floatX, (True, False))(name)


def col(name=None, dtype=None):
    return TensorType(dtype or config.floatX, (False, True))(name)


def tensor3(name=None, dtype=None):
    return TensorType(dtype or config.floatX, (False,) * 3)(name)


def tensor4(name=None, dtype=None):
    return TensorType(dtype or config.floatX, (False,) * 4)(name)


def tensor5(name=None, dtype=None):
    return TensorType(dtype or config.floatX, (False,) * 5)(name)


def tensor6(name=None, dtype=None):
    return TensorType(dtype or config.floatX, (False,) * 6)(name)


def tensor7(name=None, dtype=None):
    return TensorType(dtype or config.floatX, (False,) * 7)(name)


def tensor(dtype, broadcastable, name=None):
    return TensorType(dtype, broadcastable)(name)


def _plural(make):
    """``matrices('a', 'b')`` / ``matrices(3)``: several variables of one constructor at once, a single one for a
    single name (``_multi``, ``theano/tensor/basic.py:644-661``)."""
    def many(*names):
        if len(names) == 1 and isinstance(names[0], (int, np.integer)) and not isinstance(names[0], bool):
            return [make() for _ in range(int(names[0]))]
        if len(names) == 1 and isinstance(names[0], (list, tuple)):
            names = tuple(names[0])
        if len(names) == 1:
            return make(names[0])
        return [make(n) for n in names]
    return many


_PLURAL = {"scalar": "scalars", "vector": "vectors", "matrix": "matrices", "row": "rows", "col": "cols",
           "tensor3": "tensor3s", "tensor4": "tensor4s", "tensor5": "tensor5s", "tensor6": "tensor6s",
           "tensor7": "tensor7s"}
for _one, _many in _PLURAL.items():
    for _p in ("", "f", "d", "i", "l"):
        globals()[_p + _many] = _plural(globals()[_p + _one])
