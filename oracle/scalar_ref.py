"""TEST INFRASTRUCTURE - not part of the product.  Only ``tests/``, the
``cpu_baseline`` leg of ``bench.py`` and ``__graft_entry__.smoke()`` may import
anything under ``oracle/``.

NumPy restatement of the per-element C semantics of Theano's scalar ops
(``theano/scalar/basic.py``; sigmoid/softplus ``theano/tensor/nnet/sigm.py:60-85,
344-362``).  Each function takes NumPy arrays and the output dtype decided by
the graph, and evaluates what the generated C expression evaluates: operands
are first brought to the type C's usual arithmetic conversions give the
expression (``c_common_type``), the operation is done in that type, and the
result is converted to the output dtype as the C assignment does.

Pinning (tests/test_oracle_scalar.py): Mod / IntDiv against Python ``%`` and
``//`` on the exhaustive int8 grid of ``theano/tensor/tests/test_basic.py:878-896``, and - for every pair
of integer operand types, where the sign tests see each operand in its own type and the divisions C's
common type - against the reference's C text compiled by gcc, over the ends of every type's range
(operands whose negation overflows, which C leaves undefined and compilers treat differently, wrap here;
that choice is pinned by literal values);
comparisons and bit ops against the truth tables of
``theano/scalar/tests/test_basic.py:187-256``; sigmoid against ``1/(1+exp(-x))``
(``theano/tensor/nnet/tests/test_sigm.py:29-41``); max/min NaN propagation
(``theano/tensor/tests/test_elemwise.py:525-538``); dtype rules against the
literal tables of ``theano/scalar/basic.py:855-870`` and
``theano/scalar/tests/test_basic.py:264-380``; ``right_shift(a, 3) ==
int_div(a, 8)`` (no shift op exists in the reference); float IntDiv against a
scalar transcription of the four sign cases and against exact floor division away
from integer quotients.  The special functions are ``scipy.special`` itself, which
is what the reference's ``impl`` calls (``theano/scalar/basic_scipy.py:32-36``); every
differentiable op's value is tied to its neighbours' by the finite-difference
gradient checks of tests/test_oracle_graph.py.  The approximate sigmoid is pinned by
hand-evaluated points on each of its pieces, its symmetry and its known distance to
the sigmoid; softsign by exact quotients; the fused sigmoid cross-entropy by
``log(1 + e^x) - x t`` and, where that is well conditioned, the two-logarithm
definition.  The angle-unit conversions are pinned element by element against Python float
arithmetic (the double product rounded once - which NumPy's float32 ``deg2rad`` is not) and by
known angles; the range test against Python's comparisons on every triple of a small grid, for
the four open / closed combinations and mixed operand types.  No function here is unpinned.
"""
import numpy as np

_RANK = {"bool": 0, "int8": 1, "uint8": 1, "int16": 2, "uint16": 2, "int32": 3, "uint32": 3, "int64": 4, "uint64": 4}


def c_common_type(*dtypes):
    """Type in which C evaluates a binary arithmetic expression over operands
    of these types (integer promotion, then the usual arithmetic conversions).
    float16 operands are float here, as in the reference's device code."""
    dtypes = [str(d) for d in dtypes]
    if "float64" in dtypes:
        return "float64"
    if "float32" in dtypes or "float16" in dtypes:
        return "float32"
    cur = "int32"
    for d in dtypes:
        if _RANK[d] <= 2:
            d = "int32"  # integer promotion: every narrower type fits in int
        if d == cur:
            continue
        ud, uc = d.startswith("u"), cur.startswith("u")
        if ud == uc:
            cur = d if _RANK[d] > _RANK[cur] else cur
        else:
            u, sg = (d, cur) if ud else (cur, d)
            cur = u if _RANK[u] >= _RANK[sg] else sg
    return cur


def _conv(x, dtype):
    """C conversion of values to ``dtype`` (bool storage is one byte 0/1)."""
    x = np.asarray(x)
    if str(dtype) == "bool":
        return x != 0
    with np.errstate(all="ignore"):
        return x.astype(dtype)


def _arith(fn, out_dtype, *xs):
    ct = c_common_type(*[x.dtype for x in xs])
    with np.errstate(all="ignore"):
        r = fn(*[_conv(x, ct) for x in xs])
    return _conv(r, out_dtype)


def add(out_dtype, *xs):
    if str(out_dtype) == "bool":  # x || y ...
        r = xs[0] != 0
        for x in xs[1:]:
            r = r | (x != 0)
        return r
    def f(*a):
        r = a[0]
        for b in a[1:]:
            r = r + b
        return r
    return _arith(f, out_dtype, *xs)


def mul(out_dtype, *xs):
    if str(out_dtype) == "bool":  # x && y ...
        r = xs[0] != 0
        for x in xs[1:]:
            r = r & (x != 0)
        return r
    def f(*a):
        r = a[0]
        for b in a[1:]:
            r = r * b
        return r
    return _arith(f, out_dtype, *xs)


def sub(out_dtype, x, y):
    return _arith(lambda a, b: a - b, out_dtype, x, y)


def true_div(out_dtype, x, y):
    if x.dtype.kind in "biu" and y.dtype.kind in "biu":
        # ((double)x) / y
        with np.errstate(all="ignore"):
            return _conv(x.astype("float64") / y.astype("float64"), out_dtype)
    return _arith(lambda a, b: a / b, out_dtype, x, y)


def _promoted(dtype):
    """C's integer promotion: every type narrower than int computes as int."""
    d = str(dtype)
    return "int32" if _RANK[d] <= 2 else d


def _wrap_int(v, dtype):
    """A Python int as the two's-complement value of a C integer type.  Signed overflow is undefined in C;
    the hosts and devices the reference runs on wrap, and so does this restatement."""
    bits = np.dtype(dtype).itemsize * 8
    v &= (1 << bits) - 1
    if np.dtype(dtype).kind == "i" and v >= (1 << (bits - 1)):
        v -= 1 << bits
    return v


class _C(object):
    """One C integer value with its type, for the element-by-element restatements: arithmetic follows the
    usual arithmetic conversions, / and % truncate."""

    def __init__(self, v, dtype):
        self.t = _promoted(dtype)
        self.v = _wrap_int(int(v), self.t)

    def _pair(self, o):
        t = c_common_type(self.t, o.t)
        return _wrap_int(self.v, t), _wrap_int(o.v, t), t

    def neg(self):
        return _C(-self.v, self.t)

    def add(self, o):
        a, b, t = self._pair(o)
        return _C(a + b, t)

    def sub(self, o):
        a, b, t = self._pair(o)
        return _C(a - b, t)

    def div(self, o):
        a, b, t = self._pair(o)
        q = abs(a) // abs(b)
        return _C(-q if (a < 0) != (b < 0) else q, t)

    def mod(self, o):
        a, b, t = self._pair(o)
        q = abs(a) // abs(b)
        q = -q if (a < 0) != (b < 0) else q
        return _C(a - q * b, t)


def int_div(out_dtype, x, y):
    """theano/scalar/basic.py:2009-2025, element by element: the four sign cases over C's truncating
    division, every operand in its own C type (the sign tests see the operands as they are, the
    divisions the usual common type)."""
    ct = c_common_type(x.dtype, y.dtype)
    if np.dtype(ct).kind == "f":
        with np.errstate(all="ignore"):
            return _conv(np.floor(_conv(x, ct) / _conv(y, ct)), out_dtype)
    x, y = np.broadcast_arrays(np.asarray(x), np.asarray(y))
    res = np.zeros(x.shape, dtype=object)
    one, zero = _C(1, "int32"), _C(0, "int32")
    for idx in np.ndindex(x.shape):
        a, b = _C(x[idx], x.dtype), _C(y[idx], y.dtype)
        if b.v == 0:
            continue
        if b.v < 0:
            if a.v < 0:
                r = a.neg().div(b.neg())
            else:
                r = a.div(b.neg()).neg().sub(zero if a.mod(b.neg()).v == 0 else one)
        else:
            if a.v < 0:
                r = a.neg().div(b).neg().sub(zero if a.neg().mod(b).v == 0 else one)
            else:
                r = a.div(b)
        res[idx] = r.v
    return _wrap(res, out_dtype)


def mod(out_dtype, x, y):
    """theano/scalar/basic.py:2119-2135, element by element: remainder with the divisor's sign.  The floating-point
    text (fmod over doubles) also serves integer operands whose node type is float64: int64 beside uint64."""
    ct = c_common_type(x.dtype, y.dtype)
    if np.dtype(ct).kind == "f" or np.promote_types(np.asarray(x).dtype, np.asarray(y).dtype).kind == "f":
        a, b = np.broadcast_arrays(_conv(x, "float64"), _conv(y, "float64"))
        with np.errstate(all="ignore"):
            r = np.where(b == 0, np.fmod(a, b),
                         np.where(b < 0,
                                  np.where(a < 0, -np.fmod(-a, -b),
                                           np.fmod(a, -b) + np.where(np.fmod(a, -b) != 0, b, 0)),
                                  np.where(a < 0, -np.fmod(-a, b) + np.where(np.fmod(-a, b) != 0, b, 0),
                                           np.fmod(a, b))))
        return _conv(r, out_dtype)
    x, y = np.broadcast_arrays(np.asarray(x), np.asarray(y))
    res = np.zeros(x.shape, dtype=object)
    zero = _C(0, "int32")
    for idx in np.ndindex(x.shape):
        a, b = _C(x[idx], x.dtype), _C(y[idx], y.dtype)
        if b.v == 0:
            continue
        if b.v < 0:
            if a.v < 0:
                r = a.neg().mod(b.neg()).neg()
            else:
                m = a.mod(b.neg())
                r = m.add(b if m.v != 0 else zero)
        else:
            if a.v < 0:
                m = a.neg().mod(b)
                r = m.neg().add(b if m.v != 0 else zero)
            else:
                r = a.mod(b)
        res[idx] = r.v
    return _wrap(res, out_dtype)


def _wrap(obj_arr, dtype):
    """Python ints -> fixed-width integers with two's-complement wrap."""
    dt = np.dtype(dtype)
    if dt.kind == "f":
        return np.array(obj_arr, dtype="float64").astype(dt)
    bits = dt.itemsize * 8
    flat = np.array([int(v) & ((1 << bits) - 1) for v in obj_arr.reshape(-1)], dtype=object)
    if dt.kind == "i":
        flat = np.array([v - (1 << bits) if v >= (1 << (bits - 1)) else v for v in flat], dtype=object)
    return flat.astype(dt).reshape(obj_arr.shape)


def _cneg(a):
    """-a in C: in the promoted type, wrapping."""
    with np.errstate(all="ignore"):
        return -_conv(a, _promoted(a.dtype))


def _cbin(fn, a, b):
    ct = c_common_type(a.dtype, b.dtype)
    with np.errstate(all="ignore"):
        return fn(_conv(a, ct), _conv(b, ct))


def _ctrunc_mod(a, b):
    return _cbin(np.fmod, a, b)                     # on integers: C's %, the sign of the dividend


def _ctrunc_div(a, b):
    return _cbin(lambda p, q: (p - np.fmod(p, q)) // q, a, b)       # exact after the remainder is taken off


def mod_fast(out_dtype, x, y):
    """Vectorised ``mod``: the same C expressions over whole arrays (NumPy's fixed-width integers wrap as the
    restatement's do); zero divisors give 0 as on the device."""
    ct = c_common_type(x.dtype, y.dtype)
    if np.dtype(ct).kind == "f" or np.promote_types(np.asarray(x).dtype, np.asarray(y).dtype).kind == "f":
        return mod(out_dtype, x, y)
    x, y = np.broadcast_arrays(np.asarray(x), np.asarray(y))
    y1 = np.where(y == 0, np.ones((), y.dtype), y)
    ny, nx = _cneg(y1), _cneg(x)
    izero = np.zeros((), "int32")
    yt = c_common_type(y.dtype, "int32")            # the type of (m != 0 ? y : 0)
    y_or_0 = lambda m: np.where(m != 0, _conv(y1, yt), np.zeros((), yt))                   # noqa: E731
    with np.errstate(all="ignore"):
        mm = _cneg(_ctrunc_mod(nx, ny))
        m = _ctrunc_mod(x, ny)
        pm = _cbin(np.add, m, y_or_0(m))
        m = _ctrunc_mod(nx, y1)
        mp = _cbin(np.add, _cneg(m), y_or_0(m))
        pp = _ctrunc_mod(x, y1)
    pick = lambda v: _conv(v, out_dtype)                                                   # noqa: E731
    r = np.where(y < 0, np.where(x < 0, pick(mm), pick(pm)), np.where(x < 0, pick(mp), pick(pp)))
    return np.where(y == 0, pick(izero), r).astype(out_dtype)


def int_div_fast(out_dtype, x, y):
    """Vectorised ``int_div``.  Integers: the same C expressions over whole arrays (zero divisors give 0 as on
    the device).  Floats follow the C text (``theano/scalar/basic.py:1985-2025``): ``floor(x / y)`` over the
    magnitudes with the quotient rounded in C's common type first - so a quotient that rounds up to an
    integer floors to that integer - and the sign cases corrected through ``fmod``."""
    ct = c_common_type(x.dtype, y.dtype)
    if np.dtype(ct).kind == "f":
        a, b = np.broadcast_arrays(_conv(x, ct), _conv(y, ct))
        with np.errstate(all="ignore"):
            pp = np.floor(a / b)
            mm = np.floor((-a) / (-b))
            pm = -np.floor(a / (-b)) - np.where(np.fmod(a, -b) == 0, 0, 1)
            mp = -np.floor((-a) / b) - np.where(np.fmod(-a, b) == 0, 0, 1)
            r = np.where(b == 0, pp, np.where(b < 0, np.where(a < 0, mm, pm), np.where(a < 0, mp, pp)))
        return _conv(r, out_dtype)
    x, y = np.broadcast_arrays(np.asarray(x), np.asarray(y))
    y1 = np.where(y == 0, np.ones((), y.dtype), y)
    ny, nx = _cneg(y1), _cneg(x)
    if np.promote_types(x.dtype, y.dtype).kind == "f":
        # int64 beside uint64: the node's type is float64, so the reference takes its floating-point text
        # (theano/scalar/basic.py:1985-2003) over integer operands - x / y is still C's integer division (in
        # unsigned long long), floor() and fmod() see doubles, and the sign corrections negate the doubles
        f = lambda v: np.asarray(v).astype("float64")                                      # noqa: E731
        with np.errstate(all="ignore"):
            mm = f(_ctrunc_div(nx, ny))
            pm = -f(_ctrunc_div(x, ny)) - np.where(np.fmod(f(x), f(ny)) == 0, 0.0, 1.0)
            mp = -f(_ctrunc_div(nx, y1)) - np.where(np.fmod(f(nx), f(y1)) == 0, 0.0, 1.0)
            pp = f(_ctrunc_div(x, y1))
        r = np.where(y < 0, np.where(x < 0, mm, pm), np.where(x < 0, mp, pp))
        return _conv(np.where(y == 0, 0.0, r), out_dtype)
    step = lambda m: np.where(m == 0, np.zeros((), "int32"), np.ones((), "int32"))        # noqa: E731
    with np.errstate(all="ignore"):
        mm = _ctrunc_div(nx, ny)
        pm = _cbin(np.subtract, _cneg(_ctrunc_div(x, ny)), step(_ctrunc_mod(x, ny)))
        mp = _cbin(np.subtract, _cneg(_ctrunc_div(nx, y1)), step(_ctrunc_mod(nx, y1)))
        pp = _ctrunc_div(x, y1)
    pick = lambda v: _conv(v, out_dtype)                                                   # noqa: E731
    r = np.where(y < 0, np.where(x < 0, pick(mm), pick(pm)), np.where(x < 0, pick(mp), pick(pp)))
    return np.where(y == 0, pick(np.zeros((), "int32")), r).astype(out_dtype)


def pow_(out_dtype, x, y):
    with np.errstate(all="ignore"):
        return _conv(np.power(x.astype("float64"), y.astype("float64")), out_dtype)


def _pick(out_dtype, x, y, first):
    """``y OP x ? y : (x OP= y ? x : nan)`` (theano/scalar/basic.py:1632-1639, 1669-1675): the comparisons are
    made in C's common type, the operand that wins is stored as itself - so beside a uint64 a negative int8
    compares as a huge number and is then stored as the negative number it is."""
    ct = c_common_type(x.dtype, y.dtype)
    xs, ys = np.broadcast_arrays(np.asarray(x), np.asarray(y))
    a, b = _conv(xs, ct), _conv(ys, ct)
    with np.errstate(all="ignore"):
        take_y = (b > a) if first == "max" else (b < a)
        take_x = (a >= b) if first == "max" else (a <= b)
        if np.dtype(out_dtype).kind in "fc":
            rest = np.where(take_x, _conv(xs, out_dtype), np.asarray(np.nan, out_dtype))
        else:
            rest = _conv(xs, out_dtype)       # integers always compare one way or the other
        return np.where(take_y, _conv(ys, out_dtype), rest).astype(out_dtype)


def maximum(out_dtype, x, y):
    return _pick(out_dtype, x, y, "max")


def minimum(out_dtype, x, y):
    return _pick(out_dtype, x, y, "min")


def _cmp(fn):
    def f(out_dtype, x, y):
        ct = c_common_type(x.dtype, y.dtype)
        return fn(_conv(x, ct), _conv(y, ct))
    return f


lt, gt, le, ge, eq, neq = (_cmp(np.less), _cmp(np.greater), _cmp(np.less_equal), _cmp(np.greater_equal),
                           _cmp(np.equal), _cmp(np.not_equal))


def in_range(openlow, openhi):
    """``InRange.c_code`` (``theano/scalar/basic.py:1452-1460``): ``x > low && x < hi`` with ``>=`` / ``<=``
    at a closed end; each comparison converts its two operands as C does."""
    lo, hi = (gt if openlow else ge), (lt if openhi else le)

    def f(out_dtype, x, low, high):
        return np.logical_and(lo(out_dtype, x, low), hi(out_dtype, x, high))
    return f


def _angle_unit(factor):
    """``Deg2Rad`` / ``Rad2Deg.c_code`` (``theano/scalar/basic.py:3110-3149``): ``z = x * (M_PI / 180.0)`` resp.
    ``x * (180.0 / M_PI)`` - the product is taken in double precision whatever x is (an integer, a float32 and a
    float16 operand all promote to double against the double constant), then converted to the result type."""
    def f(out_dtype, x):
        prod = x.astype("float64") * np.float64(factor)
        if str(out_dtype) == "float16":       # float16 values are computed as float and stored as half
            prod = _conv(prod, "float32")
        return _conv(prod, out_dtype)
    return f


deg2rad, rad2deg = _angle_unit(np.pi / 180.0), _angle_unit(180.0 / np.pi)


def _bit(fn):
    def f(out_dtype, x, y):
        if str(out_dtype) == "bool":
            return fn(x != 0, y != 0)
        return _arith(fn, out_dtype, x, y)
    return f


and_, or_, xor = _bit(np.bitwise_and), _bit(np.bitwise_or), _bit(np.bitwise_xor)
right_shift = _bit(np.right_shift)
left_shift = _bit(np.left_shift)


def invert(out_dtype, x):
    if str(out_dtype) == "bool":
        return x == 0
    return _conv(np.invert(_conv(x, c_common_type(x.dtype))), out_dtype)


def isnan(out_dtype, x):
    return np.isnan(x) if x.dtype.kind == "f" else np.zeros(x.shape, bool)


def isinf(out_dtype, x):
    return np.isinf(x) if x.dtype.kind == "f" else np.zeros(x.shape, bool)


def switch(out_dtype, c, a, b):
    ct = c_common_type(a.dtype, b.dtype)
    return _conv(np.where(c != 0, _conv(a, ct), _conv(b, ct)), out_dtype)


def clip(out_dtype, x, lo, hi):
    """``z = x < min ? min : (x > max ? max : x)`` (theano/scalar/basic.py:2240-2243): each comparison in the common
    type of its own two operands; the inner conditional has the common type of max and x, the outer one that of
    min and the inner - an int8 -128 beside a uint32 max becomes 4294967168 before an int64 min widens it."""
    x, lo, hi = np.broadcast_arrays(np.asarray(x), np.asarray(lo), np.asarray(hi))
    inner_t = c_common_type(hi.dtype, x.dtype)
    outer_t = c_common_type(lo.dtype, inner_t)
    with np.errstate(all="ignore"):
        below, above = _cbin(np.less, x, lo), _cbin(np.greater, x, hi)
        inner = np.where(above, _conv(hi, inner_t), _conv(x, inner_t))
    return _conv(np.where(below, _conv(lo, outer_t), _conv(inner, outer_t)), out_dtype)


def second(out_dtype, x, y):
    return _conv(np.broadcast_arrays(x, y)[1], out_dtype)


def identity(out_dtype, x):
    return _conv(x, out_dtype)


def cast(out_dtype, x):
    return _conv(x, out_dtype)


def neg(out_dtype, x):
    return _arith(lambda a: -a, out_dtype, x)


def abs_(out_dtype, x):
    return _conv(np.abs(x), out_dtype)


def sgn(out_dtype, x):
    return _conv(np.sign(x), out_dtype)


def inv(out_dtype, x):
    with np.errstate(all="ignore"):
        return _conv(1.0 / _conv(x, "float64") if x.dtype != np.float32 and x.dtype != np.float16
                     else (np.float64(1.0) / x.astype("float64")), out_dtype)


def sqr(out_dtype, x):
    return _arith(lambda a: a * a, out_dtype, x)


def _libm(fn):
    """``z = f((out_t)x)``: the input is cast to the output type first."""
    def f(out_dtype, x):
        ct = "float32" if str(out_dtype) == "float16" else out_dtype
        with np.errstate(all="ignore"):
            return _conv(fn(_conv(x, ct)), out_dtype)
    return f


exp, exp2, expm1 = _libm(np.exp), _libm(np.exp2), _libm(np.expm1)
log, log2, log10, log1p = _libm(np.log), _libm(np.log2), _libm(np.log10), _libm(np.log1p)
sqrt, ceil, floor = _libm(np.sqrt), _libm(np.ceil), _libm(np.floor)
cos, sin, tan = _libm(np.cos), _libm(np.sin), _libm(np.tan)
arccos, arcsin, arctan = _libm(np.arccos), _libm(np.arcsin), _libm(np.arctan)
cosh, sinh, tanh = _libm(np.cosh), _libm(np.sinh), _libm(np.tanh)
arccosh, arcsinh, arctanh = _libm(np.arccosh), _libm(np.arcsinh), _libm(np.arctanh)
trunc = _libm(np.trunc)
round_half_to_even = _libm(np.rint)


def _c_round(a):
    """C ``round()`` (the reference's C text, ``theano/scalar/basic.py:2686``): the nearest integer, halves
    away from zero.  ``floor(a + 0.5)`` - what the reference's Python ``impl`` does (:2640-2643) - is not the
    same function: ``a + 0.5`` is itself rounded, so 0.49999997f becomes 1 and odd integers from 2**23
    up move by one.  Exact here: ``a - trunc(a)`` has no rounding error."""
    t = np.trunc(a)
    return t + np.copysign((np.abs(a - t) >= 0.5).astype(a.dtype), a)


round_half_away_from_zero = _libm(_c_round)


def _special(name):
    """scipy.special is what the reference's ``impl`` calls for these ops
    (``theano/scalar/basic_scipy.py:32-36`` and alike)."""
    def f(out_dtype, x):
        import scipy.special
        ct = "float32" if str(out_dtype) == "float16" else out_dtype
        with np.errstate(all="ignore"):
            return _conv(getattr(scipy.special, name)(_conv(x, ct)), out_dtype)
    return f


erf, erfc, erfcx = _special("erf"), _special("erfc"), _special("erfcx")
erfinv, erfcinv = _special("erfinv"), _special("erfcinv")
gamma, gammaln, psi = _special("gamma"), _special("gammaln"), _special("psi")


def tri_gamma(out_dtype, x):
    import scipy.special
    ct = "float32" if str(out_dtype) == "float16" else out_dtype
    with np.errstate(all="ignore"):
        return _conv(scipy.special.polygamma(1, _conv(x, ct)), out_dtype)


j0, j1, i0, i1 = _special("j0"), _special("j1"), _special("i0"), _special("i1")


def _special2(fn):
    """Binary scipy functions: both arguments in the output's compute type."""
    def f(out_dtype, a, b):
        ct = "float32" if str(out_dtype) == "float16" else out_dtype
        with np.errstate(all="ignore"):
            return _conv(fn(_conv(a, ct).astype("float64"), _conv(b, ct).astype("float64")), out_dtype)
    return f


def _sp():
    import scipy.special
    return scipy.special


gammainc = _special2(lambda k, x: _sp().gammainc(k, x))
gammaincc = _special2(lambda k, x: _sp().gammaincc(k, x))
gammau = _special2(lambda k, x: _sp().gammaincc(k, x) * _sp().gamma(k))       # basic_scipy.py:631-632
gammal = _special2(lambda k, x: _sp().gammainc(k, x) * _sp().gamma(k))        # basic_scipy.py:674-675


def chi2sf(out_dtype, x, k):
    import scipy.stats
    with np.errstate(all="ignore"):
        return _conv(scipy.stats.chi2.sf(np.asarray(x, "float64"), np.asarray(k, "float64")), out_dtype)


def arctan2(out_dtype, y, x):
    ct = "float32" if str(out_dtype) == "float16" else out_dtype
    return _conv(np.arctan2(_conv(y, ct), _conv(x, ct)), out_dtype)


def scalar_sigmoid(out_dtype, x):
    """theano/tensor/nnet/sigm.py:78-85; integer operands have no C code there and go through the Python
    ``impl`` (:36-46): 0 below -30, 1 above 30, the plain formula in between."""
    if np.asarray(x).dtype.kind in "biu":
        xd = np.asarray(x).astype("float64")
        with np.errstate(all="ignore"):
            return _conv(np.where(xd < -30.0, 0.0, np.where(xd > 30.0, 1.0, 1.0 / (1.0 + np.exp(-xd)))), out_dtype)
    if str(x.dtype) in ("float32", "float16"):
        xf = x.astype("float32")
        with np.errstate(all="ignore"):
            r = np.where(xf < np.float32(-88.0), np.float32(0),
                         np.where(xf > np.float32(15.0), np.float32(1),
                                  np.float32(1) / (np.float32(1) + np.exp(-xf))))
        return _conv(r, out_dtype)
    xd = x.astype("float64")
    with np.errstate(all="ignore"):
        r = np.where(xd < -709.0, 0.0, np.where(xd > 19.0, 1.0, 1.0 / (1.0 + np.exp(-xd))))
    return _conv(r, out_dtype)


def scalar_softplus(out_dtype, x):
    """theano/tensor/nnet/sigm.py:356-360; integer operands through the Python ``impl`` (:336-346): 0 below -30,
    x above 30, log1p(exp(x)) in between."""
    if np.asarray(x).dtype.kind in "biu":
        xd = np.asarray(x).astype("float64")
        with np.errstate(all="ignore"):
            return _conv(np.where(xd < -30.0, 0.0, np.where(xd > 30.0, xd, np.log1p(np.exp(xd)))), out_dtype)
    if str(x.dtype) in ("float32", "float16"):
        xf = x.astype("float32")
        with np.errstate(all="ignore"):
            r = np.where(xf < np.float32(-103.0), np.float32(0), np.where(xf > np.float32(14.0), xf,
                                                                          np.log1p(np.exp(xf))))
        return _conv(r, out_dtype)
    xd = x.astype("float64")
    with np.errstate(all="ignore"):
        r = np.where(xd < -745.0, 0.0, np.where(xd > 16.0, xd, np.log1p(np.exp(xd))))
    return _conv(r, out_dtype)


def ultra_fast_scalar_sigmoid(out_dtype, x):
    """theano/tensor/nnet/sigm.py:210-229 (the C text): pieces in double, rounded to the output type at
    each assignment to a variable of that type."""
    ot = np.dtype(out_dtype)
    h = (0.5 * x.astype("float64")).astype(ot)

    def piece(v):
        v = v.astype("float64")
        return np.where(v < 1.7, 1.5 * v / (1 + v), np.where(v < 3, 0.935409070603099 + 0.0458812946797165 * (v - 1.7),
                                                             0.99505475368673))
    with np.errstate(all="ignore"):
        t = np.where(h >= 0, piece(h), -piece(-h)).astype(ot)
    return _conv((0.5 * (t.astype("float64") + 1.0)).astype(ot), out_dtype)


def sigmoid_binary_crossentropy(out_dtype, x, t):
    """theano/tensor/nnet/nnet.py:2048: softplus(-abs(x)) + x * ((x > 0) - t), every step in the output's
    compute type."""
    ct = "float32" if str(out_dtype) == "float16" else out_dtype
    xc, tc = _conv(x, ct), _conv(t, ct)
    sp = scalar_softplus(ct, -np.abs(xc))
    return _conv(sp + xc * ((xc > 0).astype(ct) - tc), out_dtype)


def scalar_softsign(out_dtype, x):
    """theano/tensor/nnet/nnet.py:2511: x / (1.0 + fabs(x)), in double, rounded on assignment."""
    xd = x.astype("float64")
    return _conv((xd / (1.0 + np.abs(xd))).astype(np.dtype(out_dtype)), out_dtype)


# ---- Bessel functions of real order ------------------------------------------------------------
# theano/scalar/basic_scipy.py:698-726, 786-811: scipy.special.jv / iv themselves.
jv = _special2(lambda v, x: _sp().jv(v, x))
iv = _special2(lambda v, x: _sp().iv(v, x))


# ---- complex numbers ---------------------------------------------------------------------------
# The reference evaluates every op on complex values through NumPy on the host (``impl``; only +, -, *, /,
# unary -, abs, == and casts also have C text, theano/scalar/basic.py:498-641, 2459-2460): operands are
# converted to the result type and NumPy's complex loops do the rest.  These restatements are those NumPy
# calls.  Pinning (tests/test_oracle_scalar.py): the four arithmetic operations against the reference's C
# struct formulas written out in real arithmetic; exp / log / sqrt / sin / cos / sinh / cosh / tanh against
# their definitions through real functions (Euler's formula, log|z| + i arg z, the principal root squared
# back, the addition theorems); pow against repeated multiplication; abs against hypot; real, imag, conj,
# angle, complex and complex_from_polar against hand-written values.
def _is_complex(dt):
    return str(dt).startswith("complex")


def _cwide(out_dtype, *xs):
    with np.errstate(all="ignore"):
        return [_conv(x, out_dtype) for x in xs]


def _cplx_unary(npfn):
    def f(out_dtype, x):
        with np.errstate(all="ignore"):
            return _conv(npfn(_conv(x, out_dtype)), out_dtype)
    return f


def _cplx_nary(npfn):
    def f(out_dtype, *xs):
        with np.errstate(all="ignore"):
            r = _conv(xs[0], out_dtype)
            for x in xs[1:]:
                r = npfn(r, _conv(x, out_dtype))
            return _conv(r, out_dtype)
    return f


def _cplx_compare(npfn):
    def f(out_dtype, a, b):
        up = np.result_type(np.asarray(a).dtype, np.asarray(b).dtype)
        return npfn(_conv(a, up), _conv(b, up))
    return f


def real(out_dtype, x):
    return _conv(np.real(x), out_dtype)


def imag(out_dtype, x):
    return _conv(np.imag(x), out_dtype)


def angle(out_dtype, x):
    return _conv(np.angle(x), out_dtype)


def conj(out_dtype, x):
    return _conv(np.conj(x), out_dtype)


def complex_(out_dtype, x, y):
    part = "float32" if str(out_dtype) == "complex64" else "float64"
    r = np.empty(np.broadcast(x, y).shape, out_dtype)
    r.real, r.imag = _conv(x, part), _conv(y, part)
    return r


def complex_from_polar(out_dtype, r, theta):
    """theano/scalar/basic.py:3746-3753: (r cos theta, r sin theta) in the precision of the result's parts."""
    part = "float32" if str(out_dtype) == "complex64" else "float64"
    rr, tt = _conv(r, part), _conv(theta, part)
    return complex_(out_dtype, rr * np.cos(tt), rr * np.sin(tt))


COMPLEX_BY_CLASS = {
    "Add": _cplx_nary(np.add), "Mul": _cplx_nary(np.multiply), "Sub": _cplx_nary(np.subtract),
    "TrueDiv": _cplx_nary(np.divide), "Pow": _cplx_nary(np.power), "Neg": _cplx_unary(np.negative),
    "Sqr": _cplx_unary(np.square), "Inv": _cplx_unary(np.reciprocal), "Exp": _cplx_unary(np.exp),
    "Expm1": _cplx_unary(np.expm1), "Log": _cplx_unary(np.log), "Log2": _cplx_unary(np.log2),
    "Log10": _cplx_unary(np.log10), "Log1p": _cplx_unary(np.log1p), "Sqrt": _cplx_unary(np.sqrt),
    "Sin": _cplx_unary(np.sin), "Cos": _cplx_unary(np.cos), "Tan": _cplx_unary(np.tan), "Sinh": _cplx_unary(np.sinh),
    "Cosh": _cplx_unary(np.cosh), "Tanh": _cplx_unary(np.tanh), "Identity": _cplx_unary(lambda x: x),
    "Cast": _cplx_unary(lambda x: x), "Conj": conj,
    "Abs": lambda out_dtype, x: _conv(np.abs(x), out_dtype),
    "EQ": _cplx_compare(np.equal), "NEQ": _cplx_compare(np.not_equal),
    "IsNan": lambda out_dtype, x: np.isnan(x), "IsInf": lambda out_dtype, x: np.isinf(x),
    "Switch": lambda out_dtype, c, a, b: np.where(np.asarray(c) != 0, _conv(a, out_dtype), _conv(b, out_dtype)),
    "Second": lambda out_dtype, x, y: _conv(np.broadcast_to(y, np.broadcast(x, y).shape), out_dtype),
    "Real": real, "Imag": imag, "Angle": angle, "Complex": complex_, "ComplexFromPolar": complex_from_polar,
}


def restatement(class_name, out_dtype, in_dtypes):
    """The function restating scalar op ``class_name`` for these operand types."""
    if _is_complex(out_dtype) or any(_is_complex(d) for d in in_dtypes):
        fn = COMPLEX_BY_CLASS.get(class_name)
        if fn is None:
            raise NotImplementedError("no restatement of scalar op %s over complex numbers" % class_name)
        return fn
    return BY_CLASS.get(class_name)


# scalar op class name -> restatement
BY_CLASS = {
    "Add": add, "Mul": mul, "Sub": sub, "TrueDiv": true_div, "IntDiv": int_div_fast, "Mod": mod_fast, "Pow": pow_,
    "Maximum": maximum, "Minimum": minimum, "LT": lt, "GT": gt, "LE": le, "GE": ge, "EQ": eq, "NEQ": neq,
    "AND": and_, "OR": or_, "XOR": xor, "RightShift": right_shift, "LeftShift": left_shift, "Invert": invert,
    "IsNan": isnan, "IsInf": isinf, "Switch": switch, "Clip": clip, "Second": second, "Identity": identity,
    "Cast": cast, "Neg": neg, "Abs": abs_, "Sgn": sgn, "Inv": inv, "Sqr": sqr, "Exp": exp, "Exp2": exp2,
    "Expm1": expm1, "Log": log, "Log2": log2, "Log10": log10, "Log1p": log1p, "Sqrt": sqrt, "Ceil": ceil,
    "Floor": floor, "Trunc": trunc, "RoundHalfToEven": round_half_to_even,
    "RoundHalfAwayFromZero": round_half_away_from_zero, "Cos": cos, "Sin": sin, "Tan": tan, "ArcCos": arccos,
    "ArcSin": arcsin, "ArcTan": arctan, "ArcTan2": arctan2, "Cosh": cosh, "Sinh": sinh, "Tanh": tanh,
    "ArcCosh": arccosh, "ArcSinh": arcsinh, "ArcTanh": arctanh, "ScalarSigmoid": scalar_sigmoid,
    "ScalarSoftplus": scalar_softplus, "Erf": erf, "Erfc": erfc, "Erfcx": erfcx, "Erfinv": erfinv, "Erfcinv": erfcinv,
    "Gamma": gamma, "GammaLn": gammaln, "Psi": psi, "TriGamma": tri_gamma, "J0": j0, "J1": j1, "I0": i0, "I1": i1,
    "GammaInc": gammainc, "GammaIncC": gammaincc, "GammaU": gammau, "GammaL": gammal, "Chi2SF": chi2sf,
    "UltraFastScalarSigmoid": ultra_fast_scalar_sigmoid, "ScalarSoftsign": scalar_softsign,
    "SigmoidBinaryCrossentropy": sigmoid_binary_crossentropy, "Jv": jv, "Iv": iv,
    "Real": real, "Imag": imag, "Angle": angle, "Conj": conj, "Complex": complex_,
    "ComplexFromPolar": complex_from_polar, "Deg2Rad": deg2rad, "Rad2Deg": rad2deg,
}
