"""The ops either side of an elementwise / reduction island: basic indexing,
its scatter-back gradient, reshaping, broadcasting fills and joining.

Graph-level mirrors of ``Subtensor`` / ``IncSubtensor``
(``theano/tensor/subtensor.py:318-780, 1175-1560``), ``Reshape`` / ``flatten``
(``theano/tensor/basic.py:4701-4920, 5160-5220``), ``Alloc`` (:2769-2960) and
``Join`` / ``Split`` (:4120-4470, 3700-3860), restricted to what needs no
host-side integer arithmetic in the graph: indices and slice bounds are Python
integers, and shapes that depend on run-time extents are written as "like
dimension d of input k".  None of them computes on the host: ``perform``
exists only on the device subclasses (``theano_amd/hip/views.py``), where a
view costs nothing and a copy is one elementwise kernel.
"""
import numpy as np

from .. import scalar as scal
from ..gof import Apply, Op
from . import basic as T
from .type import TensorType, as_tensor_variable


def _no_host(op):
    raise NotImplementedError("%s runs on the device only; compile the graph with function()" % op)


# --------------------------------------------------------------------------
class Sym(object):
    """Place of the k-th scalar input of the node in an index: ``x[i]`` or ``x[a:b]`` with
    integer scalar variables, read on the host when the function runs
    (``theano/tensor/subtensor.py:318-420`` keeps scalar types in ``idx_list`` the same way)."""

    __slots__ = ("k",)

    def __init__(self, k):
        self.k = int(k)

    def __eq__(self, other):
        return type(other) is Sym and other.k == self.k

    def __hash__(self):
        return hash(("Sym", self.k))

    def __repr__(self):
        return "i%d" % self.k


def _is_index_variable(v):
    if not hasattr(v, "type") or not hasattr(v, "owner"):
        return False
    dt = getattr(v.type, "dtype", "")
    if getattr(v.type, "ndim", 0) != 0 or not (dt.startswith("int") or dt.startswith("uint")):
        raise TypeError("a symbolic index must be an integer scalar, got %s" % (v.type,))
    return True


def split_symbolic(idx_list):
    """(template, variables): every scalar variable in ``idx_list`` replaced by a ``Sym``."""
    syms = []

    def place(f):
        if _is_index_variable(f):
            for k, v in enumerate(syms):
                if v is f:
                    return Sym(k)
            syms.append(f)
            return Sym(len(syms) - 1)
        return f

    out = []
    for i in idx_list:
        if isinstance(i, slice):
            out.append(slice(place(i.start), place(i.stop), place(i.step)))
        else:
            out.append(place(i))
    return tuple(out), syms


def resolve_index(template, values):
    """The concrete index for the run-time ``values`` of the node's scalar inputs."""
    def val(f):
        return int(np.asarray(values[f.k])) if type(f) is Sym else f
    return tuple(slice(val(i.start), val(i.stop), val(i.step)) if isinstance(i, slice) else val(i) for i in template)


def n_symbolic(template):
    ks = [f.k for i in template for f in ((i.start, i.stop, i.step) if isinstance(i, slice) else (i,)) if type(f) is Sym]
    return max(ks) + 1 if ks else 0


def normalize_index(idx, ndim):
    """A tuple of ints and slices (with int / None fields), one per indexed
    dimension; Ellipsis expands, missing trailing dimensions are full slices.
    Integer scalar variables may stand where integers do."""
    if not isinstance(idx, tuple):
        idx = (idx,)
    if sum(1 for i in idx if i is Ellipsis) > 1:
        raise IndexError("an index can only have a single ellipsis")
    if any(i is None for i in idx):
        raise NotImplementedError("newaxis in an index: use dimshuffle")
    n_real = sum(1 for i in idx if i is not Ellipsis)
    if n_real > ndim:
        raise IndexError("too many indices for a tensor of rank %d" % ndim)
    out = []
    for i in idx:
        if i is Ellipsis:
            out.extend([slice(None)] * (ndim - n_real))
        elif isinstance(i, slice):
            for f in (i.start, i.stop, i.step):
                if f is not None and not isinstance(f, (int, np.integer)) and not _is_index_variable(f):
                    raise NotImplementedError("slice bounds must be integers or integer scalar variables (got %r)" % (f,))
            if isinstance(i.step, (int, np.integer)) and i.step == 0:
                raise ValueError("slice step cannot be zero")
            out.append(slice(*[f if (f is None or hasattr(f, "type")) else int(f) for f in (i.start, i.stop, i.step)]))
        elif isinstance(i, (int, np.integer)):
            out.append(int(i))
        elif _is_index_variable(i):
            out.append(i)
        else:
            raise NotImplementedError("only integers, integer scalar variables and slices index a tensor here "
                                      "(got %r)" % (i,))
    out.extend([slice(None)] * (ndim - len(out)))
    return tuple(out)


def index_view(shape, strides, offset, idx_list):
    """(shape, strides, offset) of ``x[idx_list]`` for an array header, with
    NumPy's rules: negative indices count from the end, an integer out of range
    raises IndexError, slice bounds are clipped."""
    new_shape, new_strides = [], []
    for d, i in enumerate(idx_list):
        n, st = shape[d], strides[d]
        if isinstance(i, slice):
            start, stop, step = i.indices(n)
            length = len(range(start, stop, step))
            offset += start * st
            new_shape.append(length)
            new_strides.append(st * step)
        else:
            j = i + n if i < 0 else i
            if j < 0 or j >= n:
                raise IndexError("index %d is out of bounds for axis %d with size %d" % (i, d, n))
            offset += j * st
    return tuple(new_shape), tuple(new_strides), offset


def _idx_key(idx_list):
    return tuple(("s", i.start, i.stop, i.step) if isinstance(i, slice) else ("i", i) for i in idx_list)


def _full_slice(i):
    return isinstance(i, slice) and i.start is None and i.stop is None and i.step is None


class Subtensor(Op):
    """``x[idx_list]`` with integers and slices, constant or given by integer scalar
    variables (the node's further inputs): a view
    (``theano/tensor/subtensor.py:318-780``; ``view_map = {0: [0]}`` :513)."""

    __props__ = ("idx_key",)
    view_map = {0: [0]}

    def __init__(self, idx_list):
        self.idx_list = tuple(idx_list)
        self.idx_key = _idx_key(self.idx_list)

    def _props(self):
        return (self.idx_key,)

    def __str__(self):
        def one(i):
            if isinstance(i, slice):
                return ":".join("" if f is None else str(f) for f in (i.start, i.stop, i.step))
            return str(i)
        return "%s{%s}" % (type(self).__name__, ", ".join(one(i) for i in self.idx_list))

    def out_broadcastable(self, in_broadcastable):
        # a full slice keeps the flag (theano/tensor/subtensor.py:470-500); any other slice may be empty
        return tuple(b and _full_slice(i) for b, i in zip(in_broadcastable, self.idx_list) if isinstance(i, slice))

    def check_inputs(self, x, scalars):
        if len(self.idx_list) != x.type.ndim:
            raise IndexError("index of %d entries for a tensor of rank %d" % (len(self.idx_list), x.type.ndim))
        if len(scalars) != n_symbolic(self.idx_list):
            raise ValueError("the index names %d scalar inputs, %d were given" % (n_symbolic(self.idx_list), len(scalars)))
        for v in scalars:
            _is_index_variable(v)

    def make_node(self, x, *scalars):
        x = as_tensor_variable(x)
        scalars = [as_tensor_variable(v) for v in scalars]
        self.check_inputs(x, scalars)
        return Apply(self, [x] + scalars, [TensorType(x.type.dtype, self.out_broadcastable(x.type.broadcastable))()])

    def infer_shape(self, node, shapes):
        if n_symbolic(self.idx_list):
            raise NotImplementedError("the shape of a symbolic slice is known only when the function runs")
        shape, _, _ = index_view(shapes[0], [1] * len(shapes[0]), 0, self.idx_list)
        return [shape]

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def connection_pattern(self, node):
        return [[True]] + [[False]] * (len(node.inputs) - 1)

    def L_op(self, inputs, outputs, grads):
        x = inputs[0]
        (g,) = grads
        return [IncSubtensor(self.idx_list)(x.zeros_like(), g, *inputs[1:])] + [T.scal.DisconnectedType()() for _ in inputs[1:]]

    def R_op(self, inputs, eval_points):
        if eval_points[0] is None:
            return [None]
        return [self(eval_points[0], *inputs[1:])]


class IncSubtensor(Op):
    """``x`` with ``x[idx_list]`` incremented by (or set to) ``y``
    (``theano/tensor/subtensor.py:1175-1560``).  A new array: the input is not
    modified."""

    __props__ = ("idx_key", "set_instead_of_inc")

    def __init__(self, idx_list, set_instead_of_inc=False):
        self.idx_list = tuple(idx_list)
        self.idx_key = _idx_key(self.idx_list)
        self.set_instead_of_inc = bool(set_instead_of_inc)

    def _props(self):
        return (self.idx_key, self.set_instead_of_inc)

    def __str__(self):
        return "%s{%s;%s}" % (type(self).__name__, "Set" if self.set_instead_of_inc else "Inc",
                              str(Subtensor(self.idx_list))[len("Subtensor{"):-1])

    def make_node(self, x, y, *scalars):
        x, y = as_tensor_variable(x), as_tensor_variable(y)
        scalars = [as_tensor_variable(v) for v in scalars]
        if y.type.dtype != x.type.dtype:
            y = T.cast(y, x.type.dtype)
        sub = Subtensor(self.idx_list).make_node(x, *scalars).outputs[0]
        if y.type.ndim > sub.type.ndim:
            raise TypeError("the increment has rank %d, the indexed region rank %d" % (y.type.ndim, sub.type.ndim))
        return Apply(self, [x, y] + scalars, [x.type()])

    def connection_pattern(self, node):
        return [[True], [True]] + [[False]] * (len(node.inputs) - 2)

    def infer_shape(self, node, shapes):
        return [shapes[0]]

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def R_op(self, inputs, eval_points):
        if None in eval_points[:2]:
            return [None]
        return [self(eval_points[0], eval_points[1], *inputs[2:])]

    def L_op(self, inputs, outputs, grads):
        x, y = inputs[:2]
        scalars = list(inputs[2:])
        (g,) = grads
        gy = Subtensor(self.idx_list)(g, *scalars)
        # y may have been broadcast into the region: sum the gradient back (subtensor.py:1520-1560)
        sub_ndim = gy.type.ndim
        if y.type.ndim < sub_ndim:
            gy = T.sum(gy, axis=tuple(range(sub_ndim - y.type.ndim)))
        bdims = [d for d in range(y.type.ndim) if y.type.broadcastable[d] and not gy.type.broadcastable[d]]
        if bdims:
            gy = T.sum(gy, axis=tuple(bdims), keepdims=True)
        if self.set_instead_of_inc:
            gx = IncSubtensor(self.idx_list, True)(g, T.zeros_like(Subtensor(self.idx_list)(g, *scalars)), *scalars)
        else:
            gx = g
        return [gx, gy] + [T.scal.DisconnectedType()() for _ in scalars]


def subtensor(x, idx):
    x = as_tensor_variable(x)
    idx_list = normalize_index(idx, x.type.ndim)
    # x[:] is a node of its own, as in the reference (set_subtensor(x[:], y) needs it); canonicalisation
    # takes it out of a compiled graph (local_useless_subtensor)
    template, syms = split_symbolic(idx_list)
    return Subtensor(template)(x, *syms)


def _inc_or_set(x, y, idx, set_instead_of_inc):
    x = as_tensor_variable(x)
    if idx is None:
        # the reference's calling convention: inc_subtensor(x[idx], y) - the first argument is the
        # indexed view, the op is applied to what it indexes (theano/tensor/subtensor.py:1040-1110)
        if x.owner is None or not isinstance(x.owner.op, Subtensor):
            raise TypeError("x must be the result of a subtensor operation (or pass the index as third argument)")
        template, syms, x = x.owner.op.idx_list, list(x.owner.inputs[1:]), x.owner.inputs[0]
    else:
        template, syms = split_symbolic(normalize_index(idx, x.type.ndim))
    return IncSubtensor(template, set_instead_of_inc)(x, y, *syms)


def inc_subtensor(x, y, idx=None):
    """``inc_subtensor(x[idx], y)`` as in the reference, or ``inc_subtensor(x, y, idx)``: a copy of
    the indexed tensor with the region incremented by ``y``."""
    return _inc_or_set(x, y, idx, False)


def set_subtensor(x, y, idx=None):
    """``set_subtensor(x[idx], y)`` or ``set_subtensor(x, y, idx)``."""
    return _inc_or_set(x, y, idx, True)


# --------------------------------------------------------------------------
# --------------------------------------------------------------------------
# Entries of the shape patterns of Reshape and Alloc:
#   n               a plain extent (Reshape: -1 = inferred)
#   (k, d)          the extent of dimension d of input k
#   ("in", k)       the value of input k, an integer scalar read on the host when the function runs
#   ("vec", k, j, n) element j of input k, an integer vector of n elements (n = -1: of any length) read on the host
#                   when the function runs (reshape(x, shape_vector, ndim=n), alloc(v, shape_vector[0], ...)); in a
#                   Reshape such an element may be -1
#   (op, a, b)      op in _SHAPE_OPS over two entries: arithmetic on extents, evaluated on the host from array
#                   metadata (x.reshape((x.shape[0], x.shape[1] * x.shape[2])), alloc(0., n // 2, m + 1), ...)
_SHAPE_OPS = {"add": lambda a, b: a + b, "sub": lambda a, b: a - b, "mul": lambda a, b: a * b,
              "floordiv": lambda a, b: a // b, "mod": lambda a, b: a % b, "max": max, "min": min}


def _norm_entry(p, allow_unknown):
    if isinstance(p, tuple):
        if len(p) == 2 and p[0] == "in":
            return ("in", int(p[1]))
        if len(p) == 4 and p[0] == "vec":
            return ("vec", int(p[1]), int(p[2]), int(p[3]))
        if len(p) == 3 and p[0] in _SHAPE_OPS:
            return (p[0], _norm_entry(p[1], False), _norm_entry(p[2], False))
        if len(p) == 2 and not isinstance(p[0], str):
            return (int(p[0]), int(p[1]))
        raise ValueError("invalid shape entry %r" % (p,))
    p = int(p)
    if p < (-1 if allow_unknown else 0):
        raise ValueError("invalid extent %d in a shape" % p)
    return p


def _entry_inputs(p):
    """Indices of the node inputs an entry reads."""
    if not isinstance(p, tuple):
        return []
    if p[0] in ("in", "vec"):
        return [p[1]]
    if p[0] in _SHAPE_OPS:
        return _entry_inputs(p[1]) + _entry_inputs(p[2])
    return [p[0]]


def _eval_entry(p, shapes, values):
    if not isinstance(p, tuple):
        return p
    if p[0] == "in":
        if values is None:
            raise ValueError("this shape depends on the value of an input, not only on shapes")
        v = values[p[1]]
        return int(np.asarray(v.to_numpy() if hasattr(v, "to_numpy") else v).reshape(()))
    if p[0] == "vec":
        if values is None:
            raise ValueError("this shape depends on the value of an input, not only on shapes")
        v = values[p[1]]
        v = np.asarray(v.to_numpy() if hasattr(v, "to_numpy") else v)
        if v.ndim != 1 or (v.shape[0] != p[3] if p[3] >= 0 else v.shape[0] <= p[2]):
            # theano/tensor/basic.py:4918-4921
            raise ValueError("shape argument has incorrect length %s, should be %s" % (
                v.shape, p[3] if p[3] >= 0 else "more than %d" % p[2]))
        return int(v[p[2]])
    if p[0] in _SHAPE_OPS:
        return int(_SHAPE_OPS[p[0]](_eval_entry(p[1], shapes, values), _eval_entry(p[2], shapes, values)))
    return int(shapes[p[0]][p[1]])


def vector_inputs(pattern):
    """Indices of the inputs a pattern reads as whole integer vectors (on the host)."""
    out = set()

    def walk(p):
        if isinstance(p, tuple):
            if p[0] == "vec":
                out.add(p[1])
            elif p[0] in _SHAPE_OPS:
                walk(p[1])
                walk(p[2])
    for p in pattern:
        walk(p)
    return out


def _entry_str(p):
    if not isinstance(p, tuple):
        return str(p)
    if p[0] == "in":
        return "in%d" % p[1]
    if p[0] == "vec":
        return "in%d[%d]" % (p[1], p[2])
    if p[0] in _SHAPE_OPS:
        return "%s(%s, %s)" % (p[0], _entry_str(p[1]), _entry_str(p[2]))
    return "in%d.shape[%d]" % p


def _entry_broadcastable(p, ins):
    if isinstance(p, tuple):
        return ins[p[0]].type.broadcastable[p[1]] if not isinstance(p[0], str) else False
    return p == 1


def _check_entries(pattern, ins):
    for p in pattern:
        for k in _entry_inputs(p):
            if k >= len(ins):
                raise ValueError("shape entry %s refers to a missing input" % _entry_str(p))
    for p in pattern:
        if isinstance(p, tuple) and not isinstance(p[0], str) and p[1] >= ins[p[0]].type.ndim:
            raise ValueError("shape entry %s refers to a missing input dimension" % (p,))


class Reshape(Op):
    """``x`` with a new shape (``theano/tensor/basic.py:4701-4920``).  ``pattern``
    has one entry per output dimension: a non-negative int, ``-1`` (at most one,
    inferred), ``(k, d)``: the extent of dimension ``d`` of input ``k``, ``("in", k)``: the
    run-time value of the integer scalar input ``k``, or arithmetic over such entries.
    Inputs after the first are read for their shape (or scalar value) only.  A view when the
    input is C-contiguous, else a copy."""

    __props__ = ("pattern",)
    view_map = {0: [0]}

    def __init__(self, pattern):
        pat = [_norm_entry(p, True) for p in pattern]
        if sum(1 for p in pat if p == -1) > 1:
            raise ValueError("can only specify one unknown dimension")
        self.pattern = tuple(pat)

    def _props(self):
        return (self.pattern,)

    def __str__(self):
        return "%s{%s}" % (type(self).__name__, ", ".join(_entry_str(p) for p in self.pattern))

    def make_node(self, x, *like):
        ins = [as_tensor_variable(x)] + [as_tensor_variable(v) for v in like]
        _check_entries(self.pattern, ins)
        bcast = [_entry_broadcastable(p, ins) for p in self.pattern]
        return Apply(self, ins, [TensorType(ins[0].type.dtype, bcast)()])

    def resolve(self, shapes, values=None):
        """The concrete output shape given the inputs' shapes (and, for entries that read an input's value,
        the inputs themselves)."""
        total = 1
        for s in shapes[0]:
            total *= s
        out, known, unknown = [], 1, None
        for j, p in enumerate(self.pattern):
            v = _eval_entry(p, shapes, values)
            if v < -1 or (v == -1 and isinstance(p, tuple) and p[0] != "vec"):
                raise ValueError("negative extent %d from shape entry %s" % (v, _entry_str(p)))
            if v == -1:
                if unknown is not None:
                    raise ValueError("can only specify one unknown dimension")
                unknown = j
                out.append(-1)
            else:
                out.append(int(v))
                known *= int(v)
        if unknown is not None:
            if known == 0 or total % known:
                raise ValueError("cannot reshape array of size %d into shape %s" % (total, tuple(out)))
            out[unknown] = total // known
        elif known != total:
            raise ValueError("cannot reshape array of size %d into shape %s" % (total, tuple(out)))
        return tuple(out)

    def infer_shape(self, node, shapes):
        return [self.resolve(shapes)]

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def L_op(self, inputs, outputs, grads):
        x = inputs[0]
        (g,) = grads
        gx = Reshape([(1, d) for d in range(x.type.ndim)])(g, x)
        if gx.type != x.type:          # broadcast flags the pattern could not know
            gx = T.DimShuffle(gx.type.broadcastable, list(range(x.type.ndim)))(gx)
        return [gx] + [v.zeros_like() for v in inputs[1:]]

    def R_op(self, inputs, eval_points):
        if eval_points[0] is None:
            return [None]
        return [self(eval_points[0], *inputs[1:])]

    def connection_pattern(self, node):
        return [[True]] + [[False]] * (len(node.inputs) - 1)


class _ShapeArgs(object):
    """Collects the inputs a shape pattern refers to while the entries given by the caller are
    translated: tensors whose extents are read, and integer scalars read for their value."""

    def __init__(self, first=None):
        self.ins = [] if first is None else [first]
        self.base = 1 if first is None else 0      # Alloc's input 0 is the value, never a shape source

    def index(self, v):
        for k, u in enumerate(self.ins):
            if u is v:
                return k + self.base
        self.ins.append(v)
        return len(self.ins) - 1 + self.base

    def extra(self):
        return self.ins[1:] if self.base == 0 else self.ins

    def entry(self, p):
        """The pattern entry for one element of a shape argument: an int, ``v.shape[d]``, a pair ``(v, d)``,
        an integer scalar variable, or arithmetic (+ - * // % maximum minimum) over those."""
        from .elemwise import DimShuffle, Elemwise
        if isinstance(p, (tuple, list)):
            if (len(p) == 2 and hasattr(p[0], "type") and isinstance(p[1], (int, np.integer)) and
                    0 <= p[1] < getattr(p[0].type, "ndim", 0)):
                return (self.index(as_tensor_variable(p[0])), int(p[1]))
            raise TypeError("invalid shape entry %r" % (p,))
        if not hasattr(p, "owner"):
            return int(p)
        if hasattr(p, "data"):
            if np.asarray(p.data).size != 1:
                raise TypeError("a shape entry must be a scalar: %s" % p)
            return int(np.asarray(p.data).reshape(()))
        dt = getattr(p.type, "dtype", "")
        if not all(p.type.broadcastable) or not (dt.startswith("int") or dt.startswith("uint")):
            raise TypeError("a symbolic shape entry must be an integer scalar, got %s" % (p.type,))
        node = p.owner
        if node is not None:
            if (isinstance(node.op, Subtensor) and len(node.inputs) == 1 and node.inputs[0].type.ndim == 1 and
                    isinstance(node.op.idx_list[0], (int, np.integer)) and node.op.idx_list[0] >= 0 and
                    node.inputs[0].type.dtype in scal.discrete_dtypes):
                # shape_vector[j]: read from the vector on the host, no device round trip (length -1: any length
                # that has an element j)
                v = node.inputs[0]
                n = _vector_length(v)
                return ("vec", self.index(v), int(node.op.idx_list[0]), -1 if n is None else n)
            if isinstance(node.op, T.ShapeFloat):
                return (self.index(node.inputs[0]), node.op.i)
            if isinstance(node.op, DimShuffle):
                return self.entry(node.inputs[0])
            if isinstance(node.op, Elemwise):
                sop = node.op.scalar_op
                name = {scal.Add: "add", scal.Mul: "mul", scal.Sub: "sub", scal.IntDiv: "floordiv", scal.Mod: "mod",
                        scal.Maximum: "max", scal.Minimum: "min"}.get(type(sop))
                if isinstance(sop, (scal.Cast, scal.Identity)):
                    return self.entry(node.inputs[0])
                if name is not None and len(node.inputs) >= 2:
                    e = self.entry(node.inputs[0])
                    for other in node.inputs[1:]:
                        e = (name, e, self.entry(other))
                    return e
        return ("in", self.index(p))


def _vector_length(v):
    """The number of elements of the integer vector variable ``v`` when the graph tells it (a constant, a join
    or stack of scalars; ``get_vector_length``, ``theano/tensor/basic.py:4470-4550``), else None."""
    if hasattr(v, "data"):
        return int(np.asarray(v.data).shape[0])
    node = v.owner
    if node is not None and isinstance(node.op, Join) and node.op.axis == 0:
        parts = [_vector_length(i) for i in node.inputs]
        return None if any(n is None for n in parts) else sum(parts)
    if node is not None and type(node.op).__name__ == "DimShuffle" and node.inputs[0].type.ndim == 0 and v.type.ndim == 1:
        return 1
    return None


def reshape(x, newshape, ndim=None):
    """``newshape``: a list of ints (at most one -1), ``v.shape[d]`` entries, integer scalar variables and arithmetic
    over those - or ONE integer vector (a constant, or a variable read on the host when the function runs, whose
    length ``ndim`` gives when the graph does not tell it; ``theano/tensor/basic.py:4858-4960, 5049-5068``).  An
    element of a run-time vector may be -1, as in NumPy."""
    x = as_tensor_variable(x)
    if hasattr(newshape, "owner") and getattr(newshape.type, "ndim", 0) == 1:
        vec = newshape
        dt = vec.type.dtype
        if not (dt.startswith("int") or dt.startswith("uint")):
            raise TypeError("Shape must be integers", vec, dt)
        if hasattr(vec, "data"):
            newshape = [int(n) for n in np.asarray(vec.data)]
            if ndim is not None and ndim != len(newshape):
                raise ValueError("the shape has %d entries, ndim says %d" % (len(newshape), ndim))
        else:
            n = _vector_length(vec)
            if n is None:
                n = ndim
            elif ndim is not None and ndim != n:
                raise ValueError("the shape vector has %d entries, ndim says %d" % (n, ndim))
            if n is None:
                raise ValueError("The length of the provided shape (%s) cannot be automatically determined, so the "
                                 "number of dimensions of the reshaped variable is unknown. You can provide the "
                                 "'ndim' keyword argument to 'reshape' to avoid this problem." % vec)
            args = _ShapeArgs(x)
            k = args.index(vec)
            return Reshape([("vec", k, j, n) for j in range(n)])(x, *args.extra())
    elif hasattr(newshape, "owner") and getattr(newshape.type, "ndim", 0) > 1:
        raise TypeError("New shape in reshape must be a vector or a list/tuple of scalar. Got %s" % newshape)
    if isinstance(newshape, (int, np.integer)) or hasattr(newshape, "owner"):
        newshape = (newshape,)
    if ndim is not None and ndim != len(newshape):
        raise ValueError("the shape has %d entries, ndim says %d" % (len(newshape), ndim))
    args = _ShapeArgs(x)
    pattern = [args.entry(p) for p in newshape]
    return Reshape(pattern)(x, *args.extra())


def flatten(x, ndim=None, outdim=None):
    """Keep the first ``ndim - 1`` dimensions, merge the rest
    (``theano/tensor/basic.py:5252-5310``; ``outdim`` is the older name of ``ndim``)."""
    if outdim is not None and ndim is not None:
        raise ValueError("You should only specify ndim")
    if outdim is not None:
        import warnings
        warnings.warn("flatten outdim parameter is deprecated, use ndim instead.")
        ndim = outdim
    if ndim is None:
        ndim = 1
    x = as_tensor_variable(x)
    if ndim < 1 or ndim > max(x.type.ndim, 1):
        raise ValueError("invalid output ndimensions (%d) for flatten" % ndim)
    if x.type.ndim == ndim:
        return x
    return Reshape([(0, d) for d in range(ndim - 1)] + [-1])(x)


# --------------------------------------------------------------------------
class Alloc(Op):
    """``value`` broadcast to a shape (``theano/tensor/basic.py:2769-2960``).
    ``pattern`` as for :class:`Reshape` without ``-1``; inputs after the first
    are read for their shape only."""

    __props__ = ("pattern",)

    def __init__(self, pattern):
        self.pattern = tuple(_norm_entry(p, False) for p in pattern)

    def _props(self):
        return (self.pattern,)

    def __str__(self):
        return "%s{%s}" % (type(self).__name__, ", ".join(_entry_str(p) for p in self.pattern))

    def make_node(self, value, *like):
        ins = [as_tensor_variable(value)] + [as_tensor_variable(v) for v in like]
        v = ins[0]
        if v.type.ndim > len(self.pattern):
            raise TypeError("the value has more dimensions (%d) than the shape (%d)" % (v.type.ndim, len(self.pattern)))
        _check_entries(self.pattern, ins)
        bcast = [_entry_broadcastable(p, ins) for p in self.pattern]
        return Apply(self, ins, [TensorType(v.type.dtype, bcast)()])

    def resolve(self, shapes, values=None):
        out = tuple(_eval_entry(p, shapes, values) for p in self.pattern)
        if any(v < 0 for v in out):
            raise ValueError("negative extent in shape %s" % (out,))
        return out

    def infer_shape(self, node, shapes):
        return [self.resolve(shapes)]

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def L_op(self, inputs, outputs, grads):
        v = inputs[0]
        (g,) = grads
        nd_out, nd_v = len(self.pattern), v.type.ndim
        gv = g
        if nd_out > nd_v:
            gv = T.sum(gv, axis=tuple(range(nd_out - nd_v)))
        b = [d for d in range(nd_v) if v.type.broadcastable[d] and not gv.type.broadcastable[d]]
        if b:
            gv = T.sum(gv, axis=tuple(b), keepdims=True)
        if gv.type.dtype != v.type.dtype:
            gv = T.cast(gv, v.type.dtype)
        return [gv] + [i.zeros_like() for i in inputs[1:]]

    def R_op(self, inputs, eval_points):
        if eval_points[0] is None:
            return [None]
        return [self(eval_points[0], *inputs[1:])]

    def connection_pattern(self, node):
        return [[True]] + [[False]] * (len(node.inputs) - 1)


def alloc(value, *shape):
    """``shape`` entries: ints, ``v.shape[d]``, integer scalar variables, arithmetic over those."""
    args = _ShapeArgs()
    pattern = [args.entry(p) for p in shape]
    return Alloc(pattern)(value, *args.extra())


# --------------------------------------------------------------------------
class Join(Op):
    """Concatenation along ``axis`` (``theano/tensor/basic.py:4120-4470``)."""

    __props__ = ("axis",)

    def __init__(self, axis):
        self.axis = int(axis)

    def _props(self):
        return (self.axis,)

    def __str__(self):
        return "%s{axis=%d}" % (type(self).__name__, self.axis)

    def make_node(self, *tensors):
        ts = [as_tensor_variable(t) for t in tensors]
        if not ts:
            raise ValueError("Cannot join an empty list of tensors")
        nd = ts[0].type.ndim
        if any(t.type.ndim != nd for t in ts):
            raise TypeError("Join() can only join tensors with the same number of dimensions.")
        if not 0 <= self.axis < nd:
            raise IndexError("Join axis %d out of bounds [0, %d)" % (self.axis, nd))
        dtype = ts[0].type.dtype
        for t in ts[1:]:
            dtype = T.scal.upcast(dtype, t.type.dtype)
        ts = [t if t.type.dtype == dtype else T.cast(t, dtype) for t in ts]
        # a dimension is broadcastable when it is in any input (then all must have extent 1); never the joined one
        bcast = [any(t.type.broadcastable[d] for t in ts) for d in range(nd)]
        bcast[self.axis] = len(ts) == 1 and ts[0].type.broadcastable[self.axis]
        return Apply(self, ts, [TensorType(dtype, bcast)()])

    def infer_shape(self, node, shapes):
        out = list(shapes[0])
        out[self.axis] = sum(s[self.axis] for s in shapes)
        return [tuple(out)]

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def L_op(self, inputs, outputs, grads):
        (g,) = grads
        if outputs[0].type.dtype not in T.continuous_dtypes:
            return [i.zeros_like(dtype=T.config.floatX) for i in inputs]
        return [JoinPart(self.axis, k)(g, *inputs) for k in range(len(inputs))]

    def R_op(self, inputs, eval_points):
        if None in eval_points:
            return [None]
        return [self(*eval_points)]


class JoinPart(Op):
    """The slice of a joined tensor that came from input ``k``: the gradient of
    ``Join`` (the role of ``Split``, ``theano/tensor/basic.py:3700-3860``).  The
    original tensors are read for their extents only.  A view."""

    __props__ = ("axis", "k")
    view_map = {0: [0]}

    def __init__(self, axis, k):
        self.axis, self.k = int(axis), int(k)

    def _props(self):
        return (self.axis, self.k)

    def __str__(self):
        return "%s{axis=%d, part=%d}" % (type(self).__name__, self.axis, self.k)

    def make_node(self, g, *tensors):
        g = as_tensor_variable(g)
        ts = [as_tensor_variable(t) for t in tensors]
        part = ts[self.k]
        return Apply(self, [g] + ts, [TensorType(g.type.dtype, part.type.broadcastable)()])

    def infer_shape(self, node, shapes):
        return [shapes[1 + self.k]]

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def connection_pattern(self, node):
        return [[True]] + [[False]] * (len(node.inputs) - 1)

    def L_op(self, inputs, outputs, grads):
        raise NotImplementedError("second derivatives through join are not implemented")


def join(axis, *tensors):
    ts = [as_tensor_variable(t) for t in tensors]
    nd = ts[0].type.ndim
    axis = axis + nd if axis < 0 else axis
    if len(ts) == 1:
        return ts[0]
    return Join(axis)(*ts)


concatenate = lambda tensors, axis=0: join(axis, *tensors)  # noqa: E731


def stack(*tensors, **kwargs):
    """``stack(tensors, axis=0)``: new axis at ``axis``, then join; ``stack(a, b, ...)`` is the older spelling of
    ``stack([a, b, ...], axis=0)`` (``theano/tensor/basic.py:4630-4745``)."""
    if not tensors and not kwargs:
        raise Exception("theano.tensor.stack(tensors, axis) must have at least one parameter")
    if not kwargs and not isinstance(tensors[0], (list, tuple)):
        import warnings
        warnings.warn("stack(*tensors) interface is deprecated, use stack(tensors, axis=0) instead.",
                      DeprecationWarning, stacklevel=2)
        axis = 0
    elif "tensors" in kwargs:
        tensors, axis = kwargs["tensors"], kwargs.get("axis", 0)
    else:
        axis = tensors[1] if len(tensors) == 2 else kwargs.get("axis", 0)
        tensors = tensors[0]
    if len(tensors) == 0:
        raise Exception("tensors is empty. You should at least provide one tensor to "
                        "theano.tensor.stack(tensors, axis).")
    ts = [as_tensor_variable(t) for t in tensors]
    nd = ts[0].type.ndim
    axis = axis + nd + 1 if axis < 0 else axis
    order = list(range(nd))
    order.insert(axis, "x")
    return join(axis, *[t.dimshuffle(*order) for t in ts])


def horizontal_stack(*args):
    """``concatenate(args, axis=1)`` of matrices (``theano/tensor/basic.py:4832-4851``)."""
    for a in args:
        if as_tensor_variable(a).type.ndim != 2:
            raise ValueError("Too many dimensions for horizontal_stack: use join")
    return concatenate(list(args), axis=1)


def vertical_stack(*args):
    """``concatenate(args, axis=0)`` of matrices (``theano/tensor/basic.py:4854-4865``)."""
    for a in args:
        if as_tensor_variable(a).type.ndim != 2:
            raise ValueError("Too many dimensions for vertical_stack: use join")
    return concatenate(list(args), axis=0)


def split(x, splits_size, n_splits, axis=0):
    """The ``n_splits`` consecutive parts of ``x`` along ``axis`` with the given (constant)
    lengths, as views (``theano/tensor/basic.py:3794-3797``; the reference's ``Split`` also takes
    symbolic lengths and checks that they add up to the extent when it runs)."""
    x = as_tensor_variable(x)
    sizes = [int(v) for v in splits_size]
    if len(sizes) != n_splits:
        raise ValueError("In Split.perform(), len(splits) != len_splits.", (len(sizes), n_splits))
    axis = axis + x.type.ndim if axis < 0 else axis
    parts, at = [], 0
    for n in sizes:
        idx = [slice(None)] * x.type.ndim
        idx[axis] = slice(at, at + n)
        parts.append(x[tuple(idx)])
        at += n
    return parts


class Rebroadcast(Op):
    """The same array with another static broadcast pattern: ``(axis, flag)`` pairs; making a
    dimension broadcastable is checked against its extent when the function runs
    (``theano/compile/ops.py:647-760``).  A view."""

    __props__ = ("axis",)
    view_map = {0: [0]}

    def __init__(self, *axis):
        items = sorted((int(a), bool(b)) for a, b in axis)
        self.axis = tuple(items)

    def _props(self):
        return (self.axis,)

    def __str__(self):
        flags = dict(self.axis)
        pattern = ["?"] * (1 + builtins_max(flags)) if flags else []
        for k, v in flags.items():
            pattern[k] = str(int(v))
        return "%s{%s}" % (type(self).__name__, ",".join(pattern))

    def out_type(self, x):
        flags = dict(self.axis)
        if flags and x.type.ndim <= builtins_max(flags):
            raise ValueError("Trying to rebroadcast non-existent dimension")
        return [flags.get(i, b) for i, b in enumerate(x.type.broadcastable)]

    def make_node(self, x):
        x = as_tensor_variable(x)
        return Apply(self, [x], [TensorType(x.type.dtype, self.out_type(x))()])

    def check(self, shape):
        for a, flag in self.axis:
            if flag and shape[a] != 1:
                raise ValueError("Dimension %s in Rebroadcast's input was supposed to be 1 (got %s instead)" % (a, shape[a]))

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def infer_shape(self, node, shapes):
        return [tuple(1 if dict(self.axis).get(d) else s for d, s in enumerate(shapes[0]))]

    def L_op(self, inputs, outputs, grads):
        # restore the input's pattern (theano/compile/ops.py:724-732)
        (x,) = inputs
        (g,) = grads
        return [Rebroadcast(*[(a, x.type.broadcastable[a]) for a, _ in self.axis])(g)]

    def R_op(self, inputs, eval_points):
        if eval_points[0] is None:
            return [None]
        return [self(eval_points[0])]


def builtins_max(d):
    import builtins
    return builtins.max(d)


def addbroadcast(x, *axes):
    """``theano/tensor/basic.py:4066-4093``"""
    x = as_tensor_variable(x)
    if any(a >= x.type.ndim for a in axes):
        raise ValueError("Trying to rebroadcast non-existent dimension")
    if all(x.type.broadcastable[a] for a in axes):
        return x
    return Rebroadcast(*[(a, True) for a in axes])(x)


def unbroadcast(x, *axes):
    """``theano/tensor/basic.py:4096-4123``"""
    x = as_tensor_variable(x)
    if any(a >= x.type.ndim for a in axes):
        raise ValueError("Trying to rebroadcast non-existent dimension")
    if not any(x.type.broadcastable[a] for a in axes):
        return x
    return Rebroadcast(*[(a, False) for a in axes])(x)


def patternbroadcast(x, broadcastable):
    """``theano/tensor/basic.py:4126-4153``"""
    x = as_tensor_variable(x)
    if tuple(x.type.broadcastable) == tuple(bool(b) for b in broadcastable):
        return x
    return Rebroadcast(*[(i, bool(b)) for i, b in enumerate(broadcastable)])(x)
