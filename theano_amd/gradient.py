"""Reverse-mode differentiation over the graph: ``grad(cost, wrt)``.

A reduced form of ``theano/gradient.py`` (``grad`` :414, ``_populate_grad_dict``
:977-1430): walk the nodes between ``wrt`` and ``cost`` from the cost down,
ask every op for ``L_op(inputs, outputs, output_grads)`` and accumulate the
terms per variable.  Disconnected inputs yield zeros.
"""
import numpy as np

from . import gof
from . import scalar as scal
from .config import config
from .scalar import DisconnectedType


class DisconnectedInputError(ValueError):
    pass


class NullTypeGradError(TypeError):
    """The gradient asked for runs through a term an op declared not implemented or undefined."""


class NullType(gof.Type):
    """Type of the placeholder an ``L_op`` returns for a gradient it cannot give
    (``theano/gof/null_type.py``): no value, only a reason."""

    def __init__(self, why_null="(no default value given)"):
        self.why_null = why_null

    def filter(self, data, strict=False, allow_downcast=None):
        raise ValueError("No values may be assigned to a NullType")

    def __eq__(self, other):
        return type(self) == type(other)

    def __hash__(self):
        return hash(type(self))

    def __str__(self):
        return "NullType"


def grad_not_implemented(op, x_pos, x, comment=""):
    """What an ``L_op`` returns for input ``x_pos`` when that gradient is not implemented
    (``theano/gradient.py:1995-2034``); asking for it raises NullTypeGradError."""
    return NullType("This variable is Null because the grad method for input %s (%s) of the %s op is not "
                    "implemented. %s" % (x_pos, x, op, comment))()


def grad_undefined(op, x_pos, x, comment=""):
    """Same, for a gradient that is mathematically undefined (``theano/gradient.py:2037-2074``)."""
    return NullType("This variable is Null because the grad method for input %s (%s) of the %s op is "
                    "mathematically undefined. %s" % (x_pos, x, op, comment))()


def grad(cost, wrt, known_grads=None, disconnected_inputs="zero"):
    """Symbolic gradient of the 0-d ``cost`` with respect to ``wrt`` (a variable
    or a list of variables)."""
    from .tensor import basic as T
    from .tensor.type import as_tensor_variable

    single = not isinstance(wrt, (list, tuple))
    wrt_list = [wrt] if single else list(wrt)
    grads = {}
    if cost is not None:
        if cost.type.ndim != 0:
            raise TypeError("cost must be a scalar.")
        # an integer-valued cost has zero gradients everywhere (theano/gradient.py:_float_ones_like)
        grads[cost] = (T.ones_like(cost) if cost.type.dtype in scal.continuous_dtypes
                       else T.ones_like(cost, dtype=config.floatX))
    for var, g in (known_grads or {}).items():
        grads[var] = as_tensor_variable(g)
    outputs = list(grads.keys())

    # nodes on a path from wrt to the outputs
    order = gof.io_toposort([], outputs)
    depends = set(id(w) for w in wrt_list)
    for node in order:
        if any(id(i) in depends for i in node.inputs):
            for o in node.outputs:
                depends.add(id(o))

    for node in reversed(order):
        if not any(id(o) in depends for o in node.outputs):
            continue
        ograds = []
        connected = False
        null = None
        for o in node.outputs:
            g = grads.get(o)
            if g is None:
                ograds.append(DisconnectedType()())
            else:
                connected = True
                ograds.append(g)
                if isinstance(g.type, NullType):
                    null = g
        if not connected:
            continue
        if null is not None:
            # nothing can be said about what lies behind an unknown gradient
            for i in node.inputs:
                if id(i) in depends:
                    grads[i] = null
            continue
        if len(node.outputs) == 1 and getattr(node.outputs[0].type, "dtype", "float32") not in scal.continuous_dtypes:
            # integer-valued results carry no gradient to their inputs
            continue
        # replace missing output grads by zeros for ops that cannot take placeholders
        ograds = [T.zeros_like(o) if isinstance(g.type, DisconnectedType) and len(node.outputs) > 1 else g
                  for o, g in zip(node.outputs, ograds)]
        try:
            igrads = node.op.L_op(node.inputs, node.outputs, ograds)
        except gof.MethodNotDefined:
            raise NotImplementedError("%s does not define a gradient" % node.op)
        if len(igrads) != len(node.inputs):
            raise ValueError("%s.L_op returned %d gradients for %d inputs" % (node.op, len(igrads), len(node.inputs)))
        for i, g in zip(node.inputs, igrads):
            if g is None or isinstance(g.type, DisconnectedType):
                continue
            if id(i) not in depends:
                continue
            if isinstance(g.type, NullType):
                grads[i] = g
                continue
            if i in grads and isinstance(grads[i].type, NullType):
                continue
            if g.type.dtype not in scal.continuous_dtypes:
                continue
            if hasattr(i.type, "broadcastable") and g.type.broadcastable != i.type.broadcastable:
                g = _match_broadcast(g, i)
            grads[i] = g if i not in grads else T.add(grads[i], g)

    result = []
    for w in wrt_list:
        g = grads.get(w)
        if g is not None and isinstance(g.type, NullType):
            raise NullTypeGradError("grad encountered a NaN. " + g.type.why_null)
        if g is None:
            if disconnected_inputs == "raise":
                raise DisconnectedInputError("grad method was asked to compute the gradient with respect to a "
                                             "variable that is not part of the computational graph of the cost: %s" % w)
            dt = w.type.dtype if w.type.dtype in scal.continuous_dtypes else config.floatX
            g = T.zeros_like(w, dtype=dt)
        result.append(g)
    return result[0] if single else result


def Lop(f, wrt, eval_points):
    """L operator: eval_points times the Jacobian of ``f`` with respect to
    ``wrt`` (``theano/gradient.py:348-411``): reverse mode seeded with
    ``eval_points`` as the gradients of ``f``."""
    fs = list(f) if isinstance(f, (list, tuple)) else [f]
    eps = list(eval_points) if isinstance(eval_points, (list, tuple)) else [eval_points]
    if len(fs) != len(eps):
        raise ValueError("Lop needs one evaluation point per element of f")
    return grad(None, wrt, known_grads=dict(zip(fs, eps)))


def Rop(f, wrt, eval_points, disconnected_outputs="raise"):
    """R operator: the Jacobian of ``f`` with respect to ``wrt`` times
    ``eval_points`` (``theano/gradient.py:155-345``).  Forward mode: every node
    between ``wrt`` and ``f`` is asked for ``R_op(inputs, eval_points)``;
    graph inputs outside ``wrt`` contribute zeros."""
    from .tensor import basic as T
    from .tensor.type import as_tensor_variable

    single = not isinstance(f, (list, tuple))
    fs = [f] if single else list(f)
    wrt = list(wrt) if isinstance(wrt, (list, tuple)) else [wrt]
    eval_points = list(eval_points) if isinstance(eval_points, (list, tuple)) else [eval_points]
    if len(wrt) != len(eval_points):
        raise ValueError("Rop needs one evaluation point per element of wrt")
    eval_points = [as_tensor_variable(e) for e in eval_points]
    for k, (w, e) in enumerate(zip(wrt, eval_points)):
        if w.type.ndim != e.type.ndim:
            raise ValueError("Element %d of wrt/eval_point have mismatched dimensionality: %d versus %d"
                             % (k, w.type.ndim, e.type.ndim))
    point_of = dict((id(w), e) for w, e in zip(wrt, eval_points))
    seen = {}

    for node in gof.io_toposort([], fs):
        if any(id(o) in point_of for o in node.outputs) and all(id(o) in point_of for o in node.outputs):
            continue
        local = []
        for inp in node.inputs:
            if id(inp) in point_of:
                pt = point_of[id(inp)]
            elif inp.owner is None:
                pt = T.zeros_like(inp) if hasattr(inp.type, "broadcastable") else None
            else:
                pt = seen[id(inp.owner)][inp.owner.outputs.index(inp)]
            if pt is not None and hasattr(inp.type, "dtype") and pt.type.dtype != inp.type.dtype:
                pt = T.cast(pt, inp.type.dtype)
            local.append(pt)
        try:
            seen[id(node)] = node.op.R_op(node.inputs, local)
        except gof.MethodNotDefined:
            raise NotImplementedError("%s does not define R_op" % node.op)

    result = []
    for out in fs:
        if id(out) in point_of:
            result.append(point_of[id(out)])
            continue
        r = seen[id(out.owner)][out.owner.outputs.index(out)] if out.owner is not None else None
        if r is None:
            if disconnected_outputs == "raise":
                raise DisconnectedInputError("Rop method was asked to compute the gradient with respect to a variable "
                                             "that is not part of the computational graph of variables in wrt, or is "
                                             "used only by a non-differentiable operator: %s" % out)
            r = T.zeros_like(out)
        result.append(r)
    return result[0] if single else result


def _match_broadcast(g, var):
    """Make the gradient's static broadcast pattern equal to the variable's."""
    from .tensor import basic as T
    gb, vb = g.type.broadcastable, var.type.broadcastable
    if len(gb) != len(vb):
        raise ValueError("gradient of %s has rank %d, the variable has rank %d" % (var, len(gb), len(vb)))
    to_sum = [k for k, (a, b) in enumerate(zip(gb, vb)) if b and not a]
    if to_sum:
        g = T.sum(g, axis=to_sum, keepdims=True)
    if g.type.broadcastable != vb:
        # the gradient is broadcastable where the variable is not: expand it
        g = T.second(var, g)
    return g


def numeric_grad(f, pts, eps=None):
    """Central finite differences of the scalar function ``f`` at the list of
    float64 arrays ``pts`` (the check used by ``verify_grad``,
    ``theano/gradient.py:1435-1800``)."""
    pts = [np.array(p, dtype="float64") for p in pts]
    out = []
    for k, p in enumerate(pts):
        g = np.zeros_like(p)
        flat, gflat = p.reshape(-1), g.reshape(-1)
        for j in range(flat.size):
            old = flat[j]
            h = eps or 1e-6 * max(1.0, abs(old))
            flat[j] = old + h
            fp = f(*pts)
            flat[j] = old - h
            fm = f(*pts)
            flat[j] = old
            gflat[j] = (fp - fm) / (2 * h)
        out.append(g)
    return out
