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
        if cost.type.dtype not in scal.continuous_dtypes:
            raise TypeError("cost must be floating point, not %s" % cost.type.dtype)
        grads[cost] = T.ones_like(cost)
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
        for o in node.outputs:
            g = grads.get(o)
            if g is None:
                ograds.append(DisconnectedType()())
            else:
                connected = True
                ograds.append(g)
        if not connected:
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
            if g.type.dtype not in scal.continuous_dtypes:
                continue
            if hasattr(i.type, "broadcastable") and g.type.broadcastable != i.type.broadcastable:
                g = _match_broadcast(g, i)
            grads[i] = g if i not in grads else T.add(grads[i], g)

    result = []
    for w in wrt_list:
        g = grads.get(w)
        if g is None:
            if disconnected_inputs == "raise":
                raise DisconnectedInputError("grad method was asked to compute the gradient with respect to a "
                                             "variable that is not part of the computational graph of the cost: %s" % w)
            dt = w.type.dtype if w.type.dtype in scal.continuous_dtypes else config.floatX
            g = T.zeros_like(w, dtype=dt)
        result.append(g)
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
