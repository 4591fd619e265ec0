"""Graph clean-ups run before a graph is lifted onto the device.

Only the rewrites that decide how much memory traffic the fused kernels do are
carried over from ``theano/tensor/opt.py``: DimShuffle merging / lifting
(``local_dimshuffle_lift`` :576-619), removal of useless elementwise nodes
(``local_useless_elemwise`` :1780-1860), the ``fill`` / ``second`` plumbing every
gradient produces (``local_fill_sink`` :1663-1707, ``local_useless_fill``
:1765-1779) and reduce canonicalisations (``local_sum_prod_all_to_none``
:5479-5494, ``local_reduce_broadcastable`` :5652-5702, ``local_useless_reduce``).
The algebraic canonizer is deliberately not reproduced.
"""
import numpy as np

from .. import gof
from .. import scalar as scal
from ..gof import local_optimizer
from . import basic as T
from .elemwise import CAReduce, DimShuffle, Elemwise
from .type import TensorConstant, TensorType, constant


@local_optimizer([DimShuffle])
def local_dimshuffle_fold(fgraph, node):
    """DimShuffle of a constant is a constant; DimShuffle of a DimShuffle is
    one DimShuffle; an identity DimShuffle is its input."""
    op = node.op
    (x,) = node.inputs
    if not isinstance(x.type, TensorType):
        return False
    if op.new_order == tuple(range(x.type.ndim)):
        return [x]
    if isinstance(x, TensorConstant):
        data = np.asarray(x.data)
        res = data.transpose(op.shuffle + op.drop) if data.ndim else data
        shape = list(res.shape[:len(op.shuffle)])
        for a in op.augment:
            shape.insert(a, 1)
        out = TensorConstant(node.outputs[0].type, np.asarray(res.reshape(shape), order="C"))
        return [out]
    if x.owner is not None and isinstance(x.owner.op, DimShuffle):
        inner = x.owner.op
        new_order = [o if o == "x" else inner.new_order[o] for o in op.new_order]
        base = x.owner.inputs[0]
        new = DimShuffle(base.type.broadcastable, new_order)(base)
        if new.type == node.outputs[0].type:
            return [new]
    return False


@local_optimizer([DimShuffle])
def local_dimshuffle_lift(fgraph, node):
    """DimShuffle(Elemwise(a, b)) -> Elemwise(DimShuffle(a), DimShuffle(b)) when
    nothing else uses the Elemwise result, so that permutations end up on the
    inputs of an elementwise island as strided views."""
    (x,) = node.inputs
    p = x.owner
    if p is None or not isinstance(p.op, Elemwise) or len(p.outputs) != 1 or fgraph.n_clients(x) != 1:
        return False
    if p.op.inplace_pattern:
        return False
    op = node.op
    new_inputs = [DimShuffle(i.type.broadcastable, op.new_order)(i) for i in p.inputs]
    new = p.op(*new_inputs)
    if new.type != node.outputs[0].type:
        return False
    return [new]


@local_optimizer([Elemwise])
def local_useless_elemwise(fgraph, node):
    """identity(x) -> x; second(x, y) -> y when y already has the full type;
    second(x, y) -> y' when x carries no shape (every dimension broadcastable)."""
    sop = node.op.scalar_op
    out = node.outputs[0]
    if isinstance(sop, scal.Identity) and node.inputs[0].type == out.type:
        return [node.inputs[0]]
    if isinstance(sop, scal.Cast) and node.inputs[0].type == out.type:
        return [node.inputs[0]]
    if isinstance(sop, (scal.Mul, scal.Add)) and len(node.inputs) >= 2:
        # drop neutral constants: mul(1, x) -> x, add(0, x) -> x (theano/tensor/opt.py local_mul_specialize /
        # local_add_specialize keep the same values)
        neutral = 1 if isinstance(sop, scal.Mul) else 0
        rest = [i for i in node.inputs
                if not (isinstance(i, TensorConstant) and all(i.type.broadcastable) and
                        np.all(np.asarray(i.data) == neutral) and i.type.dtype != "bool")]
        if len(rest) < len(node.inputs) and rest:
            new = rest[0] if len(rest) == 1 else node.op(*rest)
            if new.type == out.type:
                return [new]
    if isinstance(sop, scal.Pow):
        # x ** 2 -> sqr(x), x ** 1 -> x, x ** 0.5 -> sqrt(x), x ** -1 -> inv(x)
        # (local_pow_specialize, theano/tensor/opt.py:5918-5973)
        x, y = node.inputs
        if isinstance(y, TensorConstant) and all(y.type.broadcastable) and x.type.dtype == out.type.dtype:
            val = float(np.asarray(y.data).reshape(()))
            new = {2.0: T.sqr, 0.5: T.sqrt, -1.0: T.inv}.get(val)
            res = x if val == 1.0 else (new(x) if new is not None else None)
            if res is not None and res.type == out.type:
                return [res]
    if isinstance(sop, scal.Second):
        x, y = node.inputs
        if y.type == out.type:
            return [y]
        if y.type.dtype == out.type.dtype and y.type.ndim == out.type.ndim and all(
                xb or not yb for xb, yb in zip(x.type.broadcastable, y.type.broadcastable)):
            # x adds no extent that y lacks
            if y.type.broadcastable == out.type.broadcastable:
                return [y]
    return False


@local_optimizer([Elemwise])
def local_fill_sink(fgraph, node):
    """An elementwise consumer broadcasts anyway: f(second(a, b), c) -> f(b, c)
    as long as the other inputs still give the result its full pattern."""
    if isinstance(node.op.scalar_op, scal.Second) or len(node.outputs) != 1:
        return False
    out = node.outputs[0]
    new_inputs = list(node.inputs)
    changed = False
    for k, i in enumerate(node.inputs):
        p = i.owner
        if p is None or not isinstance(p.op, Elemwise) or not isinstance(p.op.scalar_op, scal.Second):
            continue
        a, b = p.inputs
        if b.type.dtype != i.type.dtype:
            continue
        trial = list(new_inputs)
        trial[k] = b
        pattern = [all(bb) for bb in zip(*[t.type.broadcastable for t in trial])]
        if tuple(pattern) == tuple(out.type.broadcastable):
            new_inputs = trial
            changed = True
    if not changed:
        return False
    new = node.op(*new_inputs)
    if new.type != out.type:
        return False
    return [new]


@local_optimizer([CAReduce])
def local_useless_reduce(fgraph, node):
    """A reduction over no axis is a cast; reducing only broadcastable
    dimensions of a sum/max/... is a DimShuffle that drops them."""
    op = node.op
    (x,) = node.inputs
    nd = x.type.ndim
    axis = tuple(range(nd)) if op.axis is None else op.axis
    out = node.outputs[0]
    if all(x.type.broadcastable[a] for a in axis):
        if isinstance(op.scalar_op, (scal.Add, scal.Mul, scal.Maximum, scal.Minimum, scal.AND, scal.OR)) or not axis:
            order = [d for d in range(nd) if d not in axis]
            new = DimShuffle(x.type.broadcastable, order)(x) if axis else x
            if new.type.dtype != out.type.dtype:
                new = T.cast(new, out.type.dtype)
            if new.type == out.type:
                return [new]
    return False


@local_optimizer([T.ShapeFloat])
def local_shape_lift(fgraph, node):
    """The extent of an elementwise / DimShuffle / reduction result is the extent
    of one of its inputs: ask the input, so that shape queries never keep an
    intermediate result alive (the role of ShapeFeature, theano/tensor/opt.py:970-1500)."""
    (x,) = node.inputs
    p = x.owner
    i = node.op.i
    if p is None:
        return False
    if isinstance(p.op, Elemwise):
        for v in p.inputs:
            if v.type.ndim == x.type.ndim and not v.type.broadcastable[i]:
                return [T.ShapeFloat(i, node.op.dtype)(v)]
        return False
    if isinstance(p.op, DimShuffle):
        src = p.op.new_order[i]
        if src == "x":
            return [constant(1, dtype=node.op.dtype)]
        return [T.ShapeFloat(src, node.op.dtype)(p.inputs[0])]
    if isinstance(p.op, CAReduce):
        nd = p.inputs[0].type.ndim
        axis = tuple(range(nd)) if p.op.axis is None else p.op.axis
        kept = [d for d in range(nd) if d not in axis]
        return [T.ShapeFloat(kept[i], node.op.dtype)(p.inputs[0])]
    return False


CANONICALIZE = [local_shape_lift, local_dimshuffle_fold, local_useless_elemwise, local_fill_sink, local_useless_reduce,
                local_dimshuffle_lift]


def canonicalize(fgraph):
    gof.merge_identical(fgraph)
    gof.apply_local(fgraph, CANONICALIZE)
    gof.merge_identical(fgraph)
    return fgraph
