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
from ..config import config
from ..gof import local_optimizer
from . import basic as T
from .elemwise import CAReduce, DimShuffle, Elemwise, Sum
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
    # dropping a broadcastable dimension and inserting one at the same place changes nothing
    if (len(op.new_order) == x.type.ndim and node.outputs[0].type == x.type and
            all(o == d or (o == "x" and x.type.broadcastable[d]) for d, o in enumerate(op.new_order))):
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
def local_useless_composite(fgraph, node):
    """An Elemwise of a Composite with several results, some of which nothing reads: the Composite is rebuilt
    with the results in use only (``theano/tensor/opt.py:7473-7491``)."""
    comp = node.op.scalar_op
    if not isinstance(comp, scal.Composite) or len(node.outputs) < 2:
        return False
    used = [i for i, o in enumerate(node.outputs) if fgraph.clients.get(o)]
    if not used or len(used) == len(node.outputs):
        return False
    smaller = scal.Composite(comp.inputs, [comp.outputs[i] for i in used])
    new = Elemwise(smaller).make_node(*node.inputs).outputs
    return {node.outputs[i]: n for i, n in zip(used, new)}


@local_optimizer([Elemwise])
def local_constant_fold(fgraph, node):
    """Arithmetic on scalar constants is done when the function is compiled
    (``constant_folding``, ``theano/tensor/opt.py:6600-6660``, restricted to
    all-broadcastable constants and to + - * / neg sqr inv cast, evaluated in
    the node's output dtype as the C expression would be): ``pow(x, 2.0 - 1)``
    from the gradient of a square becomes ``pow(x, 1.0)`` and then ``x``."""
    if len(node.outputs) != 1 or not node.inputs:
        return False
    out = node.outputs[0]
    odt = out.type.dtype
    if odt == "bool" or not all(isinstance(i, TensorConstant) and all(i.type.broadcastable) and
                                i.type.dtype != "bool" for i in node.inputs):
        return False
    sop = node.op.scalar_op
    vals = [np.asarray(i.data).reshape(()).astype(odt) for i in node.inputs]
    with np.errstate(all="ignore"):
        if isinstance(sop, scal.Add):
            res = vals[0]
            for v in vals[1:]:
                res = res + v
        elif isinstance(sop, scal.Mul):
            res = vals[0]
            for v in vals[1:]:
                res = res * v
        elif isinstance(sop, scal.Sub):
            res = vals[0] - vals[1]
        elif isinstance(sop, scal.TrueDiv) and odt in scal.float_dtypes:
            res = vals[0] / vals[1]
        elif isinstance(sop, scal.Neg):
            res = -vals[0]
        elif isinstance(sop, scal.Sqr):
            res = vals[0] * vals[0]
        elif isinstance(sop, scal.Inv) and odt in scal.float_dtypes:
            res = np.asarray(1, odt) / vals[0]
        elif isinstance(sop, (scal.Cast, scal.Identity)):
            src = np.asarray(node.inputs[0].data).reshape(())
            if odt not in scal.float_dtypes and not np.isfinite(src):
                return False
            res = src.astype(odt)
        else:
            return False
    new = TensorConstant(out.type, np.asarray(res, dtype=odt).reshape((1,) * out.type.ndim))
    return [new]


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


@local_optimizer([CAReduce])
def local_op_of_op(fgraph, node):
    """``Sum(Sum(x, a), b) -> Sum(x, a + b')`` and the same for ``Prod`` when nothing else reads
    the inner result (``theano/tensor/opt.py:5497-5563``): one pass, one rounding to the output
    dtype; ``Sum{every axis} -> Sum{None}`` so that equal reductions merge (:5479-5494)."""
    from .elemwise import Prod
    op = node.op
    if type(op) not in (Sum, Prod):
        return False
    (x,) = node.inputs
    cls = type(op)
    if op.axis is not None and set(op.axis) == set(range(x.type.ndim)) and x.type.ndim > 0:
        new = cls(None, dtype=op.dtype, acc_dtype=op.acc_dtype)(x)
        return [new] if new.type == node.outputs[0].type else False
    p = x.owner
    if p is None or type(p.op) is not cls or fgraph.n_clients(x) != 1:
        return False
    if p.op.axis is None or op.axis is None:
        new_axis = None
    else:
        new_axis = list(p.op.axis)
        for i in op.axis:                      # positions of the outer axes in the inner input
            j = i
            for ii in sorted(p.op.axis):
                if j >= ii:
                    j += 1
            new_axis.append(j)
    new = cls(new_axis, dtype=op.dtype)(p.inputs[0])
    return [new] if new.type == node.outputs[0].type else False


@local_optimizer([CAReduce])
def local_sum_invariant_factor(fgraph, node):
    """``sum(c * x, axis) -> c' * sum(x, axis)``, ``sum(x / c) -> sum(x) / c'`` and
    ``sum(-x) -> -sum(x)`` for every factor ``c`` that is constant along all the
    reduced axes (broadcastable there); ``c'`` is ``c`` without those axes.

    ``local_sum_prod_mul_by_scalar`` (``theano/tensor/opt.py:5062-5149``) does
    this for factors that are broadcastable everywhere; per-channel factors of a
    batch-norm gradient (``sum(g * gamma * (x - mean) / std**2, axis=(0, 2, 3))``)
    are the same case along the reduced axes only.  Products are searched
    through nested ``mul`` / ``true_div`` / ``neg`` nodes; other users of those nodes
    keep them.
    Floating point sums only: an integer sum in a wider dtype does not wrap where
    the narrower product would."""
    op = node.op
    if type(op) is not Sum:
        return False
    (x,) = node.inputs
    out = node.outputs[0]
    dt = x.type.dtype
    if dt not in scal.float_dtypes or out.type.dtype not in scal.float_dtypes or x.owner is None:
        return False
    nd = x.type.ndim
    axis = tuple(range(nd)) if op.axis is None else op.axis
    if not axis:
        return False

    def invariant(v):
        return v.type.ndim == nd and all(v.type.broadcastable[a] for a in axis)

    found = [False]

    def split(v):
        """(invariant factor or None, remaining factor or None, negated) with
        v == (-1 if negated) * invariant * remaining."""
        if invariant(v):
            return v, None, False
        p = v.owner
        if p is None or not isinstance(p.op, Elemwise) or v.type.dtype != dt:
            return None, v, False
        sop = p.op.scalar_op
        if isinstance(sop, scal.Mul):
            invs, rests, sign = [], [], False
            for t in p.inputs:
                if t.type.ndim != nd:
                    return None, v, False
                ci, ri, si = split(t)
                sign ^= si
                if ci is not None:
                    invs.append(ci)
                if ri is not None:
                    rests.append(ri)
            if not invs and not sign:
                return None, v, False
            found[0] = True
            inv = None if not invs else (invs[0] if len(invs) == 1 else T.mul(*invs))
            rest = None if not rests else (rests[0] if len(rests) == 1 else T.mul(*rests))
            return inv, rest, sign
        if isinstance(sop, scal.TrueDiv):
            a, b = p.inputs
            if a.type.ndim != nd or b.type.ndim != nd or a.type.dtype != dt or b.type.dtype != dt:
                return None, v, False
            ca, ra, sa = split(a)
            if invariant(b):
                found[0] = True
                inv = T.true_div(ca, b) if ca is not None else T.inv(b)
                return inv, ra, sa
            if ca is None and not sa:
                return None, v, False
            found[0] = True
            # an invariant numerator over a varying denominator leaves the reciprocal (not
            # ones / b: that quotient would be split again, forever)
            return ca, (T.true_div(ra, b) if ra is not None else T.inv(b)), sa
        if isinstance(sop, scal.Neg):
            ca, ra, sa = split(p.inputs[0])
            found[0] = True
            return ca, ra, not sa
        return None, v, False

    inv, rest, sign = split(x)
    if not found[0] or rest is None or (inv is None and not sign):
        return False
    if rest.type.dtype != dt:
        rest = T.cast(rest, dt)
    new = Sum(op.axis, dtype=op.dtype, acc_dtype=op.acc_dtype)(rest)
    if inv is not None:
        if inv.type.dtype != dt:
            return False
        keep = [d for d in range(nd) if d not in axis]
        new = T.mul(DimShuffle(inv.type.broadcastable, keep)(inv), new)
    if sign:
        new = T.neg(new)
    if new.type.dtype != out.type.dtype:
        new = T.cast(new, out.type.dtype)
    if new.type != out.type:
        return False
    return [new]


@local_optimizer([T.MaxAndArgmax])
def local_max_and_argmax(fgraph, node):
    """When nothing reads the argmax, the node is a plain ``max`` reduction
    (``local_max_and_argmax``, ``theano/tensor/opt_uncanonicalize.py:51-68``)."""
    if fgraph.n_clients(node.outputs[1]) != 0 or node.outputs[1] in fgraph.outputs:
        return False
    new = T.Max(node.op.axis)(node.inputs[0])
    if new.type != node.outputs[0].type:
        return False
    return [new, None]


@local_optimizer([Elemwise])
def local_max_to_min(fgraph, node):
    """``-max(-x) -> min(x)`` (``local_max_to_min``, ``theano/tensor/opt_uncanonicalize.py:71-94``), the form
    the reference's ``tensor.min`` writes.  Kept to floating-point operands, where negation is exact: over
    unsigned integers and at the most negative signed value the two sides differ."""
    if not isinstance(node.op.scalar_op, scal.Neg) or len(node.inputs) != 1:
        return False
    red = node.inputs[0].owner
    if red is None or not isinstance(red.op, CAReduce) or not isinstance(red.op.scalar_op, scal.Maximum):
        return False
    inner = red.inputs[0].owner
    if (inner is None or not isinstance(inner.op, Elemwise) or not isinstance(inner.op.scalar_op, scal.Neg) or
            len(inner.inputs) != 1):
        return False
    x = inner.inputs[0]
    if x.type.dtype not in scal.float_dtypes:
        return False
    new = T.Min(red.op.axis)(x)
    return [new] if new.type == node.outputs[0].type else False


def _grad_view_op():
    from ..gradient import _GradView
    return _GradView


@local_optimizer(None)
def local_remove_grad_views(fgraph, node):
    """``zero_grad`` / ``disconnected_grad`` / ``grad_clip`` / ``grad_scale`` nodes only matter while gradients
    are derived: in a graph that is compiled they stand for their operand (``local_grad_clip``,
    ``theano/tensor/opt.py:7500-7520``; the ViewOp removals of ``theano/compile/ops.py``)."""
    if not isinstance(node.op, _grad_view_op()):
        return False
    return [node.inputs[0]]


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


def _strip_broadcast_shuffle(v):
    """``v`` without DimShuffles that only insert or drop broadcastable dimensions."""
    while v.owner is not None and isinstance(v.owner.op, DimShuffle):
        order = [o for o in v.owner.op.new_order if o != "x"]
        if order != sorted(order):
            break
        v = v.owner.inputs[0]
    return v


def _extent_source(x, v, axes):
    """True when ``v`` is ``x`` or feeds ``x`` through Elemwise nodes without being
    broadcast along ``axes``: its extents along them are ``x``'s."""
    if x is v:
        return True
    if x.owner is None or not isinstance(x.owner.op, Elemwise):
        return False
    return any(i.type.ndim == x.type.ndim and not any(i.type.broadcastable[a] for a in axes) and
               _extent_source(i, v, axes) for i in x.owner.inputs)


@local_optimizer([Sum])
def local_single_pass_variance(fgraph, node):
    """``sum(sqr(x - mean(x, A)), A)`` on float16 / float32 data -> shifted sums in one pass:

        d = x - c,  c = the first element along A (per kept index)
        sum(sqr(x - mean)) = sum(d^2) - sum(d)^2 / N,      N = number of reduced elements

    with both sums accumulated in float64, so that the subtraction costs nothing the data's
    own precision could show (the shift keeps d within the spread of the data unless the first
    element is an outlier by many orders of magnitude).  The two sums read the same operand as
    the mean's own sum, so the three merge into one pass over x where the two-pass form of
    ``var`` (``theano/tensor/basic.py:3430-3459``) needs two.  float64 data keeps two passes:
    there is no wider accumulator to absorb the cancellation.  With nothing to reduce (an
    empty extent) taking the first element raises IndexError where the two-pass form yields NaN."""
    from ..config import config
    from .views import Subtensor
    if not config.single_pass_variance:
        return False
    (sq,) = node.inputs
    out = node.outputs[0]
    if out.type.dtype not in ("float32", "float64") or sq.type.dtype not in ("float16", "float32"):
        return False
    if sq.owner is None or not isinstance(sq.owner.op, Elemwise) or not isinstance(sq.owner.op.scalar_op, scal.Sqr):
        return False
    diff = sq.owner.inputs[0]
    if (diff.owner is None or not isinstance(diff.owner.op, Elemwise) or
            not isinstance(diff.owner.op.scalar_op, scal.Sub)):
        return False
    x, mb = diff.owner.inputs
    nd = x.type.ndim
    axes = tuple(range(nd)) if node.op.axis is None else tuple(node.op.axis)
    if not axes or x.type.dtype not in ("float16", "float32") or any(x.type.broadcastable[a] for a in axes):
        return False
    if mb.type.ndim != nd or not all(mb.type.broadcastable[a] for a in axes):
        return False
    # mean = sum(x, A) / extent / extent ... with one ShapeFloat divisor per reduced axis
    divisors, cur = [], _strip_broadcast_shuffle(mb)
    while (cur.owner is not None and isinstance(cur.owner.op, Elemwise) and
           isinstance(cur.owner.op.scalar_op, scal.TrueDiv)):
        divisors.append(_strip_broadcast_shuffle(cur.owner.inputs[1]))
        cur = _strip_broadcast_shuffle(cur.owner.inputs[0])
    if cur.owner is None or not isinstance(cur.owner.op, Sum) or cur.owner.inputs[0] is not x:
        return False
    m_axes = tuple(range(nd)) if cur.owner.op.axis is None else tuple(cur.owner.op.axis)
    if m_axes != axes:
        return False
    seen = []
    for dv in divisors:
        if dv.owner is None or not isinstance(dv.owner.op, T.ShapeFloat):
            return False
        if not _extent_source(x, dv.owner.inputs[0], axes):
            return False
        seen.append(dv.owner.op.i)
    if sorted(seen) != list(axes):
        return False
    # the shift: first element along the reduced axes, taken from the array the casts start from
    src = x
    while (src.owner is not None and isinstance(src.owner.op, Elemwise) and
           isinstance(src.owner.op.scalar_op, scal.Cast) and len(src.owner.inputs) == 1):
        src = src.owner.inputs[0]
    if src.owner is not None and isinstance(src.owner.op, Elemwise):
        return False            # x would have to be kept in memory only for the shift
    first = Subtensor([0 if d in axes else slice(None) for d in range(nd)])(src)
    order, k = [], 0
    for d in range(nd):
        if d in axes:
            order.append("x")
        else:
            order.append(k)
            k += 1
    cb = DimShuffle(first.type.broadcastable, order)(first)
    if src is x:
        d = T.sub(x, cb)
    else:
        a, c0 = scal.Scalar(x.type.dtype)(), scal.Scalar(src.type.dtype)()
        d = Elemwise(scal.Composite([a, c0], [scal.sub(a, scal.cast(c0, x.type.dtype))]))(x, cb)
    if src.type.dtype != "float16":
        d = T.cast(d, "float64")      # squares exact, and one fused multiply-add per element
    # float16 storage: d stays float32 (exact: both operands hold 11 bits), its square is rounded to
    # float32 (2**-24, nothing next to the data's own 2**-11) and the kernels add float32 partial
    # sums per vector into the float64 accumulators, which keeps them off the vector ALU's limit
    s2 = Sum(node.op.axis, dtype="float64", acc_dtype="float64")(T.sqr(d))
    # sum(d) = sum(x) - N c with sum(x) in float64: the same accumulator serves the mean (its own sum asks for
    # the same values), so the pass keeps two running sums per element instead of three.  With
    # dm = sum(x) / N - c the correction sum(d)^2 / N is N dm^2; the extents enter one by one, as host
    # scalars of the nodes that use them (a product node of their own would be a kernel of its own).
    exts = [T.ShapeFloat(dv.owner.op.i, "float64")(dv.owner.inputs[0]) for dv in divisors]
    dm = Sum(node.op.axis, dtype="float64", acc_dtype="float64")(x)
    for e in exts:
        dm = T.true_div(dm, e)
    dm = T.sub(dm, T.cast(first, "float64"))
    corr = T.mul(dm, dm)
    for e in exts:
        corr = T.mul(corr, e)
    res = T.maximum(T.sub(s2, corr), np.float64(0.0))
    res = T.cast(res, out.type.dtype)
    return [res] if res.type == out.type else False


@local_optimizer([Elemwise])
def local_cancel_common_factors(fgraph, node):
    """``(a / b) * b -> a``: a factor that appears above and below the line of one product -
    written with any nesting of ``mul``, ``true_div``, ``neg`` and ``inv`` of one float dtype -
    is dropped from both (the part of ``local_mul_canonizer``, ``theano/tensor/opt.py:4700-5060``,
    that turns the gradient of ``log(1 - sigmoid(x))``, ``-(g / (1 - s)) * s * (1 - s)``, into
    ``-(g * s)``, finite where ``1 - s`` rounds to zero).  Left alone when nothing cancels or
    when the dropped factor was what gave the result its shape."""
    out = node.outputs[0]
    if not isinstance(node.op.scalar_op, (scal.Mul, scal.TrueDiv)) or out.type.dtype not in scal.float_dtypes:
        return False
    dt = out.type.dtype
    num, den = [], []

    def collect(v, above, depth):
        """Appends the factors of v to num / den; returns whether v is negated."""
        p = v.owner
        if (p is not None and isinstance(p.op, Elemwise) and v.type.dtype == dt and depth < 16 and
                all(i.type.dtype == dt for i in p.inputs)):
            sop = p.op.scalar_op
            if isinstance(sop, scal.Mul):
                sign = False
                for i in p.inputs:
                    sign ^= collect(i, above, depth + 1)
                return sign
            if isinstance(sop, scal.TrueDiv):
                a, b = p.inputs
                return collect(a, above, depth + 1) ^ collect(b, not above, depth + 1)
            if isinstance(sop, scal.Neg):
                return not collect(p.inputs[0], above, depth + 1)
            if isinstance(sop, scal.Inv):
                return collect(p.inputs[0], not above, depth + 1)
        (num if above else den).append(v)
        return False

    sign = collect(out, True, 0)
    dropped = False
    for v in list(num):
        for k, w in enumerate(den):
            if w is v:
                num.remove(v)
                del den[k]
                dropped = True
                break
    if not dropped:
        return False
    new = constant(1.0, dtype=dt) if not num else (num[0] if len(num) == 1 else T.mul(*num))
    if den:
        new = T.true_div(new, den[0] if len(den) == 1 else T.mul(*den))
    if sign:
        new = T.neg(new)
    if new.type.ndim < out.type.ndim:
        new = T.shape_padleft(new, out.type.ndim - new.type.ndim)
    return [new] if new.type == out.type else False


@local_optimizer([Elemwise])
def local_split_huge_add_or_mul(fgraph, node):
    """``add`` / ``mul`` of more operands than one kernel takes becomes a tree of nodes of at most
    ``config.max_fused_inputs`` operands each (``split_inputs``, ``theano/gpuarray/opt.py:800-839``); fusion
    respects the same limit, so no other node can outgrow it."""
    limit = config.max_fused_inputs
    if not isinstance(node.op.scalar_op, (scal.Add, scal.Mul)) or len(node.inputs) <= limit:
        return False
    terms = list(node.inputs)
    while len(terms) > limit:
        terms = [node.op(*terms[k:k + limit]) if len(terms[k:k + limit]) > 1 else terms[k]
                 for k in range(0, len(terms), limit)]
    new = node.op(*terms)
    return [new] if new.type == node.outputs[0].type else False


@local_optimizer([Elemwise])
def local_mul_to_sqr(fgraph, node):
    """``x * x -> sqr(x)`` (``theano/tensor/opt.py:5865-5876``): one operand to fetch instead of two, and the
    form the reductions' prologues and the variance rewrite look for."""
    if not isinstance(node.op.scalar_op, scal.Mul) or len(node.inputs) != 2 or node.inputs[0] is not node.inputs[1]:
        return False
    new = T.sqr(node.inputs[0])
    return [new] if new.type == node.outputs[0].type else False


@local_optimizer(None)
def local_useless_subtensor(fgraph, node):
    """``x[:]``, ``x[:, :]`` ...: an index of full slices only stands for its operand
    (``local_useless_subtensor``, ``theano/tensor/opt.py:2685-2780``, its case of slices that are all None)."""
    from . import views as V
    if type(node.op) is not V.Subtensor or len(node.inputs) != 1:
        return False
    if not all(isinstance(i, slice) and i == slice(None) for i in node.op.idx_list):
        return False
    x = node.inputs[0]
    return [x] if x.type == node.outputs[0].type else False


CANONICALIZE = [local_remove_grad_views, local_useless_subtensor, local_shape_lift, local_dimshuffle_fold, local_useless_composite, local_constant_fold,
                local_useless_elemwise, local_fill_sink,
                local_useless_reduce, local_op_of_op,
                local_dimshuffle_lift, local_sum_invariant_factor, local_max_and_argmax, local_max_to_min,
                local_single_pass_variance,
                local_cancel_common_factors, local_split_huge_add_or_mul, local_mul_to_sqr]


def canonicalize(fgraph):
    """Clean-ups to a fixed point, together with the rewrites that recognise row softmax
    expressions; then the row ops are lowered to Elemwise / CAReduce graphs and those are
    cleaned up in turn."""
    from . import nnet
    gof.merge_identical(fgraph)
    gof.apply_local(fgraph, CANONICALIZE + nnet.RECOGNIZE)
    gof.merge_identical(fgraph)
    if gof.apply_local(fgraph, nnet.LOWER):
        gof.merge_identical(fgraph)
        gof.apply_local(fgraph, CANONICALIZE)
        gof.merge_identical(fgraph)
    return fgraph
