"""Row-wise activations of ``theano.tensor.nnet``.

``Softmax`` / ``SoftmaxWithBias`` / ``SoftmaxGrad`` / ``LogSoftmax`` exist as graph
nodes with the reference's interface (``theano/tensor/nnet/nnet.py:43-120, 292-345,
411-470, 602-650``): same ``make_node`` checks, gradients expressed through each other,
``R_op``, ``infer_shape``.  The rewrites that produce them are kept too
(``softmax_simplifier`` :888-925, ``local_softmax_with_bias`` :822-885,
``local_logsoftmax`` :749-769, ``local_logsoftmax_grad`` :772-804).  Where the
reference then runs hand-written C per op, these nodes are lowered, right before the
graph is lifted, to the Elemwise / CAReduce graph of their ``perform`` formulas, and the
row-chain fusion turns each (forward, gradient, or both at once) into one launch.
"""
import warnings

from .. import scalar as scal
from ..gof import Apply, Op, local_optimizer
from . import basic as T
from .elemwise import DimShuffle, Elemwise, Sum
from .type import as_tensor_variable

sigmoid = T.sigmoid
softplus = T.softplus
# the scalar ops behind them live in this module in the reference (theano/tensor/nnet/sigm.py:29-300)
ScalarSigmoid, ScalarSoftplus, UltraFastScalarSigmoid = scal.ScalarSigmoid, scal.ScalarSoftplus, scal.UltraFastScalarSigmoid
scalar_sigmoid, scalar_softplus, ultra_fast_scalar_sigmoid = (scal.scalar_sigmoid, scal.scalar_softplus,
                                                              scal.ultra_fast_scalar_sigmoid)
sigmoid_inplace = Elemwise(scal.scalar_sigmoid.make_new_inplace(scal.transfer_type(0), name="sigmoid_inplace"), {0: 0},
                           name="sigmoid_inplace")
softplus_inplace = Elemwise(scal.scalar_softplus.make_new_inplace(scal.transfer_type(0), name="softplus_inplace"), {0: 0},
                            name="softplus_inplace")
ultra_fast_sigmoid_inplace = Elemwise(scal.ultra_fast_scalar_sigmoid.make_new_inplace(
    scal.transfer_type(0), name="ultra_fast_sigmoid_inplace"), {0: 0}, name="ultra_fast_sigmoid_inplace")

_FLOATS = ("float16", "float32", "float64")


def _no_host(op):
    raise NotImplementedError("%s has no host implementation: it is lowered to Elemwise / CAReduce nodes before "
                              "the graph runs" % op)


def _row_input(x, who):
    x = as_tensor_variable(x)
    if x.type.ndim not in (1, 2) or x.type.dtype not in _FLOATS:
        raise ValueError("x must be 1-d or 2-d tensor of floats. Got %s" % x.type)
    if x.type.ndim == 1:
        warnings.warn("DEPRECATION: If x is a vector, %s will not automatically pad x anymore in next releases. "
                      "If you need it, please do it manually." % who, stacklevel=4)
        x = x.dimshuffle("x", 0)
    return x


def _rows(v):
    """(n,) per-row values as an (n, 1) column."""
    return v.dimshuffle(0, "x")


def _row_max_already_subtracted(x):
    """``x`` is ``y - max(y, 1, keepdims)``: its row maxima are exactly 0, so subtracting
    them again changes nothing (a user-written stable softmax that the simplifier turned
    into the op)."""
    from .elemwise import CAReduce
    if x.owner is None or not isinstance(x.owner.op, Elemwise) or not isinstance(x.owner.op.scalar_op, scal.Sub):
        return False
    y, m = x.owner.inputs
    if m.owner is None or not isinstance(m.owner.op, DimShuffle) or m.owner.op.new_order != (0, "x"):
        return False
    r = m.owner.inputs[0]
    return (r.owner is not None and isinstance(r.owner.op, CAReduce) and
            isinstance(r.owner.op.scalar_op, scal.Maximum) and not isinstance(r.owner.op.scalar_op, scal.Minimum) and
            r.owner.op.axis == (1,) and r.owner.inputs[0] is y)


class Softmax(Op):
    """``e = exp(x - max(x, 1)); e / sum(e, 1)`` per row
    (``theano/tensor/nnet/nnet.py:411-456``)."""

    __props__ = ()

    def make_node(self, x):
        x = _row_input(x, "Softmax")
        return Apply(self, [x], [x.type()])

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def infer_shape(self, node, shapes):
        return shapes

    def L_op(self, inputs, outputs, grads):
        return [softmax_grad(grads[0], outputs[0])]

    def R_op(self, inputs, eval_points):
        # the Jacobian is symmetric: same expression as the gradient
        if None in eval_points:
            return [None]
        return self.L_op(inputs, [self(*inputs)], eval_points)

    @staticmethod
    def lower(x):
        if not _row_max_already_subtracted(x):
            x = x - T.max(x, axis=1, keepdims=True)
        e = T.exp(x)
        return e / T.sum(e, axis=1, keepdims=True)


class SoftmaxWithBias(Op):
    """Softmax of ``x + b`` with ``b`` a vector along the rows
    (``theano/tensor/nnet/nnet.py:43-115``)."""

    __props__ = ()

    def make_node(self, x, b):
        x, b = as_tensor_variable(x), as_tensor_variable(b)
        if x.type.ndim != 2 or x.type.dtype not in _FLOATS:
            raise ValueError("x must be 2-d tensor of floats")
        if b.type.ndim != 1 or b.type.dtype not in _FLOATS:
            raise ValueError("b must be 1-d tensor of floats")
        return Apply(self, [x, b], [x.type()])

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def infer_shape(self, node, shapes):
        return [shapes[0]]

    def L_op(self, inputs, outputs, grads):
        dx = softmax_grad(grads[0], outputs[0])
        return [dx, T.sum(dx, axis=0)]

    @staticmethod
    def lower(x, b):
        # float16 rows are computed in float32 and cast back (nnet.py:93-104)
        dt = x.type.dtype
        if dt == "float16":
            x = T.cast(x, "float32")
        r = Softmax.lower(x + b.dimshuffle("x", 0))
        return T.cast(r, dt) if r.type.dtype != dt else r


class SoftmaxGrad(Op):
    """``dx = dy * sm - sum(dy * sm, 1) * sm`` per row
    (``theano/tensor/nnet/nnet.py:292-335``)."""

    __props__ = ()

    def make_node(self, dy, sm):
        dy, sm = as_tensor_variable(dy), as_tensor_variable(sm)
        if dy.type.ndim not in (1, 2) or dy.type.dtype not in _FLOATS:
            raise ValueError("dy must be 1-d or 2-d tensor of floats. Got %s" % dy.type)
        if dy.type.ndim == 1:
            dy = dy.dimshuffle("x", 0)
        if sm.type.ndim == 1:
            sm = sm.dimshuffle("x", 0)
        return Apply(self, [dy, sm], [sm.type()])

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def infer_shape(self, node, shapes):
        return [shapes[1]]

    def L_op(self, inputs, outputs, grads):
        dy, sm = inputs
        (g,) = grads
        tmp = g + T.neg(_rows(T.sum(g * sm, axis=1)))
        tmp2 = _rows(T.sum(dy * sm, axis=1))
        return [tmp * sm, tmp * dy - g * tmp2]

    @staticmethod
    def lower(dy, sm):
        t = dy * sm
        r = t - T.sum(t, axis=1, keepdims=True) * sm
        return T.cast(r, sm.type.dtype) if r.type.dtype != sm.type.dtype else r


class LogSoftmax(Op):
    """``xdev = x - max(x, 1); xdev - log(sum(exp(xdev), 1))`` per row
    (``theano/tensor/nnet/nnet.py:602-646``)."""

    __props__ = ()

    def make_node(self, x):
        x = _row_input(x, "LogSoftmax")
        return Apply(self, [x], [x.type()])

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def infer_shape(self, node, shapes):
        return shapes

    def L_op(self, inputs, outputs, grads):
        sm = softmax_op(inputs[0])
        return [grads[0] - T.sum(grads[0], axis=1, keepdims=True) * sm]

    def R_op(self, inputs, eval_points):
        if None in eval_points:
            return [None]
        return self.L_op(inputs, None, eval_points)

    @staticmethod
    def lower(x):
        xdev = x - T.max(x, axis=1, keepdims=True)
        return xdev - T.log(T.sum(T.exp(xdev), axis=1, keepdims=True))


softmax_op, softmax_with_bias = Softmax(), SoftmaxWithBias()
softmax_grad, logsoftmax_op = SoftmaxGrad(), LogSoftmax()


def softmax_graph(c):
    """The unstabilised expression ``softmax_simplifier`` recognises (nnet.py:807-808)."""
    c = as_tensor_variable(c)
    return T.exp(c) / T.sum(T.exp(c), axis=-1, keepdims=True)


def softmax(c):
    """``softmax_op`` for vectors and matrices (``theano/tensor/nnet/nnet.py:811-815``);
    tensors of higher rank, which the reference's op refuses, get the same formula along
    their last axis as a plain graph."""
    c = as_tensor_variable(c)
    if c.type.broadcastable[-1]:
        warnings.warn("The softmax is applied on a dimension of shape 1, which does not have a semantic meaning.")
    if c.type.ndim <= 2:
        return softmax_op(c)
    return T.softmax(c)


def logsoftmax(c):
    c = as_tensor_variable(c)
    if c.type.ndim <= 2:
        return logsoftmax_op(c)
    xdev = c - T.max(c, axis=-1, keepdims=True)
    return xdev - T.log(T.sum(T.exp(xdev), axis=-1, keepdims=True))


# ---- rewrites --------------------------------------------------------------------------------------

def _is_elemwise(var, scalar_cls):
    return (var.owner is not None and isinstance(var.owner.op, Elemwise) and
            isinstance(var.owner.op.scalar_op, scalar_cls))


@local_optimizer([Elemwise])
def local_softmax_simplifier(fgraph, node):
    """``exp(x) / sum(exp(x), 1).dimshuffle(0, 'x')`` on a float matrix -> ``softmax(x)``
    (``softmax_simplifier``, nnet.py:888-925; the reference runs it inside the
    multiplication canonizer over lists of numerators and denominators, here the
    two-operand quotient is matched)."""
    if not isinstance(node.op.scalar_op, scal.TrueDiv) or len(node.inputs) != 2:
        return False
    num, den = node.inputs
    if num.type.ndim != 2 or not num.type.dtype.startswith("float") or not _is_elemwise(num, type(scal.exp)):
        return False
    if den.owner is None or not isinstance(den.owner.op, DimShuffle) or den.owner.op.new_order != (0, "x"):
        return False
    z = den.owner.inputs[0]
    if z.owner is None or not isinstance(z.owner.op, Sum) or z.owner.op.axis != (1,):
        return False
    if z.owner.inputs[0] is not num or z.type.dtype != num.type.dtype:
        return False
    return [softmax_op(num.owner.inputs[0])]


@local_optimizer([Softmax])
def local_softmax_with_bias(fgraph, node):
    """``softmax(matrix + vector.dimshuffle('x', 0))`` -> ``softmax_with_bias(matrix, vector)``
    (nnet.py:822-885)."""
    (x,) = node.inputs
    if not _is_elemwise(x, scal.Add):
        return False
    vectors, others = [], []
    for t in x.owner.inputs:
        if tuple(t.type.broadcastable) == (True, False):
            if (t.owner is not None and isinstance(t.owner.op, DimShuffle) and
                    tuple(t.owner.inputs[0].type.broadcastable) == (False,)):
                vectors.append(t.owner.inputs[0])
            else:
                vectors.append(DimShuffle((True, False), (1,))(t))
        else:
            others.append(t)
    if not others:
        others.append(vectors.pop().dimshuffle("x", 0))
    if not vectors:
        return False
    vsum = T.add(*vectors) if len(vectors) > 1 else vectors[0]
    msum = T.add(*others) if len(others) > 1 else others[0]
    try:
        res = softmax_with_bias(msum, vsum)
    except (ValueError, TypeError):
        return False
    return [res] if res.type == node.outputs[0].type else False


@local_optimizer([Elemwise])
def local_logsoftmax(fgraph, node):
    """``log(softmax(x))`` -> ``logsoftmax(x)`` (nnet.py:749-769)."""
    if not isinstance(node.op.scalar_op, type(scal.log)) or len(node.inputs) != 1:
        return False
    p = node.inputs[0].owner
    if p is None or not isinstance(p.op, Softmax):
        return False
    return [logsoftmax_op(p.inputs[0])]


@local_optimizer([SoftmaxGrad])
def local_logsoftmax_grad(fgraph, node):
    """``softmax_grad(g / sm, sm)`` with ``sm = softmax(x)``: the gradient of
    ``log(softmax(x))``, rewritten to ``g - sum(g, 1, keepdims) * sm`` without the division
    (nnet.py:772-804)."""
    dy, sm = node.inputs
    if not _is_elemwise(dy, scal.TrueDiv) or len(dy.owner.inputs) != 2:
        return False
    g, den = dy.owner.inputs
    if den is not sm or sm.owner is None or not isinstance(sm.owner.op, Softmax):
        return False
    if g.type.broadcastable[1] and not sm.type.broadcastable[1]:
        g = T.second(sm, g)
    res = g - T.sum(g, axis=1, keepdims=True) * sm
    return [res] if res.type == node.outputs[0].type else False


def local_lower_row_ops(fgraph, node):
    if not hasattr(node.op, "lower"):
        return False
    res = node.op.lower(*node.inputs)
    res = list(res) if isinstance(res, (list, tuple)) else [res]
    if len(res) != len(node.outputs) or any(r.type != o.type for r, o in zip(res, node.outputs)):
        return False
    return res


local_lower_row_ops = local_optimizer(None)(local_lower_row_ops)


# ---- sigmoid / softplus stabilisation (theano/tensor/nnet/sigm.py:378-425, 588-640, 845-905) ----
def _const_value(v):
    """Python float of an all-broadcastable constant (also under a DimShuffle), else None."""
    from .type import TensorConstant
    if v.owner is not None and isinstance(v.owner.op, DimShuffle):
        v = v.owner.inputs[0]
    if isinstance(v, TensorConstant) and all(v.type.broadcastable):
        return float(v.data.reshape(()))
    return None


def _is_const(v, value):
    c = _const_value(v)
    return c is not None and abs(c - value) <= 1e-8 + 1e-5 * abs(value)


def _arg_of(var, scalar_cls):
    return var.owner.inputs[0] if _is_elemwise(var, scalar_cls) else None


def _negated(t):
    """-t, without stacking a negation on a negation."""
    inner = _arg_of(t, scal.Neg)
    return inner if inner is not None else T.neg(t)


def _one_plus_exp(v):
    """x if v is ``1 + exp(x)`` (either order), else None (``is_1pexp``, sigm.py:428-462)."""
    if not _is_elemwise(v, scal.Add) or len(v.owner.inputs) != 2:
        return None
    a, b = v.owner.inputs
    for one, e in ((a, b), (b, a)):
        x = _arg_of(e, type(scal.exp))
        if x is not None and _is_const(one, 1.0):
            return x
    return None


def _same_type(new, node):
    return [new] if new.type == node.outputs[0].type else False


@local_optimizer([Elemwise])
def local_log_of_sigmoid(fgraph, node):
    """``log(sigmoid(x)) -> -softplus(-x)``, ``log(1 - sigmoid(x)) -> -softplus(x)``,
    ``log1p(exp(x)) -> softplus(x)``, ``log1p(-sigmoid(x)) -> -softplus(x)``: finite where the
    plain formulas give -inf (``logsigm_to_softplus``, ``log1msigm_to_softplus``,
    ``log1pexp_to_softplus``, ``log1p_neg_sigmoid``, sigm.py:378-425)."""
    sop = node.op.scalar_op
    if len(node.inputs) != 1 or node.outputs[0].type.dtype not in _FLOATS:
        return False
    (v,) = node.inputs
    if isinstance(sop, type(scal.log)):
        x = _arg_of(v, scal.ScalarSigmoid)
        if x is not None:
            return _same_type(T.neg(softplus(_negated(x))), node)
        if _is_elemwise(v, scal.Sub) and _is_const(v.owner.inputs[0], 1.0):
            x = _arg_of(v.owner.inputs[1], scal.ScalarSigmoid)
            if x is not None and x.type.broadcastable == v.type.broadcastable:
                return _same_type(T.neg(softplus(x)), node)
        return False
    if isinstance(sop, type(scal.log1p)):
        x = _arg_of(v, type(scal.exp))
        if x is not None:
            return _same_type(softplus(x), node)
        inner = _arg_of(v, scal.Neg)
        x = _arg_of(inner, scal.ScalarSigmoid) if inner is not None else None
        if x is not None:
            return _same_type(T.neg(softplus(x)), node)
    return False


def _factors(v):
    return list(v.owner.inputs) if _is_elemwise(v, scal.Mul) else [v]


@local_optimizer([Elemwise])
def local_exp_over_1_plus_exp(fgraph, node):
    """``exp(x) / (1 + exp(x)) -> sigmoid(x)`` and ``c / (1 + exp(x)) -> c * sigmoid(-x)``, also with
    further factors on either side of the division (sigm.py:588-640): no overflow of exp."""
    if not isinstance(node.op.scalar_op, scal.TrueDiv) or node.outputs[0].type.dtype not in _FLOATS:
        return False
    num, den = node.inputs
    num_f, den_rest, sigmoids = _factors(num), [], []
    for d in _factors(den):
        x = _one_plus_exp(d)
        if x is None or d.type.dtype != node.outputs[0].type.dtype:
            den_rest.append(d)
            continue
        for k, f in enumerate(num_f):
            if _arg_of(f, type(scal.exp)) is x:
                del num_f[k]
                sigmoids.append(sigmoid(x))
                break
        else:
            sigmoids.append(sigmoid(_negated(x)))
    if not sigmoids:
        return False
    num_f = [f for f in num_f if not _is_const(f, 1.0)] + sigmoids
    new = num_f[0] if len(num_f) == 1 else T.mul(*num_f)
    if den_rest:
        new = new / (den_rest[0] if len(den_rest) == 1 else T.mul(*den_rest))
    return _same_type(new, node)


@local_optimizer([Elemwise])
def local_sigm_times_exp(fgraph, node):
    """``sigmoid(x) * exp(-x) -> sigmoid(-x)`` and ``sigmoid(-x) * exp(x) -> sigmoid(x)`` among the
    factors of one product (the flat case of sigm.py:845-905)."""
    if not isinstance(node.op.scalar_op, scal.Mul):
        return False
    fs = list(node.inputs)
    for i, f in enumerate(fs):
        x = _arg_of(f, scal.ScalarSigmoid)
        if x is None:
            continue
        for j, g in enumerate(fs):
            e = _arg_of(g, type(scal.exp))
            if e is None or j == i:
                continue
            if _arg_of(e, scal.Neg) is x or _arg_of(x, scal.Neg) is e:
                rest = [h for k, h in enumerate(fs) if k not in (i, j)]
                new = sigmoid(_negated(x))
                if rest:
                    new = T.mul(*(rest + [new]))
                if new.type.broadcastable != node.outputs[0].type.broadcastable:
                    return False
                return _same_type(new, node)
    return False


RECOGNIZE = [local_softmax_simplifier, local_softmax_with_bias, local_logsoftmax, local_logsoftmax_grad,
             local_log_of_sigmoid, local_exp_over_1_plus_exp, local_sigm_times_exp]
LOWER = [local_lower_row_ops]


ultra_fast_sigmoid = T._elemwise(scal.ultra_fast_scalar_sigmoid, "ultra_fast_sigmoid")
softsign = T._elemwise(scal.scalar_softsign, "softsign")


def hard_sigmoid(x):
    """``clip(0.2 * x + 0.5, 0, 1)`` in the dtype ``upgrade_to_float`` gives (sigm.py:278-297)."""
    x = as_tensor_variable(x)
    out_dtype = scal.upgrade_to_float(scal.Scalar(x.type.dtype))[0].dtype
    slope = T.constant(0.2, dtype=out_dtype)
    shift = T.constant(0.5, dtype=out_dtype)
    return T.clip(x * slope + shift, 0, 1)


def elu(x, alpha=1):
    """``x if x > 0 else alpha * (exp(x) - 1)`` (nnet.py:2437-2456)."""
    x = as_tensor_variable(x)
    return T.switch(x > 0, x, alpha * T.expm1(x))


def selu(x):
    """``scale * elu(x, alpha)`` with the self-normalising constants (nnet.py:2459-2481)."""
    alpha = 1.6732632423543772848170429916717
    scale = 1.0507009873554804934193349852946
    return scale * elu(x, alpha)


def binary_crossentropy(output, target):
    """``-(target * log(output) + (1 - target) * log(1 - output))``, per component (nnet.py:2008-2025)."""
    output, target = as_tensor_variable(output), as_tensor_variable(target)
    return -(target * T.log(output) + (1.0 - target) * T.log(1.0 - output))


_sigmoid_binary_crossentropy = T._elemwise(scal.sigmoid_binary_crossentropy, "sigmoid_binary_crossentropy")


def sigmoid_binary_crossentropy(output, target):
    """Cross-entropy of ``sigmoid(output)`` against ``target`` in its stable form
    ``softplus(-|output|) + output * ((output > 0) - target)``, with the gradients
    ``sigmoid(output) - target`` and ``-output`` (nnet.py:2028-2050).  Where the reference wraps the
    formula in an inlined sub-graph with overridden gradients, this is one scalar op of the same
    formula and gradients: it fuses like any other."""
    return _sigmoid_binary_crossentropy(as_tensor_variable(output), as_tensor_variable(target))


def categorical_crossentropy(coding_dist, true_dist):
    """``-sum(true_dist * log(coding_dist), axis=-1)`` for a distribution per row
    (nnet.py:2053-2102).  The form that takes one class index per row goes through advanced
    indexing, which this package does not have."""
    coding_dist, true_dist = as_tensor_variable(coding_dist), as_tensor_variable(true_dist)
    if true_dist.type.ndim == coding_dist.type.ndim:
        return -T.sum(true_dist * T.log(coding_dist), axis=coding_dist.type.ndim - 1)
    if true_dist.type.ndim == coding_dist.type.ndim - 1:
        raise NotImplementedError("categorical_crossentropy with class indices needs advanced indexing")
    raise TypeError("rank mismatch between coding and true distributions")


def relu(x, alpha=0):
    """``theano/tensor/nnet/nnet.py:2209-2252``: ``0.5 * (x + |x|)`` for
    ``alpha == 0``, else ``f1 * x + f2 * |x|`` with ``f1 = (1 + alpha) / 2``,
    ``f2 = (1 - alpha) / 2``."""
    x = as_tensor_variable(x)
    if isinstance(alpha, (int, float)) and alpha == 0:
        return 0.5 * (x + abs(x))
    alpha = as_tensor_variable(alpha)
    f1 = 0.5 * (1 + alpha)
    f2 = 0.5 * (1 - alpha)
    return f1 * x + f2 * abs(x)


def _bn_axes(axes, ndim):
    # theano/tensor/nnet/bn.py:88-95
    if axes == "per-activation":
        return (0,)
    if axes == "spatial":
        return (0,) + tuple(range(2, ndim))
    axes = tuple(int(a) for a in axes)
    if not axes or min(axes) < 0 or max(axes) >= ndim:
        raise ValueError("invalid axes for batch normalization: %s" % (axes,))
    return axes


def _as_common_dtype(*vs):
    dt = scal.upcast(*[v.type.dtype for v in vs])
    return [v if v.type.dtype == dt else T.cast(v, dt) for v in vs]


def _check_axes(axes, ndim):
    if min(axes) < 0 or max(axes) >= ndim:
        raise ValueError("axes should be less than ndim (<%d), but %s given" % (ndim, str(axes)))


class AbstractBatchNormTrain(Op):
    """Training-mode batch normalization over ``axes``
    (``theano/tensor/nnet/bn.py:364-499``): inputs ``x, scale, bias, epsilon,
    running_average_factor[, running_mean, running_var]``, outputs ``out, mean, invstd[,
    new_running_mean, new_running_var]``.  The gradient through ``out`` is
    ``AbstractBatchNormTrainGrad`` of the saved mean and inverse standard deviation."""

    __props__ = ("axes",)

    def __init__(self, axes=(0,)):
        assert isinstance(axes, (tuple, list)) and len(axes) > 0
        self.axes = tuple(int(a) for a in axes)

    def _props(self):
        return (self.axes,)

    def make_node(self, x, scale, bias, epsilon=1e-4, running_average_factor=0.1, running_mean=None, running_var=None):
        x, scale, bias = as_tensor_variable(x), as_tensor_variable(scale), as_tensor_variable(bias)
        epsilon, raf = as_tensor_variable(epsilon), as_tensor_variable(running_average_factor)
        assert x.type.ndim == scale.type.ndim == bias.type.ndim
        assert (running_mean is None) == (running_var is None)
        if running_mean is not None:
            running_mean, running_var = as_tensor_variable(running_mean), as_tensor_variable(running_var)
            assert running_mean.type.ndim == x.type.ndim and running_var.type.ndim == x.type.ndim
            x, scale, bias, running_mean, running_var = _as_common_dtype(x, scale, bias, running_mean, running_var)
        else:
            x, scale, bias = _as_common_dtype(x, scale, bias)
        inputs = [x, scale, bias, epsilon, raf]
        outs = [x.type(), scale.type(), scale.type()]
        if running_mean is not None:
            inputs += [running_mean, running_var]
            outs += [scale.type(), scale.type()]
        return Apply(self, inputs, outs)

    def infer_shape(self, node, shapes):
        return [shapes[0]] + [shapes[1]] * (len(node.outputs) - 1)

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def L_op(self, inputs, outputs, grads):
        x, scale, bias, epsilon = inputs[:4]
        dy = grads[0]
        if isinstance(dy.type, scal.DisconnectedType):
            dy = T.zeros_like(outputs[0])
        _, x_mean, x_invstd = outputs[:3]
        res = AbstractBatchNormTrainGrad(self.axes)(x, dy, scale, x_mean, x_invstd, epsilon, return_list=True)
        # The reference stops here (bn.py:447-459): gradients that arrive through the saved mean
        # and inverse standard deviation are dropped, which loses terms of second derivatives.
        # They are added when present: d mean / dx = 1 / m, d invstd / dx = -invstd^3 (x - mean) / m.
        extra = None
        m = None
        for a in self.axes:
            e = T.ShapeFloat(a, x.type.dtype)(x)
            m = e if m is None else m * e
        if len(grads) > 1 and not isinstance(grads[1].type, scal.DisconnectedType):
            extra = T.second(x, grads[1]) / m
        if len(grads) > 2 and not isinstance(grads[2].type, scal.DisconnectedType):
            term = grads[2] * (-(x_invstd ** 3)) * (x - x_mean) / m
            extra = term if extra is None else extra + term
        if extra is not None:
            res[0] = res[0] + extra
        return res + [scal.DisconnectedType()() for _ in inputs[3:]]

    def connection_pattern(self, node):
        n_out = len(node.outputs)
        pat = [[True, True, True] + [True] * (n_out - 3)]                   # x
        pat += [[True, True, True] + [False] * (n_out - 3) for _ in range(2)]  # scale, bias
        pat += [[False] * n_out for _ in range(2)]                          # epsilon, running_average_factor
        for k in range(5, len(node.inputs)):                                # running statistics: their new value only
            pat.append([j == 3 + (k - 5) for j in range(n_out)])
        return pat

    def lower(self, x, scale, bias, epsilon, raf, running_mean=None, running_var=None):
        # local_abstract_batch_norm_train, bn.py:679-726
        axes = self.axes
        _check_axes(axes, x.type.ndim)
        mean = T.mean(x, axis=axes, keepdims=True)
        var = T.var(x, axis=axes, keepdims=True)
        if epsilon.type.dtype != var.type.dtype:
            epsilon = T.cast(epsilon, var.type.dtype)      # the epsilon should not upcast the dtype
        invstd = T.inv(T.sqrt(var + epsilon))
        results = [(x - mean) * (scale * invstd) + bias, mean, invstd]
        if running_mean is not None:
            if raf.type.dtype != var.type.dtype:
                raf = T.cast(raf, var.type.dtype)
            results.append(running_mean * (1.0 - raf) + mean * raf)
            m = None
            for a in axes:                                 # elements per statistic
                e = T.ShapeFloat(a, var.type.dtype)(x)
                m = e if m is None else m * e
            results.append(running_var * (1.0 - raf) + (m / (m - 1)) * var * raf)
        return results


class AbstractBatchNormInference(Op):
    """``(x - mean) * (scale / sqrt(var + eps)) + bias`` with given statistics
    (``theano/tensor/nnet/bn.py:502-572``)."""

    __props__ = ("axes",)

    def __init__(self, axes=(0,)):
        assert isinstance(axes, (tuple, list)) and len(axes) > 0
        self.axes = tuple(int(a) for a in axes)

    def _props(self):
        return (self.axes,)

    def make_node(self, x, scale, bias, estimated_mean, estimated_variance, epsilon=1e-4):
        vs = [as_tensor_variable(v) for v in (x, scale, bias, estimated_mean, estimated_variance)]
        epsilon = as_tensor_variable(epsilon)
        vs = _as_common_dtype(*vs)
        assert len(set(v.type.ndim for v in vs)) == 1
        return Apply(self, vs + [epsilon], [vs[0].type()])

    def infer_shape(self, node, shapes):
        return [shapes[0]]

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def connection_pattern(self, node):
        return [[True], [True], [True], [True], [True], [False]]

    def L_op(self, inputs, outputs, grads):
        x, scale, bias, est_mean, est_var, epsilon = inputs
        dy = grads[0]
        axes = self.axes
        _check_axes(axes, x.type.ndim)
        if epsilon.type.dtype != est_var.type.dtype:
            epsilon = T.cast(epsilon, est_var.type.dtype)
        est_var_eps = est_var + epsilon
        est_std = T.sqrt(est_var_eps)
        dx = dy * (scale / est_std)
        dscale = T.sum(dy * (x - est_mean), axis=axes, keepdims=True) / est_std
        dbias = T.sum(dy, axis=axes, keepdims=True)
        dmean = -T.sum(dy, axis=axes, keepdims=True) * (scale / est_std)
        dvar = -T.sum(dy * (x - est_mean), axis=axes, keepdims=True) * (scale / (2.0 * est_var_eps * est_std))
        return [dx, dscale, dbias, dmean, dvar, scal.DisconnectedType()()]

    def lower(self, x, scale, bias, estimated_mean, estimated_variance, epsilon):
        # local_abstract_batch_norm_inference, bn.py:765-789
        if epsilon.type.dtype != estimated_variance.type.dtype:
            epsilon = T.cast(epsilon, estimated_variance.type.dtype)
        return [(x - estimated_mean) * (scale / T.sqrt(estimated_variance + epsilon)) + bias]


class AbstractBatchNormTrainGrad(Op):
    """Gradients of training-mode batch normalization with respect to the inputs, the
    scale and the bias, from the saved mean and inverse standard deviation
    (``theano/tensor/nnet/bn.py:575-676``)."""

    __props__ = ("axes",)

    def __init__(self, axes=(0,)):
        assert isinstance(axes, (tuple, list)) and len(axes) > 0
        self.axes = tuple(int(a) for a in axes)

    def _props(self):
        return (self.axes,)

    def make_node(self, x, dy, scale, x_mean, x_invstd, epsilon=1e-4):
        vs = [as_tensor_variable(v) for v in (x, dy, scale, x_mean, x_invstd)]
        epsilon = as_tensor_variable(epsilon)
        vs = _as_common_dtype(*vs)
        assert len(set(v.type.ndim for v in vs)) == 1
        return Apply(self, vs + [epsilon], [vs[0].type(), vs[2].type(), vs[2].type()])

    def infer_shape(self, node, shapes):
        return [shapes[0], shapes[2], shapes[2]]

    def perform(self, node, inputs, output_storage):
        _no_host(self)

    def connection_pattern(self, node):
        return [[True, True, False], [True, True, True], [True, False, False], [True, True, False],
                [True, True, False], [False, False, False]]

    def L_op(self, inputs, outputs, grads):
        # second derivatives, bn.py:601-650
        x, dy, scale, x_mean, x_invstd, epsilon = inputs
        ddinputs, ddscale, ddbias = grads
        axes = self.axes
        disc = lambda g: isinstance(g.type, scal.DisconnectedType)   # noqa: E731
        mean = lambda v: T.mean(v, axis=axes, keepdims=True)         # noqa: E731
        total = lambda v: T.sum(v, axis=axes, keepdims=True)         # noqa: E731
        x_diff = x - x_mean
        mean_dy_x_diff = mean(dy * x_diff)
        acc = {"x": None, "dy": None, "scale": None, "mean": None, "invstd": None}

        def add(key, term, sign=1):
            term = term if sign > 0 else -term
            acc[key] = term if acc[key] is None else acc[key] + term

        if not disc(ddinputs):
            ccc = scale * (ddinputs - mean(ddinputs))
            ddd = (x_invstd ** 3) * (ccc * mean(dy * x_diff) + dy * mean(ccc * x_diff))
            add("x", ddd, -1)
            add("dy", (ccc * x_invstd) - ((x_invstd ** 3) * x_diff * mean(ccc * x_diff)))
            eee = (dy * x_invstd) - ((x_invstd ** 3) * x_diff * mean_dy_x_diff)
            add("scale", total(ddinputs * (eee - mean(eee))))
            add("mean", total(ddd))
            add("invstd", total(ccc * (dy - 3 * (x_invstd ** 2) * x_diff * mean_dy_x_diff)))
        if not disc(ddscale):
            add("x", x_invstd * ddscale * dy)
            add("dy", x_invstd * ddscale * x_diff)
            add("mean", x_invstd * ddscale * total(dy), -1)
            add("invstd", ddscale * total(dy * x_diff))
        if not disc(ddbias):
            add("dy", T.second(dy, ddbias))
        res = [acc[k] for k in ("x", "dy", "scale", "mean", "invstd")]
        return [scal.DisconnectedType()() if r is None else r for r in res] + [scal.DisconnectedType()()]

    def lower(self, x, dy, scale, x_mean, x_invstd, epsilon):
        # local_abstract_batch_norm_train_grad, bn.py:730-761
        axes = self.axes
        _check_axes(axes, x.type.ndim)
        x_diff = x - x_mean
        mean_dy_x_diff = T.mean(dy * x_diff, axis=axes, keepdims=True)
        c = (dy * x_invstd) - x_diff * (mean_dy_x_diff * (x_invstd ** 3))
        return [scale * (c - T.mean(c, axis=axes, keepdims=True)),
                T.sum(dy * x_invstd * x_diff, axis=axes, keepdims=True), T.sum(dy, axis=axes, keepdims=True)]


def _bn_params(ndim, axes, params, names):
    """Parameters given with the input's rank must be broadcastable along ``axes``; given
    with one dimension per non-normalized axis they are padded (bn.py:186-232)."""
    non_bc = tuple(d for d in range(ndim) if d not in axes)
    params = [as_tensor_variable(p) for p in params]
    nd0 = params[0].type.ndim
    if nd0 not in (ndim, len(non_bc)) or any(p.type.ndim != nd0 for p in params):
        raise ValueError("%s dimensionality must match the number of non-normalized axes, or have the same "
                         "number of dimensions as the inputs; got %s instead of %d"
                         % (" and ".join(names), [p.type.ndim for p in params], len(non_bc)))
    if nd0 == ndim:
        for p, n in zip(params, names):
            if not all(p.type.broadcastable[a] for a in axes):
                raise TypeError("%s must be broadcastable along the normalized axes %s" % (n, axes))
        return params, None
    pattern = ["x"] * ndim
    for i, a in enumerate(non_bc):
        pattern[a] = i
    return [p.dimshuffle(*pattern) for p in params], non_bc


def batch_normalization_train(inputs, gamma, beta, axes="per-activation", epsilon=1e-4,
                              running_average_factor=0.1, running_mean=None, running_var=None):
    """Training-mode batch normalization (``theano/tensor/nnet/bn.py:79-263``): an
    ``AbstractBatchNormTrain`` node.  Returns ``(out, mean, invstd)`` plus the updated
    running mean and variance when those are given.  ``gamma`` / ``beta`` (and the running
    statistics) have the input's rank with broadcastable extent 1 along ``axes``, or one
    dimension per remaining axis."""
    x = as_tensor_variable(inputs)
    axes = _bn_axes(axes, x.type.ndim)
    if (running_mean is None) != (running_var is None):
        raise ValueError("running_mean and running_var must either both be given or both be None")
    import numpy as np
    if np.asarray(epsilon, dtype=T.config.floatX) < 1e-5:
        raise ValueError("epsilon must be at least 1e-5, got %s" % str(epsilon))
    names = ["gamma", "beta"] + (["running_mean", "running_var"] if running_mean is not None else [])
    given = [gamma, beta] + ([running_mean, running_var] if running_mean is not None else [])
    params, non_bc = _bn_params(x.type.ndim, axes, given, names)
    op = AbstractBatchNormTrain(axes)
    eps = np.asarray(epsilon, dtype=T.config.floatX)
    results = op(x, params[0], params[1], eps, running_average_factor, *params[2:], return_list=True)
    if non_bc is not None:
        results = [results[0]] + [r.dimshuffle(*non_bc) for r in results[1:]]
    return tuple(results)


def batch_normalization_train_grad(x, dy, scale, x_mean, x_invstd, axes="per-activation", epsilon=1e-4):
    """An ``AbstractBatchNormTrainGrad`` node: gradients with respect to the inputs, the
    scale and the bias, given the saved mean and inverse standard deviation."""
    x = as_tensor_variable(x)
    axes = _bn_axes(axes, x.type.ndim)
    return tuple(AbstractBatchNormTrainGrad(axes)(x, dy, scale, x_mean, x_invstd, epsilon, return_list=True))


class BNComposite(scal.Composite):
    """``(x - mean) / std * gamma + beta`` as one scalar operation with the gradients written out
    (``theano/tensor/nnet/bn.py:14-39``): nothing is kept for the backward pass."""

    def __init__(self, dtype):
        self.dtype = dtype
        x, mean, std, gamma, beta = [scal.Scalar(dtype)() for _ in range(5)]
        out = scal.add(scal.mul(scal.true_div(scal.sub(x, mean), std), gamma), beta)
        scal.Composite.__init__(self, [x, mean, std, gamma, beta], [out])

    def make_new_inplace(self, output_types_preference=None, name=None):
        return self

    def __reduce__(self):
        return (BNComposite, (self.dtype,))

    def L_op(self, inputs, outputs, gout):
        x, mean, std, gamma, beta = inputs
        (top,) = gout
        top_gamma = top * gamma
        x_mean = x - mean
        dx = top_gamma / std
        return [dx, -dx, -(top_gamma * x_mean) / (std * std), top * x_mean / std, top]


def batch_normalization(inputs, gamma, beta, mean, std, mode="low_mem"):
    """``(inputs - mean) * (gamma / std) + beta`` with statistics the caller supplies
    (``theano/tensor/nnet/bn.py:42-97``).  'low_mem': one elementwise node over ``BNComposite``, whose gradient
    recomputes what it needs; 'high_mem': the expression written with separate nodes."""
    if mode == "low_mem":
        inputs = as_tensor_variable(inputs)
        return Elemwise(BNComposite(inputs.type.dtype))(inputs, mean, std, gamma, beta)
    if mode == "high_mem":
        return (inputs - mean) * (gamma / std) + beta
    raise ValueError('mode must be either "low_mem", "high_mem"')


def batch_normalization_test(inputs, gamma, beta, mean, var, axes="per-activation", epsilon=1e-4):
    """Inference-mode batch normalization (``theano/tensor/nnet/bn.py:266-361``): an
    ``AbstractBatchNormInference`` node, one elementwise kernel once lowered."""
    x = as_tensor_variable(inputs)
    axes = _bn_axes(axes, x.type.ndim)
    import numpy as np
    if np.asarray(epsilon, dtype=T.config.floatX) < 1e-5:
        raise ValueError("epsilon must be at least 1e-5, got %s" % str(epsilon))
    params, _ = _bn_params(x.type.ndim, axes, [gamma, beta, mean, var], ["gamma", "beta", "mean", "var"])
    return AbstractBatchNormInference(axes)(x, *params, np.asarray(epsilon, dtype=T.config.floatX))
