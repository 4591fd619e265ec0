"""Row-wise activations of ``theano.tensor.nnet`` written as Elemwise / CAReduce
graphs, so that they run as one fused row kernel each (forward and gradient).

The reference implements ``softmax`` / ``logsoftmax`` as hand-written ops
(``theano/tensor/nnet/nnet.py:411-600, 603-700``) and rewrites user-written
``exp(x) / exp(x).sum(-1)`` graphs into them (``softmax_simplifier`` :888-925,
``local_logsoftmax`` :703-722).  Here the direction is the opposite: the op's
``perform`` formula is the graph, gradients come from ``grad`` of that graph
and the row-chain fusion turns either into a single launch.
"""
from . import basic as T
from .type import as_tensor_variable

sigmoid = T.sigmoid
softplus = T.softplus


def softmax(c):
    """``Softmax.perform`` (``theano/tensor/nnet/nnet.py:440-446``):
    ``e = exp(x - max(x, -1)); e / sum(e, -1)``."""
    return T.softmax(c)


def softmax_with_bias(x, b):
    """``SoftmaxWithBias`` (``theano/tensor/nnet/nnet.py:43-90``): softmax of
    ``x + b`` with ``b`` a vector along the last axis."""
    x, b = as_tensor_variable(x), as_tensor_variable(b)
    if b.type.ndim != 1:
        raise ValueError("b must be a 1-d tensor")
    return T.softmax(x + b.dimshuffle(*(["x"] * (x.type.ndim - 1) + [0])))


def logsoftmax(c):
    """``LogSoftmax.perform`` (``theano/tensor/nnet/nnet.py:628-633``):
    ``xdev = x - max(x, -1); xdev - log(sum(exp(xdev), -1))``."""
    x = as_tensor_variable(c)
    xdev = x - T.max(x, axis=-1, keepdims=True)
    return xdev - T.log(T.sum(T.exp(xdev), axis=-1, keepdims=True))


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
