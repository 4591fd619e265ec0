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


def batch_normalization_train(inputs, gamma, beta, axes="per-activation", epsilon=1e-4,
                              running_average_factor=0.1, running_mean=None, running_var=None):
    """Training-mode batch normalization as the graph the reference lowers
    ``AbstractBatchNormTrain`` to (``local_abstract_batch_norm_train``,
    ``theano/tensor/nnet/bn.py:679-726``): ``mean`` and two-pass ``var`` over
    ``axes`` (keepdims), ``invstd = inv(sqrt(var + eps))``,
    ``out = (x - mean) * (gamma * invstd) + beta``.  ``gamma`` / ``beta`` (and
    the running statistics) have the input's rank with extent 1 along ``axes``.
    Returns ``(out, mean, invstd)`` plus the updated running mean and variance
    when those are given."""
    x = as_tensor_variable(inputs)
    gamma, beta = as_tensor_variable(gamma), as_tensor_variable(beta)
    axes = _bn_axes(axes, x.type.ndim)
    mean = T.mean(x, axis=axes, keepdims=True)
    var = T.var(x, axis=axes, keepdims=True)
    eps = T.cast(as_tensor_variable(epsilon), var.type.dtype)
    invstd = T.inv(T.sqrt(var + eps))
    out = (x - mean) * (gamma * invstd) + beta
    results = [out, mean, invstd]
    if running_mean is not None:
        running_mean = as_tensor_variable(running_mean)
        results.append(running_mean * (1.0 - running_average_factor) + mean * running_average_factor)
    if running_var is not None:
        running_var = as_tensor_variable(running_var)
        m = None
        for a in axes:                                   # elements per statistic
            e = T.ShapeFloat(a, var.type.dtype)(x)
            m = e if m is None else m * e
        results.append(running_var * (1.0 - running_average_factor) + (m / (m - 1)) * var * running_average_factor)
    return tuple(results)


def batch_normalization_train_grad(x, dy, scale, x_mean, x_invstd, axes="per-activation"):
    """The graph ``AbstractBatchNormTrainGrad`` lowers to
    (``theano/tensor/nnet/bn.py:730-761``): gradients with respect to the inputs,
    the scale and the bias, given the saved mean and inverse standard deviation."""
    x, dy = as_tensor_variable(x), as_tensor_variable(dy)
    axes = _bn_axes(axes, x.type.ndim)
    x_diff = x - x_mean
    mean_dy_x_diff = T.mean(dy * x_diff, axis=axes, keepdims=True)
    c = (dy * x_invstd) - x_diff * (mean_dy_x_diff * (x_invstd ** 3))
    g_wrt_inputs = scale * (c - T.mean(c, axis=axes, keepdims=True))
    g_wrt_scale = T.sum(dy * x_invstd * x_diff, axis=axes, keepdims=True)
    g_wrt_bias = T.sum(dy, axis=axes, keepdims=True)
    return g_wrt_inputs, g_wrt_scale, g_wrt_bias


def batch_normalization_test(inputs, gamma, beta, mean, var, axes="per-activation", epsilon=1e-4):
    """Inference-mode batch normalization (``local_abstract_batch_norm_inference``,
    ``theano/tensor/nnet/bn.py:765-789``):
    ``(x - mean) * (gamma / sqrt(var + eps)) + beta``, one elementwise kernel."""
    x = as_tensor_variable(inputs)
    var = as_tensor_variable(var)
    _bn_axes(axes, x.type.ndim)
    eps = T.cast(as_tensor_variable(epsilon), var.type.dtype)
    return (x - mean) * (gamma / T.sqrt(var + eps)) + beta
