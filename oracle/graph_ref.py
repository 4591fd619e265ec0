"""TEST INFRASTRUCTURE - not part of the product.  Only ``tests/``, the
``cpu_baseline`` leg of ``bench.py`` and ``__graft_entry__.smoke()`` may import
anything under ``oracle/``.

Evaluates an *unlifted, unfused* theano_amd graph on the CPU the way Theano's
own backend would node by node:

* ``Elemwise``: broadcast check of ``Elemwise.perform``
  (``theano/tensor/elemwise.py:720-740``), the node's output dtype checked against the oracle's own
  table (``oracle/dtype_rules.py``), then the scalar op's C semantics
  from ``oracle.scalar_ref`` applied to whole arrays; Composite nodes are
  evaluated op by op.
* ``CAReduce`` family: dtype tables re-stated here from
  ``theano/tensor/elemwise.py:1721-1759``, sequential accumulation in the
  accumulator dtype by ``oracle/careduce.c`` (the loop nest of
  ``theano/tensor/elemwise_cgen.py:465-527``), then the cast to the output
  dtype (``elemwise.py:1549-1554``).  Zero-length max / min raise ValueError
  (``elemwise.py:1489-1506``).
* ``DimShuffle``: the strided view of ``theano/tensor/c_code/dimshuffle.c:55-98``.
* ``MaxAndArgmax``, the view ops (NumPy basic indexing, reshape, broadcast_to, concatenate),
  the row-softmax ops and the batch-normalization ops: the reference's ``perform`` formulas
  (``theano/tensor/basic.py:1311-1330``, ``theano/tensor/nnet/nnet.py:73-104, 316-323,
  440-444, 628-633``, ``theano/tensor/nnet/bn.py:475-499, 568-571, 659-676``).

Pinned by tests/test_oracle_graph.py and tests/test_golden.py against the reference's
literal test answers (``theano/tensor/tests/test_elemwise.py:654-748, 953-966``; fusion
table ``theano/tensor/tests/test_opt.py:964-1112``; ``test_basic.py:3114-3119, 3304-3309``)
and NumPy closed forms; the softmax and batch-normalization formulas by
tests/test_graph_api.py against ``scipy.special.log_softmax``, closed-form gradients,
NumPy's mean / var and reverse mode through plain graphs.  No function here is unpinned.
"""
import ctypes
import os

import numpy as np

from . import dtype_rules, scalar_ref

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "_build", "liboracle.so")
_lib = None

_DT_CODE = {"bool": 0, "int8": 1, "uint8": 2, "int16": 3, "uint16": 4, "int32": 5, "uint32": 6, "int64": 7,
            "uint64": 8, "float16": 9, "float32": 10, "float64": 11}
_OP_CODE = {"Add": 0, "Mul": 1, "Maximum": 2, "Minimum": 3, "AND": 4, "OR": 5, "XOR": 6, "MulWithoutZeros": 7}

# theano/tensor/elemwise.py:1733-1741 and :1748-1759
SUM_OUT_DTYPE = dict(bool="int64", int8="int64", int16="int64", int32="int64", uint8="uint64", uint16="uint64",
                     uint32="uint64")
SUM_ACC_DTYPE = dict(bool="int64", int8="int64", int16="int64", int32="int64", uint8="uint64", uint16="uint64",
                     uint32="uint64", float16="float32", float32="float64", complex64="complex128")


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            from . import build
            build.build()
        _lib = ctypes.CDLL(_LIB)
        _lib.oracle_careduce.restype = ctypes.c_int
    return _lib


def reduce_identity(op_name, dtype):
    """theano/tensor/elemwise.py:1470-1488 and the ops' own identities
    (theano/scalar/basic.py:1554, 1570, 1586, 1700, 1742)."""
    dt = np.dtype(dtype)
    if op_name == "Add" or op_name in ("OR", "XOR", "MulWithoutZeros"):   # elemwise.py:2061
        return np.zeros((), dt)
    if op_name == "Mul":
        return np.ones((), dt)
    if op_name == "AND":
        return np.asarray(True) if dt == np.bool_ else np.asarray(-1).astype(dt)
    if op_name in ("Maximum", "Minimum"):
        big = op_name == "Minimum"
        if dt.kind == "f":
            return np.asarray(np.inf if big else -np.inf, dt)
        if dt == np.bool_:
            return np.asarray(big)
        info = np.iinfo(dt)
        return np.asarray(info.max if big else info.min, dt)
    raise NotImplementedError(op_name)


def careduce(x, op_name, axis, acc_dtype, out_dtype):
    """Sequential CAReduce of a (possibly strided) host array."""
    x = np.asarray(x)
    nd = x.ndim
    axis = tuple(range(nd)) if axis is None else tuple(a + nd if a < 0 else a for a in axis)
    if op_name in ("Maximum", "Minimum") and any(x.shape[a] == 0 for a in axis):
        raise ValueError("Input of CAReduce{%s} has zero-size on axis %s" % (op_name.lower(), axis))
    acc_dtype, out_dtype = str(acc_dtype), str(out_dtype)
    if not axis:        # no axis: the reference emits an identity Elemwise, no accumulator (elemwise.py:1410-1417)
        return np.array(x).astype(out_dtype) if out_dtype != "bool" else np.array(x) != 0
    if x.dtype.kind == "c":
        # complex sums and products: the accumulator type's own + and * over the reduced elements (the reference's
        # struct operators, theano/scalar/basic.py:518-548, which are NumPy's up to the last place); NumPy adds
        # pairwise, which in a complex128 accumulator is far inside any tolerance a complex64 result is held to
        if op_name not in ("Add", "Mul"):
            raise NotImplementedError("no restatement for %s over complex numbers" % op_name)
        ufunc = np.add if op_name == "Add" else np.multiply
        with np.errstate(all="ignore"):
            return np.asarray(ufunc.reduce(x.astype(acc_dtype), axis=axis)).astype(out_dtype)
    if x.dtype == np.float16:
        x = x.astype("float32")  # no float16 C code exists in the reference (elemwise.py:1395-1398)
        if acc_dtype == "float16":  # max / min: exact in any precision
            acc_dtype = "float32"
    kept = tuple(s for d, s in enumerate(x.shape) if d not in axis)
    acc = np.empty(kept, dtype=acc_dtype)
    ident = reduce_identity(op_name, acc_dtype)
    shape = (ctypes.c_int64 * max(nd, 1))(*x.shape)
    strides = (ctypes.c_int64 * max(nd, 1))(*x.strides)
    mask = (ctypes.c_uint8 * max(nd, 1))(*[1 if d in axis else 0 for d in range(nd)])
    rc = lib().oracle_careduce(_OP_CODE[op_name], _DT_CODE[str(x.dtype)], _DT_CODE[acc_dtype], nd, shape, strides, mask,
                               ctypes.c_void_p(x.ctypes.data), ctypes.c_void_p(ident.ctypes.data),
                               ctypes.c_void_p(acc.ctypes.data))
    if rc != 0:
        raise NotImplementedError("no C restatement for %s over %s accumulated in %s" % (op_name, x.dtype, acc_dtype))
    if out_dtype == "bool":
        return acc != 0
    return acc.astype(out_dtype)


def dimshuffle(x, new_order, drop_check=True):
    x = np.asarray(x)
    shuffle = [o for o in new_order if o != "x"]
    drop = [d for d in range(x.ndim) if d not in shuffle]
    for d in drop:
        if x.shape[d] != 1:
            raise ValueError("cannot drop a dimension of extent %d" % x.shape[d])
    res = x.transpose(shuffle + drop) if x.ndim else x
    shape = list(res.shape[:len(shuffle)])
    for i, o in enumerate(new_order):
        if o == "x":
            shape.insert(i, 1)
    return res.reshape(shape)


def _check_broadcast(node, values):
    nd = node.outputs[0].type.ndim
    shape, owner = [1] * nd, [None] * nd
    for k, (var, val) in enumerate(zip(node.inputs, values)):
        for d in range(nd):
            if var.type.broadcastable[d]:
                if val.shape[d] != 1:
                    raise ValueError("input %d has extent %d on broadcastable dimension %d" % (k, val.shape[d], d))
                continue
            if owner[d] is None:
                owner[d], shape[d] = k, val.shape[d]
            elif val.shape[d] != shape[d]:
                # Elemwise.perform (theano/tensor/elemwise.py:720-751) objects only when the largest extent of
                # the dimension is not 1: an extent of 1 beside an empty operand passes and the result is empty
                # (out_shape 0 when any extent is 0) - the `empty` case of theano/tensor/tests/test_basic.py:680
                if (val.shape[d], shape[d]) == (0, 1):
                    owner[d], shape[d] = k, 0
                elif (val.shape[d], shape[d]) != (1, 0):
                    raise ValueError("Input dimension mis-match. (input[%d].shape[%d] = %d, input[%d].shape[%d] = %d)"
                                     % (owner[d], d, shape[d], k, d, val.shape[d]))


def _wide(dtype):
    """float16 / float32 -> float64, complex64 -> complex128; every other dtype stays."""
    if str(dtype) == "complex64":
        return "complex128"
    return "float64" if str(dtype) in ("float16", "float32") else str(dtype)


def _check_dtypes(scalar_op, node):
    """The node's output dtype against the oracle's own table: the dtype the product's make_node
    inferred is not taken on trust."""
    from theano_amd import config
    dtype_rules.check_node(scalar_op, [i.type.dtype for i in node.inputs], [o.type.dtype for o in node.outputs],
                           floatX=config.floatX, cast_policy=config.cast_policy)


def eval_scalar_op(op, in_values, out_dtypes, wide=False):
    """Evaluate a theano_amd ScalarOp (or Composite) over whole arrays."""
    name = type(op).__name__
    if wide:
        out_dtypes = [_wide(d) for d in out_dtypes]
        in_values = [np.asarray(v).astype(_wide(np.asarray(v).dtype), copy=False) for v in in_values]
    if any(c.__name__ == "Composite" for c in type(op).__mro__):      # Composite and its subclasses: node by node
        from theano_amd import gof
        env = dict(zip(op.inputs, in_values))
        for node in gof.io_toposort(op.inputs, op.outputs):
            _check_dtypes(node.op, node)
            args = [env[i] if i in env else np.asarray(i.data) for i in node.inputs]
            outs = eval_scalar_op(node.op, args, [o.type.dtype for o in node.outputs], wide)
            for o, v in zip(node.outputs, outs):
                env[o] = v
        return [env[o] if o in env else np.asarray(o.data) for o in op.outputs]
    if name == "InRange":
        fn = scalar_ref.in_range(op.openlow, op.openhi)
    else:
        fn = scalar_ref.restatement(name, out_dtypes[0], [np.asarray(v).dtype for v in in_values])
    if fn is None:
        raise NotImplementedError("no restatement of scalar op %s" % name)
    return [np.asarray(fn(out_dtypes[0], *[np.asarray(v) for v in in_values]))]


def max_and_argmax(x, axes):
    """``MaxAndArgmax.perform`` (``theano/tensor/basic.py:1311-1330``): ``np.max``
    over the axes; for the argmax the kept axes go in front, the reduced ones
    (original order) are flattened and ``np.argmax`` runs over that last axis,
    result as int64.  An empty reduced extent raises, as NumPy does."""
    x = np.asarray(x)
    axes = tuple(int(a) for a in axes)
    keep = [i for i in range(x.ndim) if i not in axes]
    t = np.transpose(x, keep + list(axes))
    kept_shape = t.shape[:len(keep)]
    r = t.reshape(kept_shape + (int(np.prod(t.shape[len(keep):], dtype="int64")),))
    return np.asarray(np.max(x, axes), dtype=x.dtype), np.asarray(np.argmax(r, axis=-1), dtype="int64")


def _softmax(x):
    """Softmax.perform, theano/tensor/nnet/nnet.py:440-444"""
    e_x = np.exp(x - x.max(axis=1)[:, None])
    return e_x / e_x.sum(axis=1)[:, None]


def _softmax_with_bias(x, b):
    """SoftmaxWithBias.perform, theano/tensor/nnet/nnet.py:73-104"""
    if b.shape[0] != x.shape[1]:
        raise ValueError("b must have same number of columns as x")
    if x.size == 0:
        return np.zeros(x.shape, dtype=x.dtype)
    x_dtype = x.dtype
    if x.dtype == "float16":
        x = x.astype("float32")
    x_plus_b = x + b[None, :]
    e_x = np.exp(x_plus_b - x_plus_b.max(axis=1)[:, None])
    e_x *= 1.0 / e_x.sum(axis=1)[:, None]
    return e_x.astype(x_dtype, copy=False)


def _softmax_grad(dy, sm):
    """SoftmaxGrad.perform, theano/tensor/nnet/nnet.py:316-323"""
    dx = np.zeros_like(sm)
    for i in range(sm.shape[0]):
        dy_times_sm_i = dy[i] * sm[i]
        dx[i] = dy_times_sm_i - sum(dy_times_sm_i) * sm[i]
    return dx


def _logsoftmax(x):
    """LogSoftmax.perform, theano/tensor/nnet/nnet.py:628-633"""
    xdev = x - x.max(axis=1)[:, None]
    return xdev - np.log(np.sum(np.exp(xdev), axis=1, keepdims=True))


def _bn_train(op, x, scale, bias, epsilon, running_average_factor, running_mean=None, running_var=None):
    """AbstractBatchNormTrain.perform, theano/tensor/nnet/bn.py:475-499"""
    axes = op.axes
    mean = x.mean(axes, keepdims=True)
    var = x.var(axes, keepdims=True)
    invstd = 1.0 / np.sqrt(var + epsilon)
    res = [(x - mean) * (scale * invstd) + bias, mean, invstd]
    if running_mean is not None:
        res.append(running_mean * (1.0 - running_average_factor) + mean * running_average_factor)
        m = float(np.prod(x.shape) / np.prod(scale.shape))
        res.append(running_var * (1.0 - running_average_factor) + (m / (m - 1)) * var * running_average_factor)
    return res


def _bn_inference(op, x, scale, bias, estimated_mean, estimated_variance, epsilon):
    """AbstractBatchNormInference.perform, theano/tensor/nnet/bn.py:568-571"""
    return [(x - estimated_mean) * (scale / np.sqrt(estimated_variance + epsilon)) + bias]


def _bn_train_grad(op, x, dy, scale, x_mean, x_invstd, epsilon):
    """AbstractBatchNormTrainGrad.perform, theano/tensor/nnet/bn.py:659-676"""
    axes = op.axes
    x_diff = x - x_mean
    mean_dy_x_diff = np.mean(dy * x_diff, axis=axes, keepdims=True)
    c = (dy * x_invstd) - (x_diff * mean_dy_x_diff * (x_invstd ** 3))
    return [scale * (c - np.mean(c, axis=axes, keepdims=True)), np.sum(dy * x_invstd * x_diff, axis=axes, keepdims=True),
            np.sum(dy, axis=axes, keepdims=True)]


_BN_OPS = {"AbstractBatchNormTrain": _bn_train, "AbstractBatchNormInference": _bn_inference,
           "AbstractBatchNormTrainGrad": _bn_train_grad}

_ROW_OPS = {"Softmax": _softmax, "SoftmaxWithBias": _softmax_with_bias, "SoftmaxGrad": _softmax_grad,
            "LogSoftmax": _logsoftmax}


def evaluate(inputs, outputs, values, wide=False):
    """Values of ``outputs`` (theano_amd variables) given ``values`` for
    ``inputs``; every Apply node is computed separately, as an unfused graph.

    ``wide=True`` gives the graph's mathematical value instead of the reference's arithmetic: every
    float16 / float32 value, intermediate, accumulator and result is float64 (casts between float
    types then change nothing), integer and boolean nodes are evaluated as they are.  Tests use it as
    the truth that both this oracle and the device are measured against where float32 rounding noise
    of the reference's own evaluation order exceeds the parity tolerance."""
    from theano_amd import gof
    from theano_amd.tensor.elemwise import CAReduce, CAReduceDtype, DimShuffle, Elemwise
    from theano_amd.tensor.basic import MaxAndArgmax, ShapeFloat
    from theano_amd.tensor import views as V
    env = {}
    for var, val in zip(inputs, values):
        env[var] = var.type.filter(np.asarray(val), strict=False, allow_downcast=False)
        if wide:
            env[var] = env[var].astype(_wide(env[var].dtype), copy=False)
    odt = (lambda o: _wide(o.type.dtype)) if wide else (lambda o: o.type.dtype)
    for node in gof.io_toposort(inputs, outputs):
        args = [env[i] if i in env else np.asarray(i.data) for i in node.inputs]
        if wide:
            args = [a.astype(_wide(a.dtype), copy=False) for a in args]
        op = node.op
        if isinstance(op, Elemwise):
            _check_broadcast(node, args)
            _check_dtypes(op.scalar_op, node)
            res = eval_scalar_op(op.scalar_op, args, [o.type.dtype for o in node.outputs], wide)
            shape = np.broadcast_shapes(*[a.shape for a in args])
            res = [np.broadcast_to(r, shape).astype(odt(o), copy=False) if o.type.dtype != "bool"
                   else np.broadcast_to(r, shape) != 0 for r, o in zip(res, node.outputs)]
        elif isinstance(op, DimShuffle):
            res = [dimshuffle(args[0], op.new_order)]
        elif isinstance(op, CAReduce):
            x = args[0]
            idt = str(x.dtype)
            sname = type(op.scalar_op).__name__
            if isinstance(op, CAReduceDtype):
                out_dt = op.dtype if op.dtype is not None else SUM_OUT_DTYPE.get(idt, idt)
                acc_dt = op.acc_dtype if op.acc_dtype is not None else SUM_ACC_DTYPE.get(idt, idt)
            else:                                   # elemwise.py:1273-1274; All / Any: 1597-1598, 1628-1629
                out_dt = "bool" if type(op).__name__ in ("All", "Any") else idt
                acc_dt = "bool" if out_dt == "bool" else idt
            decl = node.inputs[0].type.dtype            # as declared: ``idt`` is already float64 in wide mode
            if isinstance(op, CAReduceDtype):
                want = op.dtype if op.dtype is not None else SUM_OUT_DTYPE.get(decl, decl)
            else:
                want = "bool" if out_dt == "bool" else decl
            assert node.outputs[0].type.dtype == want, "%s of %s is %s, the reference gives %s" % (
                op, node.inputs[0].type.dtype, node.outputs[0].type.dtype, want)
            if acc_dt == "float32" and idt == "float16":
                x = x.astype("float32")
            if wide:
                acc_dt, out_dt = _wide(acc_dt), _wide(out_dt)
            res = [careduce(x, sname, op.axis, acc_dt, out_dt)]
        elif isinstance(op, ShapeFloat):
            res = [np.asarray(args[0].shape[op.i], dtype=_wide(op.dtype) if wide else op.dtype)]
        elif isinstance(op, MaxAndArgmax):
            res = list(max_and_argmax(args[0], op.axis))
        elif isinstance(op, V.Subtensor):          # NumPy basic indexing is the definition (subtensor.py:318-780)
            res = [args[0][V.resolve_index(op.idx_list, args[1:])]]
        elif isinstance(op, V.IncSubtensor):       # subtensor.py:1460-1500
            x = np.array(args[0], copy=True)
            idx = V.resolve_index(op.idx_list, args[2:])
            if op.set_instead_of_inc:
                x[idx] = args[1]
            else:
                x[idx] += args[1]
            res = [x]
        elif isinstance(op, V.Reshape):
            res = [np.reshape(args[0], op.resolve([a.shape for a in args], args))]
        elif isinstance(op, V.Alloc):
            res = [np.array(np.broadcast_to(args[0], op.resolve([a.shape for a in args], args)))]
        elif isinstance(op, V.Join):
            res = [np.concatenate(args, axis=op.axis)]
        elif isinstance(op, V.Rebroadcast):        # theano/compile/ops.py:711-722
            op.check(args[0].shape)
            res = [args[0]]
        elif isinstance(op, V.JoinPart):
            at = sum(a.shape[op.axis] for a in args[1:1 + op.k])
            idx = [slice(None)] * args[0].ndim
            idx[op.axis] = slice(at, at + args[1 + op.k].shape[op.axis])
            res = [args[0][tuple(idx)]]
        elif type(op).__name__ in _BN_OPS:
            res = [np.asarray(r).astype(odt(o), copy=False)
                   for r, o in zip(_BN_OPS[type(op).__name__](op, *args), node.outputs)]
        elif type(op).__name__ in _ROW_OPS:
            res = [_ROW_OPS[type(op).__name__](*args).astype(odt(node.outputs[0]), copy=False)]
        else:
            raise NotImplementedError("oracle cannot evaluate %s" % op)
        for o, v in zip(node.outputs, res):
            env[o] = np.asarray(v)
    return [env[o] if o in env else np.asarray(o.data) for o in outputs]
