"""The HIP Op family: device type, transfers and the lifted Elemwise /
DimShuffle / CAReduce ops.

Each op subclasses its host counterpart and overrides ``make_node`` (device
types) and ``perform`` (one ctypes call), the arrangement the reference uses
for ``GpuElemwise(HideC, Elemwise)`` (``theano/gpuarray/elemwise.py:86-396``),
``GpuDimShuffle`` (:406-446) and ``GpuCAReduceCuda`` (:449-2420); the type and
transfer ops follow ``theano/gpuarray/type.py:129-517`` and
``theano/gpuarray/basic_ops.py:565-744``.
"""
import ctypes

import numpy as np

from .. import scalar as scal
from ..gof import Apply, Op, Type, Variable
from ..tensor.elemwise import CAReduce, DimShuffle, Elemwise
from ..tensor.type import TensorType, _tensor_py_operators
from . import codegen
from .runtime import THX_INDEX, THX_MAX_ND, HipArray, call_flags, check, host_scalar_thx, lib, mark_reused, thx_array


class HipArrayType(Type):
    """dtype and broadcast pattern of an array living in device memory."""

    def __init__(self, dtype, broadcastable, name=None):
        self.dtype = str(dtype)
        if self.dtype not in scal.all_dtypes:
            raise TypeError("Unsupported dtype for HipArrayType: %s" % self.dtype)
        self.broadcastable = tuple(bool(b) for b in broadcastable)
        self.ndim = len(self.broadcastable)
        self.name = name

    def clone(self, dtype=None, broadcastable=None):
        return type(self)(self.dtype if dtype is None else dtype,
                          self.broadcastable if broadcastable is None else broadcastable)

    def filter(self, data, strict=False, allow_downcast=None):
        if not isinstance(data, HipArray):
            if strict:
                raise TypeError("%s expected a HipArray, got %s" % (self, type(data)))
            data = HipArray.from_numpy(TensorType(self.dtype, self.broadcastable).filter(
                data, strict=False, allow_downcast=allow_downcast))
        if str(data.dtype) != self.dtype:
            raise TypeError("%s cannot hold a HipArray of dtype %s" % (self, data.dtype))
        if data.ndim != self.ndim:
            raise TypeError("Wrong number of dimensions: expected %s, got %s with shape %s." %
                            (self.ndim, data.ndim, data.shape))
        for i, b in enumerate(self.broadcastable):
            if b and data.shape[i] != 1:
                raise TypeError("Non-unit value on shape on a broadcastable dimension.", data.shape,
                                self.broadcastable)
        return data

    def __eq__(self, other):
        return (type(self) is type(other) and self.dtype == other.dtype and
                self.broadcastable == other.broadcastable)

    def __hash__(self):
        return hash((type(self), self.dtype, self.broadcastable))

    def __str__(self):
        return "HipArrayType(%s, %s)" % (self.dtype, self.broadcastable)

    __repr__ = __str__

    def as_tensor_variable(self, var):
        return host_from_hip(var)

    # -- the value-level helpers of theano/gpuarray/type.py:260-420; comparisons bring the values to the host
    @staticmethod
    def _host(v):
        return v.to_numpy() if isinstance(v, HipArray) else np.asarray(v)

    @classmethod
    def values_eq(cls, a, b, force_same_dtype=True):
        return TensorType.values_eq(cls._host(a), cls._host(b), force_same_dtype)

    @classmethod
    def values_eq_approx(cls, a, b, rtol=None, atol=None):
        return TensorType.values_eq_approx(cls._host(a), cls._host(b), rtol, atol)

    @staticmethod
    def may_share_memory(a, b):
        """Two device arrays may overlap when they are views of one allocation (``:300-306``)."""
        return isinstance(a, HipArray) and isinstance(b, HipArray) and a.buffer is b.buffer

    def value_zeros(self, shape):
        return HipArray.from_numpy(np.zeros(shape, dtype=self.dtype))

    def get_shape_info(self, obj):
        return obj.shape

    def get_size(self, shape_info):
        n = np.dtype(self.dtype).itemsize
        for s in shape_info:
            n *= int(s)
        return n

    def convert_variable(self, var):
        """``var`` under this type's broadcast pattern (a host variable is moved to the device first) when dtype
        and rank agree and it is at least as broadcastable wherever this type is; None otherwise (``:243-258``)."""
        vt = var.type
        if vt == self:
            return var
        if (isinstance(vt, (TensorType, HipArrayType)) and vt.dtype == self.dtype and vt.ndim == self.ndim and
                all(sb == ob or ob for sb, ob in zip(self.broadcastable, vt.broadcastable))):
            # the pattern is changed on the host-typed variable; the transfers either side of it are cut when
            # the graph is compiled
            host = var if isinstance(vt, TensorType) else host_from_hip(var)
            return as_hip_variable(TensorType(self.dtype, self.broadcastable).convert_variable(host))
        return None

    def filter_variable(self, other, allow_convert=True):
        """A symbolic variable (or a value, made a device constant's source) as a variable of this type, or
        TypeError (``:204-241``)."""
        if not isinstance(other, Variable):
            from ..tensor.type import constant
            other = constant(TensorType(self.dtype, self.broadcastable).filter(other))
        if other.type == self:
            return other
        if allow_convert:
            conv = self.convert_variable(other)
            if conv is not None and conv.type == self:
                return conv
        raise TypeError("Cannot convert Type %s (of Variable %s) into Type %s. You can try to manually convert %s "
                        "into a %s." % (other.type, other, self, other, self))


class HipArrayVariable(_tensor_py_operators, Variable):
    pass


HipArrayType.Variable = HipArrayVariable


def _is_host_scalar(var):
    """A host tensor whose every dimension is broadcastable travels as a
    kernel argument instead of being copied to the device (values of up to 8
    bytes: a complex128 goes through device memory like any array)."""
    return isinstance(var.type, TensorType) and all(var.type.broadcastable) and var.type.dtype != "complex128"


def as_hip_variable(x):
    """Device version of ``x``; a transfer of a transfer is short-circuited
    (``theano/gpuarray/basic_ops.py:37-98``)."""
    if isinstance(x, Variable) and isinstance(x.type, HipArrayType):
        return x
    if isinstance(x, Variable) and isinstance(x.type, TensorType):
        if x.owner is not None and isinstance(x.owner.op, HipToHost):
            return x.owner.inputs[0]
        return hip_from_host(x)
    from ..tensor.type import as_tensor_variable
    return hip_from_host(as_tensor_variable(x))


class HostToHip(Op):
    __props__ = ()

    def make_node(self, x):
        if not isinstance(x.type, TensorType):
            raise TypeError("HostToHip takes a host tensor", x)
        return Apply(self, [x], [HipArrayType(x.type.dtype, x.type.broadcastable)()])

    def perform(self, node, inputs, output_storage):
        x = inputs[0]
        output_storage[0][0] = x if isinstance(x, HipArray) else HipArray.from_numpy(x)

    def infer_shape(self, node, shapes):
        return shapes

    def grad(self, inputs, grads):
        return [host_from_hip(as_hip_variable(grads[0]))]

    def __str__(self):
        return "HostToHip"


class HipToHost(Op):
    __props__ = ()

    def make_node(self, x):
        if not isinstance(x.type, HipArrayType):
            raise TypeError("HipToHost takes a device array", x)
        return Apply(self, [x], [TensorType(x.type.dtype, x.type.broadcastable)()])

    def perform(self, node, inputs, output_storage):
        output_storage[0][0] = inputs[0].to_numpy()

    def infer_shape(self, node, shapes):
        return shapes

    def grad(self, inputs, grads):
        return [as_hip_variable(grads[0])]

    def __str__(self):
        return "HipToHost"


hip_from_host = HostToHip()
host_from_hip = HipToHost()


class HipDimShuffle(DimShuffle):
    """DimShuffle of a device array: a new (shape, strides) header over the
    same buffer, computed like ``theano/tensor/c_code/dimshuffle.c:55-98``."""

    def make_node(self, input):
        input = as_hip_variable(input)
        host = DimShuffle.make_node(self, TensorType(input.type.dtype, input.type.broadcastable)())
        ot = host.outputs[0].type
        return Apply(self, [input], [HipArrayType(ot.dtype, ot.broadcastable)()])

    def __str__(self):
        return "HipDimShuffle{%s}" % ",".join(str(x) for x in self.new_order)

    def perform(self, node, inputs, output_storage):
        (x,) = inputs
        # the header computed for the previous call stands while the input's layout is the same
        memo = node.tag.get("view")
        if memo is not None and memo[0] == x.shape and memo[1] == x.strides:
            output_storage[0][0] = HipArray._raw(x.buffer, x.offset, memo[2], memo[3], x.dtype, x.code)
            return
        if x.ndim != len(self.input_broadcastable):
            raise TypeError("input has %d dimensions, DimShuffle was built for %d" %
                            (x.ndim, len(self.input_broadcastable)))
        if len(self.new_order) > THX_MAX_ND:    # the reference raises ValueError past NumPy's limit (test_too_big_rank)
            raise ValueError("DimShuffle to rank %d: device arrays have at most %d dimensions" %
                             (len(self.new_order), THX_MAX_ND))
        for d in self.drop:
            if x.shape[d] != 1:
                raise ValueError("cannot drop dimension %d of extent %d" % (d, x.shape[d]))
        shape, strides = [], []
        for v in self.new_order:
            if v == "x":
                shape.append(1)
                strides.append(0)
            else:
                shape.append(x.shape[v])
                strides.append(x.strides[v])
        # extent-1 dimensions get the stride a C-contiguous array would have
        for i in range(len(shape) - 1, -1, -1):
            if shape[i] == 1:
                strides[i] = x.dtype.itemsize if i == len(shape) - 1 else strides[i + 1] * shape[i + 1]
        node.tag["view"] = (x.shape, x.strides, tuple(shape), tuple(strides))
        output_storage[0][0] = x.view(shape, strides)


def _operand(value, nd, slot):
    if isinstance(value, HipArray):
        return value.as_thx(slot)
    return host_scalar_thx(value, nd, slot)


def _check_runtime_broadcast(node_inputs, values, nd):
    """Non-broadcastable dimensions must agree exactly; an extent of 1 only
    broadcasts where the type says so (``theano/tensor/elemwise.py:720-740``)."""
    shape = None
    for k, (var, val) in enumerate(zip(node_inputs, values)):
        if type(val) is not HipArray:
            if not isinstance(val, np.ndarray) or val.size != 1:
                raise TypeError("input %d must be a device array or a one-element host array" % k)
            continue
        if shape is None and not any(var.type.broadcastable):
            shape = val.shape  # fast path: the first full-shaped input fixes the result shape
            if len(shape) != nd:
                raise TypeError("input %d has rank %d, expected %d" % (k, len(shape), nd))
            first = k
    if shape is not None:
        ok = True
        for k, (var, val) in enumerate(zip(node_inputs, values)):
            if type(val) is HipArray and val.shape != shape:
                vs = val.shape
                if len(vs) != nd or any(v != s and not (b and v == 1)
                                        for v, s, b in zip(vs, shape, var.type.broadcastable)) or any(
                                            b and v != 1 for v, b in zip(vs, var.type.broadcastable)):
                    ok = False
                    break
        if ok:
            return shape
    shape = [1] * nd
    owner = [None] * nd
    for k, (var, val) in enumerate(zip(node_inputs, values)):
        if not isinstance(val, HipArray):
            continue
        if val.ndim != nd:
            raise TypeError("input %d has rank %d, expected %d" % (k, val.ndim, nd))
        vshape = val.shape
        for d in range(nd):
            if var.type.broadcastable[d]:
                if vshape[d] != 1:
                    raise ValueError("input %d has extent %d on a broadcastable dimension %d" % (k, vshape[d], d))
                continue
            if owner[d] is None:
                owner[d], shape[d] = k, vshape[d]
            elif vshape[d] != shape[d]:
                # an extent of 1 beside an empty operand is let through and the result is empty, as in
                # Elemwise.perform (theano/tensor/elemwise.py:720-751: the check fires only when the largest
                # extent is not 1; `[] + [1]` is a good case of the reference's broadcast testers)
                if (vshape[d], shape[d]) == (0, 1):
                    owner[d], shape[d] = k, 0
                elif (vshape[d], shape[d]) != (1, 0):
                    raise ValueError("Input dimension mis-match. (input[%d].shape[%d] = %d, input[%d].shape[%d] = %d)" %
                                     (owner[d], d, shape[d], k, d, vshape[d]))
    return tuple(shape)


_elemwise_handles = {}
_reduce_handles = {}


class HipElemwise(Elemwise):
    """Elemwise executed by one fused kernel.  Inputs are device arrays, or host
    tensors broadcastable in every dimension, which are passed by value."""

    def make_node(self, *inputs):
        from ..tensor.type import as_tensor_variable
        ins = []
        for i in inputs:
            if not isinstance(i, Variable):
                i = as_tensor_variable(i)
            if isinstance(i.type, HipArrayType) or _is_host_scalar(i):
                ins.append(i)
            else:
                ins.append(as_hip_variable(i))
        shadow = [TensorType(i.type.dtype, i.type.broadcastable)() for i in ins]
        out_dtypes, out_b, shadow2 = self.get_output_info(DimShuffle, *shadow)
        # rank alignment, mirrored on the real inputs
        target = max(i.type.ndim for i in ins)
        aligned = []
        for i in ins:
            diff = target - i.type.ndim
            if diff and isinstance(i.type, HipArrayType):
                i = HipDimShuffle(i.type.broadcastable, ["x"] * diff + list(range(i.type.ndim)))(i)
            aligned.append(i)  # host scalars are passed by value whatever their rank
        if len(out_dtypes) < 1:
            raise NotImplementedError("an Elemwise needs at least one output")
        outputs = [HipArrayType(dt, b)() for dt, b in zip(out_dtypes, out_b)]
        return Apply(self, aligned, outputs)

    def _handle(self, node):
        in_dt = tuple(i.type.dtype for i in node.inputs)
        key = (self.scalar_op, in_dt)
        h = _elemwise_handles.get(key)
        if h is None:
            src, name, out_dt = codegen.elemwise_functor(self.scalar_op, in_dt, [o.type.dtype for o in node.outputs])
            codes = (ctypes.c_int32 * (len(in_dt) + len(out_dt)))(*[scal.dtype_code(d) for d in in_dt + tuple(out_dt)])
            handle = ctypes.c_void_p()
            check(lib.thx_elemwise_new(src.encode(), name.encode(), len(in_dt), len(out_dt), codes,
                                       ctypes.byref(handle)))
            h = (handle, len(in_dt), len(out_dt))
            _elemwise_handles[key] = h
        return h

    def perform(self, node, inputs, output_storage):
        flags = call_flags(node)
        cache = node.tag.get("thx")
        if cache is None:
            handle, nin, nout = self._handle(node)
            # inputs whose layout decides the outputs' (theano/tensor/elemwise.py:928-937): all but
            # the ones broadcast along every dimension
            full = [k for k, v in enumerate(node.inputs) if not all(v.type.broadcastable)]
            cache = node.tag["thx"] = (handle, nin, nout, (thx_array * nin)(), (thx_array * nout)(),
                                       node.outputs[0].type.ndim, dict(self.inplace_pattern),
                                       [np.dtype(o.type.dtype) for o in node.outputs],
                                       full if node.outputs[0].type.ndim > 1 else [])
        handle, nin, nout, ins, outs, nd, inplace, out_dt, full = cache
        shape = _check_runtime_broadcast(node.inputs, inputs, nd)
        last = node.tag.get("thx_last")
        if last is None:
            last = node.tag["thx_last"] = [None] * len(inputs)
        k = 0
        for v in inputs:
            if type(v) is HipArray:
                v.as_thx(ins[k])
            elif last[k] is not v:              # the same host array as last time: its descriptor stands
                host_scalar_thx(v, nd, ins[k])
                last[k] = v
            k += 1
        # column-major outputs when every such input is column-major, as the reference allocates them
        fortran = False
        for k in full:
            v = inputs[k]
            if type(v) is not HipArray or not v.is_fortran:
                break
        else:
            fortran = bool(full)
        results = []
        for k in range(nout):
            if k in inplace:
                arr = inputs[inplace[k]]
                if arr.shape != shape:
                    raise ValueError("in-place output %d has shape %s, the result has %s" % (k, arr.shape, shape))
            elif fortran:
                arr = HipArray._new_fortran(shape, out_dt[k])
            else:
                arr = HipArray._new_contiguous(shape, out_dt[k])
            arr.as_thx(outs[k])
            results.append(arr)
        mark_reused(node, ins, outs)
        rc = lib.thx_elemwise_call(handle, ins, outs, flags)
        if rc:
            check(rc)
        for k in range(nout):
            output_storage[k][0] = results[k]


class HipCAReduce(CAReduce):
    """K simultaneous reductions over the same axes in one pass.

    ``scalar_ops[k]`` folds, in ``acc_dtypes[k]``, the k-th value produced per
    element by ``pre_scalar_op`` applied to the inputs (None: the single input
    itself).  ``post_scalar_op`` maps the K results to the outputs (None: cast
    result k to ``out_dtypes[k]``).  A lifted ``CAReduce`` is the K = 1 case
    without prologue or epilogue; the fusion pass widens it.  The generalisation
    of ``GpuCAReduceCuda``'s ``pre_scalar_op`` (``theano/gpuarray/elemwise.py:492-493``)."""

    __props__ = ("scalar_ops", "axis", "acc_dtypes", "out_dtypes", "pre_scalar_op", "post_scalar_op",
                 "post_in_dtypes", "n_extra")

    def __init__(self, scalar_ops, axis, acc_dtypes, out_dtypes, pre_scalar_op=None, post_scalar_op=None,
                 post_in_dtypes=None, n_extra=0):
        scalar_ops = tuple(scalar_ops)
        for op in scalar_ops:
            if op.nin not in (-1, 2) or op.nout != 1:
                raise NotImplementedError("CAReduce only supports binary functions with a single output.")
        self.scalar_ops = scalar_ops
        self.scalar_op = scalar_ops[0]
        if axis is None:
            self.axis = None
        elif isinstance(axis, (int, np.integer)):
            self.axis = (int(axis),)
        else:
            self.axis = tuple(sorted(set(int(a) for a in axis)))
        self.acc_dtypes = tuple(acc_dtypes)
        self.out_dtypes = tuple(out_dtypes)
        self.pre_scalar_op = pre_scalar_op
        self.post_scalar_op = post_scalar_op
        # with an epilogue: the dtype each reduction result has before the epilogue reads it, and the
        # number of trailing inputs that only the epilogue uses (host scalars, or device arrays with
        # one element per result)
        self.post_in_dtypes = None if post_in_dtypes is None else tuple(post_in_dtypes)
        self.n_extra = int(n_extra)
        if len(self.acc_dtypes) != len(scalar_ops):
            raise ValueError("one accumulator dtype per reduction")
        if self.n_extra and post_scalar_op is None:
            raise ValueError("extra scalars need an epilogue")

    def _props(self):
        return (self.scalar_ops, self.axis, self.acc_dtypes, self.out_dtypes, self.pre_scalar_op, self.post_scalar_op,
                self.post_in_dtypes, self.n_extra)

    def __str__(self):
        ops = ",".join(str(o) for o in self.scalar_ops)
        ax = "" if self.axis is None else "{%s}" % ", ".join(str(a) for a in self.axis)
        extra = ""
        if self.pre_scalar_op is not None:
            extra += ", pre=%s" % self.pre_scalar_op
        if self.post_scalar_op is not None:
            extra += ", post=%s" % self.post_scalar_op
        return "HipCAReduce{%s}%s{acc=%s%s}" % (ops, ax, ",".join(self.acc_dtypes), extra)

    def make_node(self, *inputs):
        extras = list(inputs[len(inputs) - self.n_extra:]) if self.n_extra else []
        inputs = inputs[:len(inputs) - self.n_extra] if self.n_extra else inputs
        for e in extras:
            if not (_is_host_scalar(e) or isinstance(e.type, HipArrayType)):
                raise TypeError("epilogue operands must be host scalars or device arrays", e)
        ins = [i if (isinstance(i.type, HipArrayType) or _is_host_scalar(i)) else as_hip_variable(i) for i in inputs]
        nd = max(i.type.ndim for i in ins)
        if any(i.type.ndim != nd for i in ins if isinstance(i.type, HipArrayType)):
            raise TypeError("HipCAReduce inputs must share one rank")
        if self.pre_scalar_op is None and len(ins) != 1:
            raise TypeError("a reduction without prologue takes exactly one input")
        axis = self.axis if self.axis is not None else tuple(range(nd))
        for a in axis:
            if a >= nd or a < 0:
                raise ValueError("Not enough dimensions on the input to reduce on axis %s" % a)
        bcast = [all(b) for b in zip(*[i.type.broadcastable for i in ins if i.type.ndim == nd])]
        ob = [b for d, b in enumerate(bcast) if d not in axis]
        return Apply(self, ins + extras, [HipArrayType(dt, ob)() for dt in self.out_dtypes])

    def infer_shape(self, node, shapes):
        shapes = shapes[:len(shapes) - self.n_extra] if self.n_extra else shapes
        nd = max(i.type.ndim for i in node.inputs[:len(shapes)])
        axis = self.axis if self.axis is not None else tuple(range(nd))
        full = [max(s[d] for s in shapes if len(s) == nd) for d in range(nd)]
        kept = tuple(full[d] for d in range(nd) if d not in axis)
        return [kept for _ in node.outputs]

    def _handle(self, node):
        n_red = len(node.inputs) - self.n_extra
        in_dt = tuple(i.type.dtype for i in node.inputs[:n_red])
        ex_dt = tuple(i.type.dtype for i in node.inputs[n_red:])
        ex_arr = tuple(isinstance(i.type, HipArrayType) for i in node.inputs[n_red:])
        # float16 storage behind every operand that varies along a reduced dimension
        nd = max(i.type.ndim for i in node.inputs[:n_red])
        axis = self.axis if self.axis is not None else tuple(range(nd))
        data = [i for i in node.inputs[:n_red] if isinstance(i.type, HipArrayType) and
                not all(i.type.broadcastable[a] for a in axis)]
        half_data = bool(data) and all(i.type.dtype == "float16" for i in data)
        key = (self._props(), in_dt, ex_dt, ex_arr, half_data)
        h = _reduce_handles.get(key)
        if h is None:
            src, name, acc_bytes = codegen.reduce_functor(self.scalar_ops, self.acc_dtypes, in_dt, self.out_dtypes,
                                                          self.pre_scalar_op, self.post_scalar_op, ex_dt,
                                                          self.post_in_dtypes, ex_arr, half_data)
            all_dt = in_dt + self.out_dtypes + ex_dt
            codes = (ctypes.c_int32 * len(all_dt))(*[scal.dtype_code(d) for d in all_dt])
            handle = ctypes.c_void_p()
            check(lib.thx_reduce_new(src.encode(), name.encode(), len(in_dt), len(self.out_dtypes), len(ex_dt), codes,
                                     acc_bytes, ctypes.byref(handle)))
            h = (handle, len(in_dt), len(self.out_dtypes))
            _reduce_handles[key] = h
        return h

    def perform(self, node, inputs, output_storage):
        flags = call_flags(node)
        cache = node.tag.get("thx")
        if cache is None:
            handle, nin, nout = self._handle(node)
            nd = max(i.type.ndim for i in node.inputs[:nin])
            axis = self.axis if self.axis is not None else tuple(range(nd))
            mask = (ctypes.c_uint8 * max(nd, 1))(*[1 if d in axis else 0 for d in range(nd)])
            cache = node.tag["thx"] = (handle, nin, nout, (thx_array * len(node.inputs))(), (thx_array * nout)(), nd,
                                       axis, mask, [np.dtype(d) for d in self.out_dtypes])
        handle, nin, nout, ins, outs, nd, axis, mask, out_dt = cache
        shape = _check_runtime_broadcast(node.inputs[:nin], inputs[:nin], nd)
        n_red = 1
        for a in axis:
            n_red *= shape[a]
        if n_red == 0:
            for op in self.scalar_ops:
                if codegen.reduce_identity(op, "float32") is None or isinstance(op, (scal.Maximum, scal.Minimum)):
                    raise ValueError("Input of CAReduce{%s} has zero-size on axis %s" % (op, axis))
        kept = tuple(shape[d] for d in range(nd) if d not in axis)
        for k in range(nin, len(inputs)):
            v = inputs[k]
            if type(v) is HipArray:
                if [d for d in v.shape if d != 1] != [d for d in kept if d != 1]:
                    raise ValueError("Input dimension mis-match. (epilogue operand %d has shape %s, the result has %s)"
                                     % (k - nin, v.shape, kept))
                if not v.scaled_contiguous:     # the epilogue reads one value per result at index x one stride
                    inputs = list(inputs)
                    inputs[k] = v.copy()
        last = node.tag.get("thx_last")
        if last is None:
            last = node.tag["thx_last"] = [None] * len(inputs)
        for k, v in enumerate(inputs):
            if type(v) is HipArray:
                v.as_thx(ins[k])
            elif last[k] is not v:              # the same host array as last time: its descriptor stands
                host_scalar_thx(v, nd, ins[k])
                last[k] = v
        results = []
        for k in range(nout):
            arr = HipArray._new_contiguous(kept, out_dt[k])
            arr.as_thx(outs[k])
            results.append(arr)
        mark_reused(node, ins, outs)
        rc = lib.thx_reduce_call(handle, ins, mask, outs, flags)
        if rc:
            check(rc)
        for k, arr in enumerate(results):
            output_storage[k][0] = arr


_elemwise_reduce_handles = {}


class HipElemwiseReduce(HipElemwise):
    """An elementwise kernel that also reduces some of its results over every dimension but the last:
    ``r = f(a, b, ...)`` stored, and ``reduce(r, axis=all but the last)`` alongside, e.g. the per-channel
    sum of an NHWC result that is an output too.  Outputs: the elementwise results, then one reduction
    result per entry of ``red_of`` (the index of the elementwise output it reduces).  Where the kernel
    reads its inputs through LDS tiles (permuted views) the reduction rides along in the same launch
    and the result is never read back; otherwise the library reduces the stored result.  The
    reference runs GpuElemwise and GpuCAReduceCuda one after the other
    (``theano/gpuarray/elemwise.py:376, 1095-1723``)."""

    __props__ = ("scalar_op", "red_of", "red_scalar_ops", "red_acc_dtypes", "red_out_dtypes")

    def __init__(self, scalar_op, red_of, red_scalar_ops, red_acc_dtypes, red_out_dtypes):
        HipElemwise.__init__(self, scalar_op, None)
        self.red_of = tuple(int(k) for k in red_of)
        self.red_scalar_ops = tuple(red_scalar_ops)
        self.red_acc_dtypes = tuple(red_acc_dtypes)
        self.red_out_dtypes = tuple(red_out_dtypes)

    def _props(self):
        return (self.scalar_op, self.red_of, self.red_scalar_ops, self.red_acc_dtypes, self.red_out_dtypes)

    def __str__(self):
        return "HipElemwiseReduce{%s; %s}" % (self.scalar_op, ", ".join(
            "%s(out %d)" % (o, k) for o, k in zip(self.red_scalar_ops, self.red_of)))

    def make_node(self, *inputs):
        base = HipElemwise.make_node(self, *inputs)
        nd = base.outputs[0].type.ndim
        if nd < 2:
            raise TypeError("HipElemwiseReduce needs results of rank 2 or more")
        last = base.outputs[0].type.broadcastable[-1]
        outs = [o.type() for o in base.outputs] + [HipArrayType(dt, (last,))() for dt in self.red_out_dtypes]
        return Apply(self, base.inputs, outs)

    def infer_shape(self, node, shapes):
        n_ew = len(node.outputs) - len(self.red_of)
        nd = node.outputs[0].type.ndim
        full = [max(s[d] for s in shapes if len(s) == nd) for d in range(nd)]
        return [tuple(full)] * n_ew + [(full[-1],)] * len(self.red_of)

    def _handle(self, node):
        in_dt = tuple(i.type.dtype for i in node.inputs)
        key = (self._props(), in_dt)
        h = _elemwise_reduce_handles.get(key)
        if h is None:
            n_ew = len(node.outputs) - len(self.red_of)
            ew_dt = [o.type.dtype for o in node.outputs[:n_ew]]
            red_in = tuple(ew_dt[k] for k in self.red_of)
            K = len(self.red_of)
            if K == 1:
                pre = None
            else:       # several reductions in one functor: input j feeds accumulator j
                s_in = [scal.Scalar(dt)() for dt in red_in]
                pre = scal.Composite(s_in, [scal.identity(v) for v in s_in])
            rsrc, rname, acc_bytes = codegen.reduce_functor(self.red_scalar_ops, self.red_acc_dtypes, red_in,
                                                            self.red_out_dtypes, pre)
            fsrc, fname, out_dt = codegen.elemwise_functor(self.scalar_op, in_dt, ew_dt, red=(rname, self.red_of))
            rcodes = (ctypes.c_int32 * (2 * K))(*[scal.dtype_code(d) for d in red_in + self.red_out_dtypes])
            rh = ctypes.c_void_p()
            check(lib.thx_reduce_new(rsrc.encode(), rname.encode(), K, K, 0, rcodes, acc_bytes, ctypes.byref(rh)))
            codes = (ctypes.c_int32 * (len(in_dt) + n_ew))(*[scal.dtype_code(d) for d in in_dt + tuple(out_dt)])
            eh = ctypes.c_void_p()
            check(lib.thx_elemwise_new((rsrc + fsrc).encode(), fname.encode(), len(in_dt), n_ew, codes, ctypes.byref(eh)))
            check(lib.thx_elemwise_attach_reduce(eh, rh, (ctypes.c_int32 * K)(*self.red_of)))
            h = _elemwise_reduce_handles[key] = (eh, rh, len(in_dt), n_ew)
        return h

    def perform(self, node, inputs, output_storage):
        cache = node.tag.get("thx")
        if cache is None:
            eh, rh, nin, n_ew = self._handle(node)
            K = len(self.red_of)
            cache = node.tag["thx"] = (eh, nin, n_ew, K, (thx_array * nin)(), (thx_array * n_ew)(), (thx_array * K)(),
                                       node.outputs[0].type.ndim, [np.dtype(o.type.dtype) for o in node.outputs])
        eh, nin, n_ew, K, ins, outs, routs, nd, out_dt = cache
        shape = _check_runtime_broadcast(node.inputs, inputs, nd)
        for op in self.red_scalar_ops:
            if 0 in shape[:-1] and isinstance(op, (scal.Maximum, scal.Minimum)):
                raise ValueError("Input of CAReduce{%s} has zero-size on axis %s" % (op, tuple(range(nd - 1))))
        for k, v in enumerate(inputs):
            if type(v) is HipArray:
                v.as_thx(ins[k])
            else:
                host_scalar_thx(v, nd, ins[k])
        results = []
        for k in range(n_ew):
            arr = HipArray._new_contiguous(shape, out_dt[k])
            arr.as_thx(outs[k])
            results.append(arr)
        for k in range(K):
            arr = HipArray._new_contiguous((shape[-1],), out_dt[n_ew + k])
            arr.as_thx(routs[k])
            results.append(arr)
        # the positions recorded for the node's results run over the stored results first, then the reduced ones
        mark_reused(node, ins, [outs[k] if k < n_ew else routs[k - n_ew] for k in range(n_ew + K)])
        rc = lib.thx_elemwise_reduce_call(eh, ins, outs, routs, call_flags(node))
        if rc:
            check(rc)
        for k, arr in enumerate(results):
            output_storage[k][0] = arr


_argmax_handles = {}


class HipMaxAndArgmax(Op):
    """``MaxAndArgmax`` on the device (the role of ``GpuMaxAndArgmax``,
    ``theano/gpuarray/reduction.py:14-137``): one pass of the reduction kernels
    over (value, position) pairs; the position comes from the library's index
    operand, so no index array exists in memory.  ``pre_scalar_op`` (one output)
    is an elementwise producer computed on the fly, e.g. the negation ``argmin``
    puts in front."""

    __props__ = ("axis", "pre_scalar_op")

    def __init__(self, axis, pre_scalar_op=None):
        self.axis = tuple(sorted(int(a) for a in axis))
        self.pre_scalar_op = pre_scalar_op

    def _props(self):
        return (self.axis, self.pre_scalar_op)

    def __str__(self):
        pre = "" if self.pre_scalar_op is None else ", pre=%s" % self.pre_scalar_op
        return "HipMaxAndArgmax{%s%s}" % (", ".join(map(str, self.axis)), pre)

    def make_node(self, *inputs):
        ins = [i if (isinstance(i.type, HipArrayType) or _is_host_scalar(i)) else as_hip_variable(i) for i in inputs]
        nd = max(i.type.ndim for i in ins)
        if any(i.type.ndim != nd for i in ins if isinstance(i.type, HipArrayType)):
            raise TypeError("HipMaxAndArgmax inputs must share one rank")
        if self.pre_scalar_op is None:
            if len(ins) != 1:
                raise TypeError("without prologue the reduction takes exactly one input")
            vdt = ins[0].type.dtype
        else:
            vdt = self.pre_scalar_op.make_node(*[scal.Scalar(i.type.dtype)() for i in ins]).outputs[0].type.dtype
        for a in self.axis:
            if a < 0 or a >= nd:
                raise ValueError("MaxAndArgmax: bad axis argument")
        bcast = [all(b) for b in zip(*[i.type.broadcastable for i in ins if i.type.ndim == nd])]
        ob = [b for d, b in enumerate(bcast) if d not in self.axis]
        return Apply(self, ins, [HipArrayType(vdt, ob)(), HipArrayType("int64", ob)()])

    def infer_shape(self, node, shapes):
        nd = max(len(s) for s in shapes)
        full = [max(s[d] for s in shapes if len(s) == nd) for d in range(nd)]
        kept = tuple(full[d] for d in range(nd) if d not in self.axis)
        return [kept, kept]

    def _handle(self, node, packed):
        in_dt = tuple(i.type.dtype for i in node.inputs)
        vdt = node.outputs[0].type.dtype
        key = (self._props(), in_dt, packed)
        h = _argmax_handles.get(key)
        if h is None:
            src, name, acc_bytes = codegen.argmax_functor(in_dt, vdt, self.pre_scalar_op, packed)
            all_dt = in_dt + ("int64", vdt, "int64")
            codes = (ctypes.c_int32 * len(all_dt))(*[scal.dtype_code(d) for d in all_dt])
            handle = ctypes.c_void_p()
            check(lib.thx_reduce_new(src.encode(), name.encode(), len(in_dt) + 1, 2, 0, codes, acc_bytes,
                                     ctypes.byref(handle)))
            h = _argmax_handles[key] = handle
        return h

    def perform(self, node, inputs, output_storage):
        cache = node.tag.get("thx")
        if cache is None:
            small = np.dtype(node.outputs[0].type.dtype).itemsize <= 4
            # one 64-bit key per (value, position) pair while positions fit 31 bits, else the pair itself
            handle = (self._handle(node, True) if small else None, self._handle(node, False))
            nin = len(node.inputs)
            nd = max(i.type.ndim for i in node.inputs)
            ins = (thx_array * (nin + 1))()
            ix = ins[nin]                       # the index operand: int64, extent 1 everywhere, no memory
            ix.base, ix.offset_bytes, ix.nd, ix.dtype = None, 0, nd, scal.dtype_code("int64") | THX_INDEX
            for d in range(nd):
                ix.shape[d], ix.strides_bytes[d] = 1, 0
            mask = (ctypes.c_uint8 * max(nd, 1))(*[1 if d in self.axis else 0 for d in range(nd)])
            cache = node.tag["thx"] = (handle, nin, ins, (thx_array * 2)(), nd, mask,
                                       np.dtype(node.outputs[0].type.dtype))
        handle, nin, ins, outs, nd, mask, vdt = cache
        shape = _check_runtime_broadcast(node.inputs, inputs, nd)
        n_red = 1
        for a in self.axis:
            n_red *= shape[a]
        if n_red == 0:
            raise ValueError("attempt to get argmax of an empty sequence")
        handle = handle[0] if (handle[0] is not None and n_red < 2 ** 31) else handle[1]
        for k, v in enumerate(inputs):
            _operand(v, nd, ins[k])
        kept = tuple(shape[d] for d in range(nd) if d not in self.axis)
        mx = HipArray._new_contiguous(kept, vdt)
        am = HipArray._new_contiguous(kept, np.dtype("int64"))
        mx.as_thx(outs[0])
        am.as_thx(outs[1])
        mark_reused(node, ins, outs)
        rc = lib.thx_reduce_call(handle, ins, mask, outs, call_flags(node))
        if rc:
            check(rc)
        output_storage[0][0] = mx
        output_storage[1][0] = am
