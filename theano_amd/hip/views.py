"""Device versions of the view / data-movement ops of ``theano_amd.tensor.views``.

Indexing, reshaping a contiguous array and taking a part of a joined gradient
are new headers over the same buffer.  Copies (reshape of a strided array,
``alloc``, ``join``, ``inc_subtensor``) run as the library's elementwise kernel
with a strided output: ``identity`` / ``add`` of the source written straight
into the destination view, so each costs one read and one write of the data.
The counterparts in the reference are ``GpuSubtensor`` / ``GpuIncSubtensor``
(``theano/gpuarray/subtensor.py:30-420``), ``GpuReshape``, ``GpuAlloc`` and
``GpuJoin`` (``theano/gpuarray/basic_ops.py:820-1000, 1090-1400``).
"""
import ctypes

import numpy as np

from .. import scalar as scal
from ..gof import Apply
from ..tensor import views as V
from . import codegen
from .ops import HipArrayType, _is_host_scalar, as_hip_variable
from .runtime import HipArray, call_flags, check, host_scalar_thx, lib, thx_array

_copy_handles = {}


def _elemwise_handle(scalar_op, in_dtypes, out_dtype):
    key = (scalar_op, tuple(in_dtypes), out_dtype)
    h = _copy_handles.get(key)
    if h is None:
        src, name, out_dt = codegen.elemwise_functor(scalar_op, list(in_dtypes), [out_dtype])
        all_dt = list(in_dtypes) + [out_dtype]
        codes = (ctypes.c_int32 * len(all_dt))(*[scal.dtype_code(d) for d in all_dt])
        h = ctypes.c_void_p()
        check(lib.thx_elemwise_new(src.encode(), name.encode(), len(in_dtypes), 1, codes, ctypes.byref(h)))
        _copy_handles[key] = h
    return h


def _run(scalar_op, sources, dest):
    """dest[...] = scalar_op(*sources), sources broadcast against dest."""
    nd = dest.ndim
    ins = (thx_array * len(sources))()
    for k, s in enumerate(sources):
        if isinstance(s, HipArray):
            if s.ndim < nd:    # left-pad with broadcast dimensions
                s = s.view((1,) * (nd - s.ndim) + s.shape, (0,) * (nd - s.ndim) + s.strides)
            s.as_thx(ins[k])
        else:
            host_scalar_thx(s, nd, ins[k])
    outs = (thx_array * 1)()
    dest.as_thx(outs[0])
    dtypes = [str(s.dtype) for s in sources]
    check(lib.thx_elemwise_call(_elemwise_handle(scalar_op, dtypes, str(dest.dtype)), ins, outs, call_flags()))


def copy_into(source, dest):
    if dest.size:
        _run(scal.identity, [source], dest)


def _device(v):
    return v if (isinstance(v.type, HipArrayType) or _is_host_scalar(v)) else as_hip_variable(v)


def _as_device_value(v, dtype):
    """A run-time operand as something ``_run`` accepts."""
    if isinstance(v, HipArray):
        return v
    return np.asarray(v, dtype=dtype).reshape((1,) * np.ndim(v))


def _index_values(vals):
    """Run-time values of an index's scalar inputs; one computed on the device (``i * n``) is
    fetched, which waits for the kernels before it."""
    return [v.to_numpy() if isinstance(v, HipArray) else v for v in vals]


class HipSubtensor(V.Subtensor):
    def make_node(self, x, *scalars):
        x = as_hip_variable(x)
        self.check_inputs(x, scalars)
        return Apply(self, [x] + list(scalars),
                     [HipArrayType(x.type.dtype, self.out_broadcastable(x.type.broadcastable))()])

    def perform(self, node, inputs, output_storage):
        x = inputs[0]
        idx = V.resolve_index(self.idx_list, _index_values(inputs[1:])) if len(inputs) > 1 else self.idx_list
        shape, strides, offset = V.index_view(x.shape, x.strides, x.offset, idx)
        output_storage[0][0] = x.view(shape, strides, offset)


class HipRebroadcast(V.Rebroadcast):
    def __init__(self, axis):
        V.Rebroadcast.__init__(self, *axis)

    def make_node(self, x):
        x = as_hip_variable(x)
        return Apply(self, [x], [HipArrayType(x.type.dtype, self.out_type(x))()])

    def perform(self, node, inputs, output_storage):
        (x,) = inputs
        self.check(x.shape)
        output_storage[0][0] = x


class HipIncSubtensor(V.IncSubtensor):
    def make_node(self, x, y, *scalars):
        x = as_hip_variable(x)
        y = _device(y)
        if y.type.dtype != x.type.dtype:
            raise TypeError("the increment must have the dtype of the tensor (%s), got %s" % (x.type.dtype, y.type.dtype))
        V.Subtensor(self.idx_list).check_inputs(x, scalars)
        return Apply(self, [x, y] + list(scalars), [x.type()])

    def perform(self, node, inputs, output_storage):
        x, y = inputs[:2]
        idx = V.resolve_index(self.idx_list, _index_values(inputs[2:])) if len(inputs) > 2 else self.idx_list
        out = HipArray.empty(x.shape, x.dtype)
        copy_into(x, out)
        shape, strides, offset = V.index_view(out.shape, out.strides, out.offset, idx)
        region = out.view(shape, strides, offset)
        yv = _as_device_value(y, x.dtype)
        if region.size:
            if self.set_instead_of_inc:
                _run(scal.identity, [yv], region)
            else:
                _run(scal.add, [region, yv], region)
        output_storage[0][0] = out


def _shape_operands(pattern, like, first):
    """The inputs after the first `first` ones as a device op takes them: arrays whose extents are read go to the
    device like any array, host scalars stay, and an integer vector that is read for its values (a shape given as
    one vector) stays on the host when it is there - its elements are needed before anything can be launched."""
    vec = V.vector_inputs(pattern)
    return [v if (k + first in vec and not isinstance(v.type, HipArrayType)) else _device(v) for k, v in enumerate(like)]


class HipReshape(V.Reshape):
    def make_node(self, x, *like):
        ins = [as_hip_variable(x)] + _shape_operands(self.pattern, like, 1)
        host = V.Reshape.make_node(self, *[V.TensorType(i.type.dtype, i.type.broadcastable)() for i in ins])
        ot = host.outputs[0].type
        return Apply(self, ins, [HipArrayType(ot.dtype, ot.broadcastable)()])

    def perform(self, node, inputs, output_storage):
        x = inputs[0]
        shape = self.resolve([np.shape(v) if not isinstance(v, HipArray) else v.shape for v in inputs], inputs)
        if not x.c_contiguous:
            flat = HipArray.empty(x.shape, x.dtype)
            copy_into(x, flat)
            x = flat
        n = x.dtype.itemsize
        strides = []
        for s in reversed(shape):
            strides.append(n)
            n *= max(s, 1)
        output_storage[0][0] = x.view(shape, tuple(reversed(strides)))


class HipAlloc(V.Alloc):
    def make_node(self, value, *like):
        ins = [_device(value)] + _shape_operands(self.pattern, like, 1)
        host = V.Alloc.make_node(self, *[V.TensorType(i.type.dtype, i.type.broadcastable)() for i in ins])
        ot = host.outputs[0].type
        return Apply(self, ins, [HipArrayType(ot.dtype, ot.broadcastable)()])

    def perform(self, node, inputs, output_storage):
        v = inputs[0]
        shape = self.resolve([np.shape(i) if not isinstance(i, HipArray) else i.shape for i in inputs], inputs)
        dtype = np.dtype(node.outputs[0].type.dtype)
        vs = v.shape if isinstance(v, HipArray) else np.shape(v)
        for a, b in zip(reversed(vs), reversed(shape)):
            if a != b and a != 1:
                raise ValueError("Alloc: value of shape %s cannot be broadcast to %s" % (tuple(vs), shape))
        out = HipArray.empty(shape, dtype)
        if out.size:
            _run(scal.identity, [_as_device_value(v, dtype)], out)
        output_storage[0][0] = out


class HipJoin(V.Join):
    def make_node(self, *tensors):
        ts = [as_hip_variable(t) for t in tensors]
        host = V.Join.make_node(self, *[V.TensorType(t.type.dtype, t.type.broadcastable)() for t in ts])
        if any(i.type.dtype != host.outputs[0].type.dtype for i in host.inputs):
            raise TypeError("HipJoin inputs must share one dtype")
        ot = host.outputs[0].type
        return Apply(self, ts, [HipArrayType(ot.dtype, ot.broadcastable)()])

    def perform(self, node, inputs, output_storage):
        ax = self.axis
        first = inputs[0].shape
        total = 0
        for k, t in enumerate(inputs):
            if t.ndim != len(first) or any(a != b for d, (a, b) in enumerate(zip(t.shape, first)) if d != ax):
                raise ValueError("Join: input %d has shape %s, expected %s except along axis %d" %
                                 (k, t.shape, first, ax))
            total += t.shape[ax]
        shape = first[:ax] + (total,) + first[ax + 1:]
        out = HipArray.empty(shape, inputs[0].dtype)
        at = 0
        for t in inputs:
            part = out.view(t.shape, out.strides, out.offset + at * out.strides[ax])
            copy_into(t, part)
            at += t.shape[ax]
        output_storage[0][0] = out


class HipJoinPart(V.JoinPart):
    def make_node(self, g, *tensors):
        g = as_hip_variable(g)
        ts = [_device(t) for t in tensors]
        return Apply(self, [g] + ts, [HipArrayType(g.type.dtype, ts[self.k].type.broadcastable)()])

    def perform(self, node, inputs, output_storage):
        g, parts = inputs[0], inputs[1:]
        ax = self.axis
        at = sum(p.shape[ax] for p in parts[:self.k])
        shape = parts[self.k].shape
        if g.shape[ax] != sum(p.shape[ax] for p in parts):
            raise ValueError("JoinPart: the joined extent %d does not match the parts" % g.shape[ax])
        output_storage[0][0] = g.view(shape, g.strides, g.offset + at * g.strides[ax])


LIFT = {V.Subtensor: lambda op: HipSubtensor(op.idx_list),
        V.IncSubtensor: lambda op: HipIncSubtensor(op.idx_list, op.set_instead_of_inc),
        V.Reshape: lambda op: HipReshape(op.pattern),
        V.Alloc: lambda op: HipAlloc(op.pattern),
        V.Join: lambda op: HipJoin(op.axis),
        V.JoinPart: lambda op: HipJoinPart(op.axis, op.k),
        V.Rebroadcast: lambda op: HipRebroadcast(op.axis)}
DEVICE_OPS = (HipSubtensor, HipIncSubtensor, HipReshape, HipAlloc, HipJoin, HipJoinPart, HipRebroadcast)
