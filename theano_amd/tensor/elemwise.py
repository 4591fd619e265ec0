"""DimShuffle, Elemwise and the CAReduce family at graph level.

Mirrors ``theano/tensor/elemwise.py``: ``DimShuffle`` :53-306, ``Elemwise``
:338-858 (``get_output_info`` :417-472, ``L_op``/``_bgrad`` :540-645,
``infer_shape`` :827-858), ``CAReduce`` :1180-1382, ``All`` :1587, ``Any``
:1618, ``CAReduceDtype`` :1649-1815 (dtype tables :1721-1780), ``Sum`` :1818,
``Prod`` :1905.  These classes define graphs only; they are executed after
being lifted onto the HIP ops of ``theano_amd.hip``, which subclass them.
"""
from copy import copy

import numpy as np

from .. import scalar as scal
from ..config import config
from ..gof import Apply, Op
from ..scalar import DisconnectedType, Scalar
from .type import TensorType, as_tensor_variable, constant


def _no_host_execution(op):
    raise NotImplementedError(
        "%s has no host implementation: compile the graph with theano_amd.function(), which lifts it onto the "
        "HIP ops" % (op,))


class DimShuffle(Op):
    """Permute dimensions, drop broadcastable ones, insert new ('x') ones.
    Always a view of its input."""

    __props__ = ("input_broadcastable", "new_order")

    def __init__(self, input_broadcastable, new_order, inplace=True):
        if inplace is not True:
            raise ValueError("DimShuffle is inplace by default and hence the inplace for DimShuffle must be true")
        self.input_broadcastable = tuple(bool(b) for b in input_broadcastable)
        self.new_order = tuple(new_order)
        self.inplace = True
        for i, j in enumerate(self.new_order):
            if j != "x":
                if not isinstance(j, (int, np.integer)):
                    raise TypeError("DimShuffle indices must be python ints. Got: '%s' of type '%s'." % (j, type(j)))
                if j >= len(self.input_broadcastable) or j < 0:
                    raise ValueError("new_order[%d] is %d, but the input only has %d axes." %
                                     (i, j, len(self.input_broadcastable)))
                if j in self.new_order[(i + 1):]:
                    raise ValueError("The same input dimension may not appear twice in the list of output dimensions",
                                     self.new_order)
        self.new_order = tuple(j if j == "x" else int(j) for j in self.new_order)
        self.drop = []
        for i, b in enumerate(self.input_broadcastable):
            if i not in self.new_order:
                if b:
                    self.drop.append(i)
                else:
                    raise ValueError("You cannot drop a non-broadcastable dimension.",
                                     (self.input_broadcastable, self.new_order))
        self.shuffle = [x for x in self.new_order if x != "x"]
        self.augment = [i for i, x in enumerate(self.new_order) if x == "x"]
        self.view_map = {0: [0]}

    def make_node(self, input):
        input = as_tensor_variable(input)
        ib = tuple(input.type.broadcastable)
        if ib != self.input_broadcastable:
            if len(ib) != len(self.input_broadcastable):
                raise TypeError("The number of dimensions of the input is incorrect for this op. Expected %s, got %s."
                                % (self.input_broadcastable, ib))
            for expected, b in zip(self.input_broadcastable, ib):
                if expected is True and b is False:
                    raise TypeError("The broadcastable pattern of the input is incorrect for this op. Expected %s, "
                                    "got %s." % (self.input_broadcastable, ib))
        ob = [True if v == "x" else ib[v] for v in self.new_order]
        return Apply(self, [input], [TensorType(input.type.dtype, ob)()])

    def __str__(self):
        return "DimShuffle{%s}" % ",".join(str(x) for x in self.new_order)

    def perform(self, node, inputs, output_storage):
        # a host array is only re-viewed, never computed on
        (x,) = inputs
        if not isinstance(x, np.ndarray):
            raise TypeError("DimShuffle.perform takes a host ndarray; device arrays go through HipDimShuffle")
        res = x.transpose(self.shuffle + self.drop) if x.ndim else x
        shape = list(res.shape[:len(self.shuffle)])
        for augm in self.augment:
            shape.insert(augm, 1)
        output_storage[0][0] = res.reshape(shape)

    def infer_shape(self, node, shapes):
        (ishp,) = shapes
        rval = [ishp[i] for i in self.shuffle]
        for augm in self.augment:
            rval.insert(augm, 1)
        return [rval]

    def R_op(self, inputs, eval_points):
        if None in eval_points:
            return [None]
        return [self(*eval_points)]

    def grad(self, inp, grads):
        (x,) = inp
        (gz,) = grads
        gz = as_tensor_variable(gz)
        grad_order = ["x"] * len(x.type.broadcastable)
        for i, v in enumerate(self.new_order):
            if v != "x":
                grad_order[v] = i
        if x.type.dtype in scal.discrete_dtypes:
            return [x.zeros_like(dtype=config.floatX)]
        return [DimShuffle(gz.type.broadcastable, grad_order)(Elemwise(scal.identity)(gz))]


class Elemwise(Op):
    """Apply a ScalarOp to every element of its (broadcast) tensor inputs."""

    __props__ = ("scalar_op", "inplace_pattern")

    def __init__(self, scalar_op, inplace_pattern=None, name=None, nfunc_spec=None, openmp=None):
        # nfunc_spec names the NumPy function the reference's host ``perform`` may call and ``openmp`` switches its C
        # loop's pragma (theano/tensor/elemwise.py:389-414): neither changes what is computed; the first is kept
        self.name = name
        self.nfunc_spec = nfunc_spec if nfunc_spec is not None else getattr(scalar_op, "nfunc_spec", None)
        self.scalar_op = scalar_op
        self.inplace_pattern = tuple(sorted((inplace_pattern or {}).items())) if not isinstance(
            inplace_pattern, tuple) else inplace_pattern
        self.destroy_map = dict((o, [i]) for o, i in self.inplace_pattern)
        self.nout = getattr(scalar_op, "nout", 1)

    def __str__(self):
        if self.name:
            return self.name
        if self.inplace_pattern:
            return "%s{%s}%s" % (type(self).__name__, self.scalar_op, dict(self.inplace_pattern))
        return "%s{%s}" % (type(self).__name__, self.scalar_op)

    def get_output_info(self, dim_shuffle, *inputs):
        """Output dtypes, broadcast patterns and the rank-aligned inputs."""
        shadow = self.scalar_op.make_node(*[Scalar(i.type.dtype)() for i in inputs])
        target = max(i.type.ndim for i in inputs)
        args = []
        for i in inputs:
            diff = target - i.type.ndim
            if diff:
                i = dim_shuffle(i.type.broadcastable, ["x"] * diff + list(range(i.type.ndim)))(i)
            args.append(i)
        inputs = args
        out_b = [[all(b) for b in zip(*[i.type.broadcastable for i in inputs])]] * len(shadow.outputs)
        for overwriter, overwritten in self.inplace_pattern:
            for ob, ib in zip(out_b[overwriter], inputs[overwritten].type.broadcastable):
                if ib and not ob:
                    raise ValueError("Operation cannot be done inplace on an input with broadcasted dimensions.")
        out_dtypes = [o.type.dtype for o in shadow.outputs]
        if any(inputs[i].type.dtype != out_dtypes[o] for o, i in self.inplace_pattern):
            raise TypeError("Cannot do an inplace operation on incompatible data types.",
                            ([i.type.dtype for i in inputs], out_dtypes, self.inplace_pattern))
        return out_dtypes, out_b, inputs

    def make_node(self, *inputs):
        inputs = [as_tensor_variable(i) for i in inputs]
        out_dtypes, out_b, inputs = self.get_output_info(DimShuffle, *inputs)
        outputs = [TensorType(dt, b)() for dt, b in zip(out_dtypes, out_b)]
        return Apply(self, inputs, outputs)

    def perform(self, node, inputs, output_storage):
        _no_host_execution(self)

    def infer_shape(self, node, i_shapes):
        rval = []
        for o in node.outputs:
            oshp = []
            for dim, b in enumerate(o.type.broadcastable):
                if b:
                    oshp.append(1)
                    continue
                for ishp, i in zip(i_shapes, node.inputs):
                    if not i.type.broadcastable[dim]:
                        oshp.append(ishp[dim])
                        break
            rval.append(tuple(oshp))
        return rval

    def connection_pattern(self, node):
        if hasattr(self.scalar_op, "connection_pattern"):
            try:
                return self.scalar_op.connection_pattern(node)
            except TypeError:
                pass
        return [[True] * len(node.outputs) for _ in node.inputs]

    def R_op(self, inputs, eval_points):
        """Sum over the inputs of d out / d input times that input's evaluation
        point (``theano/tensor/elemwise.py:499-531``); inputs without a
        gradient count as zero."""
        from . import basic
        outs = self.make_node(*inputs).outputs
        rval = []
        for idx, out in enumerate(outs):
            ograds = [basic.zeros_like(o) for o in outs]
            ograds[idx] = basic.ones_like(out)
            bgrads = self._bgrad(inputs, outs, ograds)
            acc = None
            for g, pt in zip(bgrads, eval_points):
                if g is None or isinstance(g.type, DisconnectedType) or pt is None:
                    continue
                term = basic.mul(g, pt)
                acc = term if acc is None else basic.add(acc, term)
            rval.append(acc)
        return rval

    def L_op(self, inputs, outs, ograds):
        rval = self._bgrad(inputs, outs, ograds)
        if any(o.type.dtype not in scal.continuous_dtypes for o in outs):
            new = []
            for elem, ipt in zip(rval, inputs):
                if isinstance(elem.type, DisconnectedType) or not hasattr(elem.type, "dtype"):
                    new.append(elem)
                else:
                    z = ipt.zeros_like()
                    if z.type.dtype not in scal.continuous_dtypes:
                        z = z.astype(config.floatX)
                    new.append(z)
            return new
        from . import basic
        for i, ipt in enumerate(inputs):
            if rval[i] is None or isinstance(rval[i].type, DisconnectedType) or not hasattr(rval[i].type, "dtype"):
                continue
            to_sum = [j for j, b in enumerate(ipt.type.broadcastable) if b and not outs[0].type.broadcastable[j]]
            if to_sum:
                rval[i] = basic.sum(rval[i], axis=to_sum, keepdims=True)
        return rval

    def _bgrad(self, inputs, outputs, ograds):
        """Gradient w.r.t. the broadcast inputs: take the scalar op's symbolic
        gradient and rebuild it as a graph of Elemwise nodes."""
        def passes_through(t):
            return isinstance(t.type, DisconnectedType) or not hasattr(t.type, "dtype")    # no value behind it

        def as_scalar(t):
            if passes_through(t):
                return t
            return Scalar(t.type.dtype)()

        scalar_inputs = [as_scalar(i) for i in inputs]
        scalar_ograds = [as_scalar(g) for g in ograds]
        scalar_outputs = self.scalar_op.make_node(*[Scalar(i.type.dtype)() for i in inputs]).outputs
        scalar_igrads = self.scalar_op.L_op(scalar_inputs, scalar_outputs, scalar_ograds)
        if not isinstance(scalar_igrads, (list, tuple)):
            raise TypeError("%s.grad returned %s instead of list or tuple" % (self.scalar_op, type(scalar_igrads)))
        nd = inputs[0].type.ndim
        memo = {}

        def transform(r):
            if passes_through(r):
                return r
            for group, tgroup in ((scalar_inputs, inputs), (scalar_outputs, outputs), (scalar_ograds, ograds)):
                for s, t in zip(group, tgroup):
                    if r is s:
                        return t
            if id(r) in memo:
                return memo[id(r)]
            node = r.owner
            if node is None:
                res = constant(np.asarray(r.data), dtype=r.type.dtype)
                out = DimShuffle((), ["x"] * nd)(res)
            else:
                out = Elemwise(node.op)(*[transform(i) for i in node.inputs])
            memo[id(r)] = out
            return out

        return [None if g is None else transform(g) for g in scalar_igrads]


class CAReduce(Op):
    """Reduce over ``axis`` with a commutative, associative binary ScalarOp."""

    __props__ = ("scalar_op", "axis")

    def __init__(self, scalar_op, axis=None):
        if scalar_op.nin not in (-1, 2) or scalar_op.nout != 1:
            raise NotImplementedError("CAReduce only supports binary functions with a single output.")
        self.scalar_op = scalar_op
        if axis is None:
            self.axis = None
        elif isinstance(axis, (int, np.integer)):
            self.axis = (int(axis),)
        elif isinstance(axis, np.ndarray) and axis.ndim == 0:
            self.axis = (int(axis),)
        else:
            self.axis = tuple(sorted(set(int(a) for a in axis)))

    def _output_dtype(self, input_dtype):
        return input_dtype

    def _acc_dtype(self, input_dtype):
        return input_dtype

    def make_node(self, input):
        input = as_tensor_variable(input)
        nd = input.type.ndim
        if self.axis is not None:
            for a in self.axis:
                if a >= nd or (a < 0 and abs(a) > nd):
                    raise ValueError("Not enough dimensions on %s to reduce on axis %s" % (input, a))
        axis = self.axis
        if axis is None:
            axis = tuple(range(nd))
        op = self
        if any(a < 0 for a in axis):
            axis = tuple(sorted(set(a + nd if a < 0 else a for a in axis)))
            op = copy(self)
            op.axis = axis
        broadcastable = [b for i, b in enumerate(input.type.broadcastable) if i not in axis]
        output = TensorType(op._output_dtype(input.type.dtype), broadcastable)()
        return Apply(op, [input], [output])

    def __str__(self):
        if self.axis is not None:
            return "Reduce{%s}{%s}" % (self.scalar_op, ", ".join(str(x) for x in self.axis))
        return "Reduce{%s}" % self.scalar_op

    def perform(self, node, inputs, output_storage):
        _no_host_execution(self)

    def infer_shape(self, node, shapes):
        (ishape,) = shapes
        axis = self.axis
        if axis is None:
            return ((),)
        return ([ishape[i] for i in range(node.inputs[0].type.ndim) if i not in axis],)


class All(CAReduce):
    """Logical AND along axes; non-bool inputs are compared with zero first."""

    __props__ = ("axis",)

    def __init__(self, axis=None):
        CAReduce.__init__(self, scal.and_, axis)

    def _props(self):
        return (self.axis,)

    def _output_dtype(self, idtype):
        return "bool"

    def __str__(self):
        return "All" if self.axis is None else "All{%s}" % ", ".join(map(str, self.axis))

    def make_node(self, input):
        input = as_tensor_variable(input)
        if input.type.dtype != "bool":
            from . import basic
            input = basic.neq(input, 0)
        return CAReduce.make_node(self, input)

    def grad(self, inp, grads):
        (x,) = inp
        return [x.zeros_like(config.floatX)]


class Any(CAReduce):
    """Logical OR along axes; non-bool inputs are compared with zero first."""

    __props__ = ("axis",)

    def __init__(self, axis=None):
        CAReduce.__init__(self, scal.or_, axis)

    def _props(self):
        return (self.axis,)

    def _output_dtype(self, idtype):
        return "bool"

    def __str__(self):
        return "Any" if self.axis is None else "Any{%s}" % ", ".join(map(str, self.axis))

    def make_node(self, input):
        input = as_tensor_variable(input)
        if input.type.dtype != "bool":
            from . import basic
            input = basic.neq(input, 0)
        return CAReduce.make_node(self, input)

    def grad(self, inp, grads):
        (x,) = inp
        return [x.zeros_like(config.floatX)]


class CAReduceDtype(CAReduce):
    """CAReduce with an explicit output dtype and accumulator dtype."""

    __props__ = ("scalar_op", "axis", "dtype", "acc_dtype")

    def __init__(self, scalar_op, axis=None, dtype=None, acc_dtype=None):
        CAReduce.__init__(self, scalar_op, axis=axis)
        self.dtype = None if dtype is None else str(np.dtype(dtype)) if dtype != "bool" else "bool"
        self.acc_dtype = None if acc_dtype is None else str(np.dtype(acc_dtype))

    def _output_dtype(self, idtype):
        if self.dtype is None:
            return dict(bool="int64", int8="int64", int16="int64", int32="int64", uint8="uint64", uint16="uint64",
                        uint32="uint64").get(idtype, idtype)
        return self.dtype

    def _acc_dtype(self, idtype):
        acc = self.acc_dtype
        if acc is None:
            return dict(bool="int64", int8="int64", int16="int64", int32="int64", uint8="uint64", uint16="uint64",
                        uint32="uint64", float16="float32", float32="float64", complex64="complex128").get(idtype, idtype)
        if acc in scal.continuous_dtypes and idtype in scal.discrete_dtypes:
            return acc
        up = scal.upcast(idtype, acc)
        if acc != up:
            raise TypeError("Cannot build %s node with input dtype %s and acc_dtype %s, as precision would be lost. "
                            "To correct this error, you can:\n  - not specify acc_dtype, or\n  - use an acc_dtype at "
                            "least as precise as %s.\n  - specify \"dtype\" instead of \"acc_dtype\", so the reduction "
                            "will be precise, but the result will be casted into \"dtype\" at the end.\nIf you are "
                            "expecting the precision loss, you can use tensor.cast(..., dtype=\"%s\"), on your input."
                            % (self, idtype, acc, up, acc))
        return acc

    def make_node(self, input):
        input = as_tensor_variable(input)
        dtype = self._output_dtype(input.type.dtype)
        acc_dtype = self._acc_dtype(input.type.dtype)
        if dtype == self.dtype and acc_dtype == self.acc_dtype:
            op = self
        else:
            op = copy(self)
            op.dtype = dtype
            op.acc_dtype = acc_dtype
        return CAReduce.make_node(op, input)

    def __str__(self):
        name = type(self).__name__
        if name == "CAReduceDtype":
            name = "ReduceDtype{%s}" % self.scalar_op
        axis = ""
        if self.axis is not None:
            axis = "axis=[%s], " % ", ".join(str(x) for x in self.axis)
        return "%s{%sacc_dtype=%s}" % (name, axis, self.acc_dtype)


class Sum(CAReduceDtype):
    __props__ = ("axis", "dtype", "acc_dtype")

    def __init__(self, axis=None, dtype=None, acc_dtype=None):
        CAReduceDtype.__init__(self, scal.add, axis=axis, dtype=dtype, acc_dtype=acc_dtype)

    def _props(self):
        return (self.axis, self.dtype, self.acc_dtype)

    def L_op(self, inp, out, grads):
        (x,) = inp
        if out[0].type.dtype not in scal.continuous_dtypes:
            return [x.zeros_like(dtype=config.floatX)]
        gz = as_tensor_variable(grads[0])
        axis = self.axis
        if axis is None:
            axis = tuple(range(x.type.ndim))
        if axis == ():
            return [gz]
        new_dims, i = [], 0
        for j in range(x.type.ndim):
            if j in axis:
                new_dims.append("x")
            else:
                new_dims.append(i)
                i += 1
        gx = Elemwise(scal.second)(x, DimShuffle(gz.type.broadcastable, new_dims)(gz))
        return [gx]

    def R_op(self, inputs, eval_points):
        if None in eval_points:
            return [None]
        return [self(*eval_points)]


class Prod(CAReduceDtype):
    """Product along axes (``theano/tensor/elemwise.py:1905-2051``).  The
    gradient divides the product by each element where a group holds no zero,
    takes the product of the other elements (ProdWithoutZeros) where it holds
    exactly one, and is zero where it holds more; ``no_zeros_in_input`` keeps
    only the first case."""

    __props__ = ("axis", "dtype", "acc_dtype")

    def __init__(self, axis=None, dtype=None, acc_dtype=None, no_zeros_in_input=False):
        CAReduceDtype.__init__(self, scal.mul, axis=axis, dtype=dtype, acc_dtype=acc_dtype)
        self.no_zeros_in_input = no_zeros_in_input

    def _props(self):
        return (self.axis, self.dtype, self.acc_dtype)

    def L_op(self, inp, out, grads):
        (x,) = inp
        if out[0].type.dtype in scal.discrete_dtypes or self.acc_dtype in scal.discrete_dtypes:
            return [x.zeros_like(dtype=config.floatX)]
        gz = as_tensor_variable(grads[0])
        axis = self.axis
        if axis is None:
            axis = tuple(range(x.type.ndim))
        if axis == ():
            return [gz]
        new_dims, i = [], 0
        for j in range(x.type.ndim):
            if j in axis:
                new_dims.append("x")
            else:
                new_dims.append(i)
                i += 1

        def over_groups(v):
            return DimShuffle(v.type.broadcastable, new_dims)(v)

        from . import basic as T
        prod_out = over_groups(out[0])
        gz = over_groups(gz)
        without_zeros = T.true_div(T.mul(gz, prod_out), x)
        if self.no_zeros_in_input:
            return [without_zeros]
        where_zeros = T.eq(x, 0.0)
        n_zeros = T.sum(where_zeros, axis=self.axis)
        single_zero = over_groups(T.eq(n_zeros, 1))
        where_single_zero = T.mul(single_zero, where_zeros)
        # only groups with one zero and a non-zero incoming gradient keep their values
        taken = T.mul(T.mul(single_zero, T.neq(gz, 0.0)), x)
        others = over_groups(ProdWithoutZeros(axis=self.axis)(taken))
        no_zero = over_groups(T.eq(n_zeros, 0))
        return [T.switch(no_zero, without_zeros, T.mul(T.switch(where_single_zero, others, 0.0), gz))]


# the scalar op behind ProdWithoutZeros lives here in the reference (theano/tensor/elemwise.py:2054-2083)
MulWithoutZeros, mul_without_zeros = scal.MulWithoutZeros, scal.mul_without_zeros


class ProdWithoutZeros(CAReduceDtype):
    """Product of the non-zero elements along axes; 0 for a group of zeros
    (``theano/tensor/elemwise.py:2086-2101``)."""

    __props__ = ("axis", "dtype", "acc_dtype")

    def __init__(self, axis=None, dtype=None, acc_dtype=None):
        CAReduceDtype.__init__(self, scal.mul_without_zeros, axis=axis, dtype=dtype, acc_dtype=acc_dtype)

    def _props(self):
        return (self.axis, self.dtype, self.acc_dtype)

    def grad(self, inp, grads):
        raise NotImplementedError("second derivatives of prod(a) are not supported; if a holds no zeros use "
                                  "prod(a, no_zeros_in_input=True)")
