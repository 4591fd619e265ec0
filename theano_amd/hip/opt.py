"""Graph rewrites that move a graph onto the HIP ops and fuse it.

Order: lift every Elemwise / DimShuffle / CAReduce node onto the device ops
(the job of ``GraphToGPU`` with ``local_gpua_elemwise``, ``local_gpua_dimshuffle``
and ``local_gpua_careduce``, ``theano/gpuarray/opt.py:325-478, 740-866,
1194-1286``), fuse chains of elementwise nodes into one ``Composite``
(``local_elemwise_fusion_op``, ``theano/tensor/opt.py:7071-7313``, registered for
the GPU op at ``theano/gpuarray/opt.py:842-851``), then fold elementwise
producers into the reductions that consume them (generalising
``local_gpu_elemwise_careduce``, ``theano/gpuarray/opt.py:2405-2428``) and merge
sibling reductions that read the same data.
"""
import numpy as np

from .. import gof
from .. import scalar as scal
from ..config import config
from ..gof import Constant
from ..tensor import basic as T
from ..tensor.elemwise import All, Any, CAReduce, CAReduceDtype, DimShuffle, Elemwise
from ..tensor.type import TensorConstant, TensorType
from . import views as hip_views
from .ops import (HipArrayType, HipCAReduce, HipDimShuffle, HipElemwise, HipElemwiseReduce, HipMaxAndArgmax, HipToHost,
                  HostToHip,
                  _is_host_scalar, as_hip_variable, hip_from_host, host_from_hip)


class DeviceConstant(Constant):
    """A non-scalar constant uploaded once when the function is compiled."""

    def signature(self):
        return (self.type, id(self.data))


HipArrayType.Constant = DeviceConstant


def _lift_reduce(node, x):
    op = node.op
    idt = x.type.dtype
    if isinstance(op, CAReduceDtype):
        acc, out = op._acc_dtype(idt), op._output_dtype(idt)
    else:
        acc, out = idt, op._output_dtype(idt)
        if isinstance(op, (All, Any)):
            acc = "bool"
    if acc == "float16" and not isinstance(op.scalar_op, (scal.Maximum, scal.Minimum)):
        # max / min are exact in any precision; a float16 running sum or product has no reference C code
        raise NotImplementedError("float16 accumulators are not supported (as theano/tensor/elemwise.py:1395-1398)")
    return HipCAReduce((op.scalar_op,), op.axis if op.axis is not None else tuple(range(x.type.ndim)),
                       (acc,), (out,))(x)


def _shape_vector_inputs(fgraph):
    """Function inputs that every client reads as a whole shape vector on the host (``reshape(x, v, ndim=n)``):
    they are never copied to the device."""
    from ..tensor import views as V
    keep = set()
    for i in fgraph.inputs:
        if not isinstance(i.type, TensorType) or i.type.ndim != 1 or i.type.dtype not in scal.discrete_dtypes:
            continue
        clients = fgraph.clients.get(i, []) if hasattr(fgraph, "clients") else []
        uses = [(node, k) for node, k in clients if node != "output"]
        if uses and len(uses) == len(clients) and all(
                isinstance(node.op, (V.Reshape, V.Alloc)) and k in V.vector_inputs(node.op.pattern) and k > 0
                for node, k in uses):
            keep.add(i)
    return keep


def lift_to_hip(fgraph):
    """Return a new FunctionGraph computing the same outputs with device ops.
    Raises NotImplementedError for an op with no device counterpart: there is
    no host execution to fall back to."""
    mapping = {}
    shape_vectors = _shape_vector_inputs(fgraph)
    for i in fgraph.inputs:
        if isinstance(i.type, TensorType) and not _is_host_scalar(i) and i not in shape_vectors:
            mapping[i] = hip_from_host(i)
        else:
            mapping[i] = i

    def mapped(v):
        if v in mapping:
            return mapping[v]
        if isinstance(v, Constant):
            if isinstance(v.type, TensorType) and not _is_host_scalar(v):
                mapping[v] = DeviceConstant(HipArrayType(v.type.dtype, v.type.broadcastable), v.data, name=v.name)
            else:
                mapping[v] = v
            return mapping[v]
        if v.owner is None and hasattr(v, "container"):  # a shared variable
            mapping[v] = v
            return v
        raise gof.InconsistencyError("variable %s is not computed from the function inputs" % v)

    for node in fgraph.toposort():
        ins = [mapped(i) for i in node.inputs]
        op = node.op
        if isinstance(op, (HipElemwise, HipCAReduce, HipMaxAndArgmax, HipDimShuffle, HostToHip, HipToHost, T.ShapeFloat) +
                      hip_views.DEVICE_OPS):
            if isinstance(op, HostToHip) and isinstance(ins[0].type, HipArrayType):
                outs = [ins[0]]
            elif isinstance(op, HipToHost):
                # transfers inside the graph are cut (theano/gpuarray/opt.py:566-737): every lifted
                # consumer takes the device value, and results go back to the host at the outputs
                outs = [ins[0]]
            else:
                outs = op.make_node(*ins).outputs
        elif isinstance(op, Elemwise):
            outs = HipElemwise(op.scalar_op, op.inplace_pattern).make_node(*ins).outputs
        elif isinstance(op, DimShuffle):
            if isinstance(ins[0].type, HipArrayType):
                outs = HipDimShuffle(op.input_broadcastable, op.new_order).make_node(ins[0]).outputs
            else:
                outs = op.make_node(ins[0]).outputs  # host scalar: a view on the host
        elif isinstance(op, CAReduce):
            x = ins[0]
            if not isinstance(x.type, HipArrayType):
                x = as_hip_variable(x)
            outs = [_lift_reduce(node, x)]
        elif isinstance(op, T.MaxAndArgmax):
            outs = HipMaxAndArgmax(op.axis).make_node(ins[0]).outputs
        elif type(op) in hip_views.LIFT:
            outs = hip_views.LIFT[type(op)](op).make_node(*ins).outputs

        else:
            raise NotImplementedError("%s has no HIP implementation and nothing runs on the host" % op)
        for o, no in zip(node.outputs, outs):
            mapping[o] = no
    new_outputs = []
    for o in fgraph.outputs:
        m = mapped(o)
        want_device = isinstance(o.type, HipArrayType)
        if isinstance(m.type, HipArrayType) and not want_device:
            m = host_from_hip(m)
        elif isinstance(m.type, TensorType) and want_device:
            m = hip_from_host(m)
        new_outputs.append(m)
    return fgraph.rebuild(new_outputs)


# --------------------------------------------------------------------------
def _scalar_constant(var):
    """The scalar Constant standing for an all-broadcastable tensor constant."""
    if isinstance(var, TensorConstant) and all(var.type.broadcastable):
        return scal.ScalarConstant(scal.Scalar(var.type.dtype), np.asarray(var.data).reshape(())[()])
    return None


_TRIVIAL_OPS = (scal.Cast, scal.Add, scal.Sub, scal.Mul, scal.Neg, scal.Sqr, scal.Abs, scal.Sgn, scal.Identity,
              scal.Second, scal.LogicalComparison, scal.Switch, scal.BinaryBitOp, scal.Invert, scal.Maximum,
              scal.Minimum, scal.Clip, scal.IsNan, scal.IsInf)
# float32 division compiles to a few instructions (2.5-ulp form): cheap enough to recompute once per
# consumer of a same-shaped value, not cheap enough to redo per element for a broadcast operand
_CHEAP_OPS = _TRIVIAL_OPS + (scal.TrueDiv, scal.Inv)


# one hardware transcendental plus a few multiplies: worth redoing once per consumer kernel when that saves
# writing a full-size array and reading it back, never per element of a broadcast
_TRANSCENDENTAL_OPS = tuple(type(o) for o in (scal.exp, scal.exp2, scal.expm1, scal.log, scal.log2, scal.log10,
                                              scal.log1p, scal.sqrt, scal.tanh)) + (scal.ScalarSigmoid,)


def _cheap(scalar_op, ops=None, transcendentals=0):
    """True when recomputing the op per consumer costs a few ALU instructions (at most
    ``transcendentals`` calls of exp / log / sqrt / tanh / sigmoid among them)."""
    ops = ops or _CHEAP_OPS
    sops = ([n.op for n in gof.io_toposort(scalar_op.inputs, scalar_op.outputs)]
            if isinstance(scalar_op, scal.Composite) else [scalar_op])
    heavy = [o for o in sops if not isinstance(o, ops)]
    return len(heavy) <= transcendentals and all(isinstance(o, _TRANSCENDENTAL_OPS) for o in heavy)


def _absorbs(client, var):
    """Can this consumer take the producer of ``var`` into its own kernel?"""
    if client == "output":
        return False
    op = client.op
    if isinstance(op, HipElemwise):
        return (not op.inplace_pattern and
                tuple(client.outputs[0].type.broadcastable) == tuple(var.type.broadcastable))
    if isinstance(op, HipCAReduce):
        return op.post_scalar_op is None and all(
            i.type.ndim == var.type.ndim for i in client.inputs if isinstance(i.type, HipArrayType))
    return False


def _duplicable(fgraph, var):
    """A cheap elementwise result used by several kernels is recomputed inside
    each of them when that moves fewer bytes than writing it once and reading
    it back: inputs x consumers <= inputs + output x (1 + consumers)."""
    node = var.owner
    clients = fgraph.clients.get(var, [])
    if len(clients) < 2 or len(clients) > 8:
        return False
    # The gradient of max / min (and what users write with argmax) compares the reduction's result with
    # its operand for equality: both kernels must see the very same floating-point values, which two
    # compilations of one expression do not promise (contraction into fused multiply-adds depends on the
    # surrounding code).  Such an operand is stored once and read back.
    if var.type.dtype in scal.continuous_dtypes and any(
            c != "output" and (isinstance(c.op, HipMaxAndArgmax) or (isinstance(c.op, HipCAReduce) and any(
                isinstance(o, (scal.Maximum, scal.Minimum)) for o in c.op.scalar_ops))) for c, _ in clients):
        return False
    # exp(x - m) read by a sum and by a division is worth two evaluations (the sum's kernel never writes
    # it); among elementwise consumers only, the sibling merge computes it once in one kernel anyway
    def full_size_operand_of(c):
        if c == "output" or not isinstance(c.op, HipCAReduce):
            return False
        arrays = [i.type.broadcastable for i in c.inputs[:len(c.inputs) - c.op.n_extra] if isinstance(i.type, HipArrayType)]
        return tuple(var.type.broadcastable) == tuple(all(bs) for bs in zip(*arrays))

    feeds_reduction = any(full_size_operand_of(c) for c, _ in clients)   # per element of a broadcast: never
    if not _cheap(node.op.scalar_op, transcendentals=config.duplicate_transcendentals if feeds_reduction else 0):
        return False
    if not all(_absorbs(c, var) for c, _ in clients):
        return False
    out_b = var.type.broadcastable
    in_bytes = sum(np.dtype(i.type.dtype).itemsize for i in node.inputs
                   if isinstance(i.type, HipArrayType) and tuple(i.type.broadcastable) == tuple(out_b))
    out_bytes = np.dtype(var.type.dtype).itemsize
    n = len(set(id(c) for c, _ in clients))
    return in_bytes * n <= in_bytes + out_bytes * (1 + n)


def _fusable(fgraph, var, out_bcast):
    node = var.owner
    if (node is None or not isinstance(node.op, HipElemwise) or len(node.outputs) != 1 or node.op.inplace_pattern or
            len(var.type.broadcastable) != len(out_bcast)):
        return False
    if tuple(var.type.broadcastable) == tuple(out_bcast):
        return fgraph.n_clients(var) == 1 or _duplicable(fgraph, var)
    # a producer that is broadcast against the consumer (a per-channel cast, say) is recomputed per
    # element only when that costs next to nothing; the reference keeps such nodes apart
    # (theano/tensor/opt.py:7171-7175) because its C loops would redo real work
    return (fgraph.n_clients(var) == 1 and _cheap(node.op.scalar_op, _TRIVIAL_OPS) and
            all(pb or not cb for pb, cb in zip(var.type.broadcastable, out_bcast)))


def _fuse_node(fgraph, node):
    """Splice single-client elementwise producers of ``node`` into it
    (acceptance rule of ``theano/tensor/opt.py:7168-7218``)."""
    if not isinstance(node.op, HipElemwise) or node.op.inplace_pattern:
        return None
    out = node.outputs[0]               # the results of one node share a broadcast pattern
    inputs, s_inputs = [], []

    def scalar_for(v):
        for t, s in zip(inputs, s_inputs):
            if t is v:
                return s
        s = scal.Scalar(v.type.dtype)()
        inputs.append(v)
        s_inputs.append(s)
        return s

    def arg_for(v):
        c = _scalar_constant(v)
        return c if c is not None else scalar_for(v)

    s_args, fused = [], False
    for i in node.inputs:
        if _fusable(fgraph, i, out.type.broadcastable):
            p = i.owner
            before = len(inputs)
            args = [arg_for(j) for j in p.inputs]
            if len(inputs) > config.max_fused_inputs:
                del inputs[before:], s_inputs[before:]
                s_args.append(scalar_for(i))
                continue
            s_args.append(p.op.scalar_op(*args))
            fused = True
        else:
            c = _scalar_constant(i)
            if c is not None:
                s_args.append(c)
                fused = True
            else:
                s_args.append(scalar_for(i))
    if not fused or not inputs or len(inputs) > max(config.max_fused_inputs, len(node.inputs)):
        return None
    s_outs = node.op.scalar_op(*s_args, return_list=True)
    if [s.type.dtype for s in s_outs] != [o.type.dtype for o in node.outputs]:
        return None
    comp = scal.Composite(s_inputs, s_outs)
    new_outs = HipElemwise(comp).make_node(*inputs).outputs
    if [n.type for n in new_outs] != [o.type for o in node.outputs]:
        return None
    return new_outs


def fuse_elemwise(fgraph):
    """Apply ``_fuse_node`` from the outputs towards the inputs until the graph
    stops changing (``FusionOptimizer``, ``theano/tensor/opt.py:7328-7386``)."""
    changed = True
    total = 0
    while changed:
        changed = False
        for node in reversed(fgraph.toposort()):
            if node not in fgraph.apply_nodes:
                continue
            new_outs = _fuse_node(fgraph, node)
            if new_outs is not None:
                for o, no in zip(node.outputs, new_outs):
                    fgraph.replace(o, no)
                changed = True
                total += 1
    return total


# --------------------------------------------------------------------------
def _as_composite_inputs(node):
    """Scalar inputs / tensor inputs of an elementwise node with scalar
    constants turned into literals."""
    inputs, s_inputs, args = [], [], []
    for v in node.inputs:
        c = _scalar_constant(v)
        if c is not None:
            args.append(c)
            continue
        for t, s in zip(inputs, s_inputs):
            if t is v:
                args.append(s)
                break
        else:
            s = scal.Scalar(v.type.dtype)()
            inputs.append(v)
            s_inputs.append(s)
            args.append(s)
    return inputs, s_inputs, args


def fuse_reduce_prologue(fgraph):
    """``reduce(f(a, b, ...))`` becomes one reduction whose prologue is f, when
    nothing else needs f's result (or f is cheap enough to recompute)."""
    count = 0
    changed = True
    while changed:
        changed = False
        work = [n for n in fgraph.toposort() if isinstance(n.op, HipCAReduce)]
        work.reverse()
        while work:
            node = work.pop()
            op = node.op
            if not isinstance(op, HipCAReduce) or op.post_scalar_op is not None or node not in fgraph.apply_nodes:
                continue
            nd = max(i.type.ndim for i in node.inputs)
            target = None
            for x in node.inputs:
                p = x.owner
                if (p is None or not isinstance(p.op, HipElemwise) or len(p.outputs) != 1 or p.op.inplace_pattern or
                        x.type.ndim != nd):
                    continue
                if fgraph.n_clients(x) != 1 and not _duplicable(fgraph, x):
                    continue
                if any(isinstance(i.type, HipArrayType) and i.type.ndim != nd for i in p.inputs):
                    continue
                target = x
                break
            if target is None:
                continue
            # new operand list: the node's inputs with `target` replaced by its producer's inputs
            inputs, s_inputs = [], []

            def scalar_for(v):
                for t, sv in zip(inputs, s_inputs):
                    if t is v:
                        return sv
                sv = scal.Scalar(v.type.dtype)()
                inputs.append(v)
                s_inputs.append(sv)
                return sv

            p = target.owner
            p_args = []
            for v in p.inputs:
                c = _scalar_constant(v)
                p_args.append(c if c is not None else scalar_for(v))
            p_out = p.op.scalar_op(*p_args)
            outer_args = [p_out if v is target else scalar_for(v) for v in node.inputs]
            if len(inputs) > config.max_fused_inputs or not inputs:
                continue
            if op.pre_scalar_op is None:
                pre_outs = [outer_args[0]]
            else:
                pre_outs = op.pre_scalar_op(*outer_args, return_list=True)
            pre = scal.Composite(s_inputs, pre_outs)
            new_node = HipCAReduce(op.scalar_ops, op.axis, op.acc_dtypes, op.out_dtypes, pre, None).make_node(*inputs)
            if [o.type for o in new_node.outputs] != [o.type for o in node.outputs]:
                continue
            for o, no in zip(node.outputs, new_node.outputs):
                fgraph.replace(o, no)
            count += 1
            changed = True
            work.append(new_node)       # its new operands may have absorbable producers too
    return count


def fuse_argmax_prologue(fgraph):
    """``max_and_argmax(f(a, b, ...))`` computes f on the fly when nothing else
    reads f's result (``argmin`` is ``argmax(-x)``)."""
    count = 0
    for node in fgraph.toposort():
        op = node.op
        if not isinstance(op, HipMaxAndArgmax) or op.pre_scalar_op is not None or len(node.inputs) != 1:
            continue
        x = node.inputs[0]
        p = x.owner
        if (p is None or not isinstance(p.op, HipElemwise) or len(p.outputs) != 1 or p.op.inplace_pattern or
                fgraph.n_clients(x) != 1):
            continue
        if any(isinstance(i.type, HipArrayType) and i.type.ndim != x.type.ndim for i in p.inputs):
            continue
        inputs, s_inputs, s_args = [], [], []
        for v in p.inputs:
            c = _scalar_constant(v)
            if c is not None:
                s_args.append(c)
                continue
            if v in inputs:
                s_args.append(s_inputs[inputs.index(v)])
                continue
            sv = scal.Scalar(v.type.dtype)()
            inputs.append(v)
            s_inputs.append(sv)
            s_args.append(sv)
        if not inputs or len(inputs) > config.max_fused_inputs:
            continue
        pre = scal.Composite(s_inputs, [p.op.scalar_op(*s_args)])
        new_node = HipMaxAndArgmax(op.axis, pre).make_node(*inputs)
        if [o.type for o in new_node.outputs] != [o.type for o in node.outputs]:
            continue
        for o, no in zip(node.outputs, new_node.outputs):
            fgraph.replace(o, no)
        count += 1
    return count


def fuse_reduce_epilogue(fgraph):
    """``g(reduce(...), ...)`` - the division of a mean, ``sqrt(var + eps)``, the
    per-channel algebra between the two passes of a batch-norm gradient - runs in
    the reduction's own last step instead of a launch of its own; repeated until
    no consumer qualifies, so a chain of such nodes ends up in one epilogue."""
    count = 0
    changed = True
    while changed:
        changed = False
        work = [n for n in fgraph.toposort() if isinstance(n.op, HipCAReduce)]
        work.reverse()
        while work:
            red = work.pop()
            rop = red.op
            if not isinstance(rop, HipCAReduce) or red not in fgraph.apply_nodes:
                continue
            cands = []
            for r in red.outputs:
                for c, _ in fgraph.clients.get(r, []):
                    if c == "output":
                        continue
                    if isinstance(c.op, HipDimShuffle):
                        for c2, _ in fgraph.clients.get(c.outputs[0], []):
                            if c2 != "output" and isinstance(c2.op, HipElemwise) and c2 not in cands:
                                cands.append(c2)
                    elif isinstance(c.op, HipElemwise) and c not in cands:
                        cands.append(c)
            for cand in cands:
                new_red = _try_epilogue(fgraph, red, cand)
                if new_red is not None:
                    count += 1
                    changed = True
                    work.append(new_red)    # the next consumer in the chain
                    break
    return count


def _try_epilogue(fgraph, red, cand):
    """Moves the elementwise node ``cand`` into the epilogue of the reduction
    ``red`` (composing it with an epilogue that is already there); returns the new
    reduction node, or None.  Every array
    input of ``cand`` must be a result of ``red`` (directly or through one and the
    same keepdims DimShuffle), a host scalar, or a device array of the results'
    own shape that does not depend on ``red`` (a per-channel scale, the result
    of an earlier reduction): the epilogue reads that one at the result's index."""
    rop = red.op
    if len(cand.outputs) != 1 or cand.op.inplace_pattern:
        return None
    n_red_in = len(red.inputs) - rop.n_extra
    extras = list(red.inputs[n_red_in:])
    post_in = rop.post_in_dtypes if rop.post_scalar_op is not None else rop.out_dtypes
    s_acc = [scal.Scalar(dt)() for dt in post_in]
    s_extras = [scal.Scalar(e.type.dtype)() for e in extras]
    if rop.post_scalar_op is None:
        cur = list(s_acc)
    else:
        cur = rop.post_scalar_op(*(s_acc + s_extras), return_list=True)
    # the DimShuffle (if any) between the reduction and the consumer
    ds_op, seen_direct = None, False
    for i in cand.inputs:
        if i.owner is not None and isinstance(i.owner.op, HipDimShuffle) and i.owner.inputs[0].owner is red:
            if ds_op is not None and i.owner.op != ds_op:
                return None
            ds_op = i.owner.op
        elif i.owner is red:
            seen_direct = True
    if ds_op is not None and seen_direct:
        return None
    if ds_op is not None:
        # only DimShuffles that insert or drop broadcast dimensions: with a transposition in
        # between, "the result's index" is no longer the consumer's index
        kept_order = [o for o in ds_op.new_order if o != "x"]
        if kept_order != sorted(kept_order):
            return None
        layout = ds_op.make_node(red.outputs[0]).outputs[0].type.broadcastable
    else:
        layout = red.outputs[0].type.broadcastable
    s_args, used = [], set()

    def operand(i, depth):
        """Scalar expression for an input that does not come from ``red``: a constant, a host
        scalar or per-result device array (an extra operand of the epilogue), or a cheap
        elementwise node over such values (a cast of gamma, say), recomputed in the epilogue."""
        c = _scalar_constant(i)
        if c is not None:
            return c
        per_result = (isinstance(i.type, HipArrayType) and tuple(i.type.broadcastable) == tuple(layout) and
                      not _depends_on(i, red))
        if not (_is_host_scalar(i) or per_result):
            return None
        p = i.owner
        if (per_result and p is not None and isinstance(p.op, HipElemwise) and len(p.outputs) == 1 and depth < 4 and
                _cheap(p.op.scalar_op, _TRIVIAL_OPS)):
            args = [operand(v, depth + 1) for v in p.inputs]
            if all(a is not None for a in args):
                return p.op.scalar_op(*args)
        for e, se in zip(extras, s_extras):
            if e is i:
                return se
        sv = scal.Scalar(i.type.dtype)()
        extras.append(i)
        s_extras.append(sv)
        return sv

    for i in cand.inputs:
        src = i.owner.inputs[0] if (ds_op is not None and i.owner is not None and i.owner.op == ds_op and
                                   i.owner.inputs[0].owner is red) else i
        if src.owner is red:
            k = red.outputs.index(src)
            used.add(k)
            s_args.append(cur[k])
            continue
        c = _scalar_constant(i)
        if c is not None:
            s_args.append(c)
            continue
        expr = operand(i, 0)
        if expr is None:
            return None
        s_args.append(expr)
    if not used or len(extras) > 12:
        return None
    e_out = cand.op.scalar_op(*s_args)
    # results something else still needs stay outputs of the new node
    keep = []
    for k, r in enumerate(red.outputs):
        others = False
        for c, _ in fgraph.clients.get(r, []):
            if c == "output":
                others = True
            elif isinstance(c.op, HipDimShuffle) and c.op == ds_op:
                if any(c2 is not cand for c2, _ in fgraph.clients.get(c.outputs[0], [])):
                    others = True
            elif c is not cand:
                others = True
        if others:
            keep.append(k)
    post_outs = [scal.identity(cur[k]) if cur[k] in s_acc else cur[k] for k in keep] + [e_out]
    post = scal.Composite(s_acc + s_extras, post_outs)
    out_dtypes = tuple(rop.out_dtypes[k] for k in keep) + (cand.outputs[0].type.dtype,)
    new_op = HipCAReduce(rop.scalar_ops, rop.axis, rop.acc_dtypes, out_dtypes, rop.pre_scalar_op, post, post_in,
                         len(extras))
    new_node = new_op.make_node(*(list(red.inputs[:n_red_in]) + extras))
    new_e = new_node.outputs[-1]
    if ds_op is not None:
        new_e = HipDimShuffle(ds_op.input_broadcastable, ds_op.new_order)(new_e)
    if new_e.type != cand.outputs[0].type:
        return None
    for j, k in enumerate(keep):
        fgraph.replace(red.outputs[k], new_node.outputs[j])
    fgraph.replace(cand.outputs[0], new_e)
    return new_node


def _depends_on(var, node, limit=10000, pos=None):
    """True when ``var`` is computed (transitively) from an output of ``node``.  ``pos``: for each node the
    span (first, last) of positions in a topological order that it stands for - one position for an original
    node, the span of its parts for a node merged from several; a producer whose parts all lie before every
    part of ``node`` cannot depend on it."""
    if pos is not None and var.owner is not None:
        pv, pn = pos.get(var.owner), pos.get(node)
        if pv is not None and pn is not None and pv[1] < pn[0]:
            return False
    stack, seen = [var], set()
    while stack and len(seen) < limit:
        v = stack.pop()
        if id(v) in seen or v.owner is None:
            continue
        seen.add(id(v))
        if v.owner is node:
            return True
        stack.extend(v.owner.inputs)
    return False


def merge_sibling_reductions(fgraph):
    """Two reductions over the same axes whose inputs have the same full shape
    pattern and share at least one input of that full shape become one
    multi-output reduction, so shared operands are read once (e.g. ``sum(g)`` and
    ``sum(g * xhat)``, or ``any`` and ``all`` of one tensor)."""
    count = 0
    changed = True
    while changed:
        changed = False
        reds = [n for n in fgraph.toposort() if isinstance(n.op, HipCAReduce) and n.op.post_scalar_op is None]
        for ai in range(len(reds)):
            a = reds[ai]
            for b in reds[ai + 1:]:
                if a.op.axis != b.op.axis:
                    continue
                if a.outputs[0].type.broadcastable != b.outputs[0].type.broadcastable:
                    continue
                nd = max(i.type.ndim for i in a.inputs)
                pa = [all(bb) for bb in zip(*[i.type.broadcastable for i in a.inputs if i.type.ndim == nd])]
                pb = [all(bb) for bb in zip(*[i.type.broadcastable for i in b.inputs if i.type.ndim == nd])]
                if pa != pb:
                    continue
                # Equal run-time shapes are certain only when the two share an array that spans the whole
                # reduce domain: a common operand that is broadcast in both (a per-channel weight) says
                # nothing about the extents of the others.
                full_a = set(id(i) for i in a.inputs if isinstance(i.type, HipArrayType) and
                             list(i.type.broadcastable) == pa)
                if not any(id(i) in full_a for i in b.inputs):
                    continue
                if any(_depends_on(i, a) for i in b.inputs) or any(_depends_on(i, b) for i in a.inputs):
                    continue
                merged = _merge_two(a, b)
                if merged is None:
                    continue
                outs = merged.outputs
                ka = len(a.outputs)
                for o, no in zip(a.outputs, outs[:ka]):
                    fgraph.replace(o, no)
                for o, no in zip(b.outputs, outs[ka:]):
                    fgraph.replace(o, no)
                count += 1
                changed = True
                break
            if changed:
                break
    return count


def _merge_two(a, b):
    inputs, s_inputs = [], []

    def scalar_for(v):
        for t, s in zip(inputs, s_inputs):
            if t is v:
                return s
        s = scal.Scalar(v.type.dtype)()
        inputs.append(v)
        s_inputs.append(s)
        return s

    outs = []
    for n in (a, b):
        args = [scalar_for(v) for v in n.inputs]
        if n.op.pre_scalar_op is None:
            outs.extend(scal.identity(x) for x in args)
        else:
            res = n.op.pre_scalar_op(*args, return_list=True)
            outs.extend(res)
    if len(inputs) > config.max_fused_inputs:
        return None
    pre = scal.Composite(s_inputs, outs)
    op = HipCAReduce(a.op.scalar_ops + b.op.scalar_ops, a.op.axis, a.op.acc_dtypes + b.op.acc_dtypes,
                     a.op.out_dtypes + b.op.out_dtypes, pre, None)
    return op.make_node(*inputs)


def share_equal_accumulators(fgraph):
    """A multi-reduction that accumulates one expression twice with the same op - ``sum(x)`` asked for by a
    mean and again by a variance - keeps one accumulator (the wider of two float types) and an epilogue
    that hands it to both results."""
    from .hoist import _unique_accumulators
    count = 0
    for node in fgraph.toposort():
        op = node.op
        if not isinstance(op, HipCAReduce) or op.pre_scalar_op is None or op.post_scalar_op is not None:
            continue
        pre = op.pre_scalar_op
        new_pre, u_ops, u_accs, where = _unique_accumulators(pre.inputs, pre.outputs, op.scalar_ops, op.acc_dtypes)
        if len(u_ops) == len(op.scalar_ops):
            continue
        s_acc = [scal.Scalar(dt)() for dt in u_accs]
        post_outs = []
        for k, dt in enumerate(op.out_dtypes):
            r = scal.cast(s_acc[where[k]], dt)
            post_outs.append(scal.identity(r) if r in s_acc else r)
        new_op = HipCAReduce(tuple(u_ops), op.axis, tuple(u_accs), op.out_dtypes, new_pre, scal.Composite(s_acc, post_outs),
                             tuple(u_accs), 0)
        new_node = new_op.make_node(*node.inputs)
        if [o.type for o in new_node.outputs] != [o.type for o in node.outputs]:
            continue
        for o, no in zip(node.outputs, new_node.outputs):
            fgraph.replace(o, no)
        count += 1
    return count


def merge_sibling_elemwise(fgraph):
    """Two elementwise kernels of one and the same shape become one kernel with several results
    when that saves reading an array again: siblings that read a common array (the two moment
    updates of an Adam step), or a kernel and a consumer of its results that something else
    needs as well (the parameter update that reads both new moments, which are outputs too).
    Equal shapes are certain because both hold an array of exactly the results' broadcast
    pattern in common; apart from the direct use of one's results by the other, neither may
    depend on the other.  The reference's GPU op stops at one output
    (``theano/gpuarray/elemwise.py:114-115``); the kernels here take several."""
    count = 0
    order = fgraph.toposort()
    pos = dict((n, (k, k)) for k, n in enumerate(order))
    nodes = [n for n in order if isinstance(n.op, HipElemwise) and not n.op.inplace_pattern]
    for ai in range(len(nodes)):
        a = nodes[ai]
        if a not in fgraph.apply_nodes:
            continue
        pa = tuple(a.outputs[0].type.broadcastable)
        if all(pa):
            continue
        for bi in range(ai + 1, len(nodes)):
            b = nodes[bi]
            if b not in fgraph.apply_nodes or tuple(b.outputs[0].type.broadcastable) != pa:
                continue
            full_a = set(id(i) for i in a.inputs if isinstance(i.type, HipArrayType) and
                         tuple(i.type.broadcastable) == pa)
            full_a.update(id(o) for o in a.outputs)
            if not any(id(i) in full_a for i in b.inputs):
                continue
            if any(i.owner is not a and _depends_on(i, a, pos=pos) for i in b.inputs):
                continue
            if any(_depends_on(i, b, pos=pos) for i in a.inputs):
                continue
            inputs, s_inputs = [], []

            def scalar_for(v):
                for t, sv in zip(inputs, s_inputs):
                    if t is v:
                        return sv
                sv = scal.Scalar(v.type.dtype)()
                inputs.append(v)
                s_inputs.append(sv)
                return sv

            a_souts = a.op.scalar_op(*[scalar_for(v) for v in a.inputs], return_list=True)
            b_args = [a_souts[a.outputs.index(v)] if v.owner is a else scalar_for(v) for v in b.inputs]
            b_souts = b.op.scalar_op(*b_args, return_list=True)
            # results of the first kernel that only the second one read stay inside
            keep = [k for k, o in enumerate(a.outputs)
                    if any(c is not b for c, _ in fgraph.clients.get(o, []))]
            olds = [a.outputs[k] for k in keep] + list(b.outputs)
            if len(inputs) > config.max_fused_inputs or len(olds) > 8:
                continue
            # an array that is both read and produced here would be an output equal to an input
            s_outs = [a_souts[k] for k in keep] + b_souts
            if any(so in s_inputs for so in s_outs):
                continue
            merged = HipElemwise(scal.Composite(s_inputs, s_outs)).make_node(*inputs)
            if [o.type for o in merged.outputs] != [o.type for o in olds]:
                continue
            for o, no in zip(olds, merged.outputs):
                fgraph.replace(o, no)
            count += 1
            # the merged node stands for both spans: what lies between its parts may depend on the first of them
            # and be depended on by the second
            pos[merged] = (min(pos[a][0], pos[b][0]), max(pos[a][1], pos[b][1]))
            a = merged              # keeps collecting partners among the nodes that follow
    return count


# --------------------------------------------------------------------------
def inplace_elemwise(fgraph):
    """The role of ``InplaceElemwiseOptimizer`` (``theano/tensor/opt.py:150-410``):
    an elementwise kernel writes its result over an input of identical type when
    nothing else reads that input - it is an intermediate computed by another
    kernel of this function, used once, not a view, not an output.  Each thread
    reads exactly the positions it writes, so the aliasing is safe in every
    elementwise plan.  Saves the allocation and lowers the function's peak memory;
    on this device it moves no fewer bytes."""
    from .rowchain import HipRowChain
    count = 0
    for node in fgraph.toposort():
        op = node.op
        if not isinstance(op, HipElemwise) or len(node.outputs) != 1 or op.inplace_pattern:
            continue
        out = node.outputs[0]
        for idx, i in enumerate(node.inputs):
            if (i.type != out.type or i.owner is None or i in fgraph.outputs or
                    not isinstance(i.owner.op, (HipElemwise, HipCAReduce, HipRowChain))):
                continue
            if fgraph.n_clients(i) != 1 or list(node.inputs).count(i) != 1:
                continue
            new = HipElemwise(op.scalar_op, {0: idx}).make_node(*node.inputs).outputs[0]
            if new.type != out.type:
                continue
            fgraph.replace(out, new)
            count += 1
            break
    return count


def fuse_reduction_of_stored_result(fgraph):
    """An elementwise result that something else needs as well (it is an output, say) and a plain reduction
    of it over every dimension but the last - the per-channel sum of an NHWC result - become one node,
    whose kernel accumulates while it stores wherever its access plan allows (``HipElemwiseReduce``).  Runs
    after every other fusion pass: those would have folded the elementwise node into the reduction had
    nothing else read it."""
    count = 0
    for red in fgraph.toposort():
        op = red.op
        if (type(op) is not HipCAReduce or red not in fgraph.apply_nodes or op.pre_scalar_op is not None or
                op.post_scalar_op is not None or len(op.scalar_ops) != 1 or len(red.inputs) != 1):
            continue
        x = red.inputs[0]
        ew = x.owner
        if ew is None or type(ew.op) is not HipElemwise or ew.op.inplace_pattern:
            continue
        nd = x.type.ndim
        if nd < 2 or op.axis != tuple(range(nd - 1)) or any(x.type.broadcastable[:-1]):
            continue
        if isinstance(op.scalar_ops[0], (scal.Maximum, scal.Minimum)) or codegen_identity(op.scalar_ops[0]) is None:
            continue            # the zero-length error of max / min stays with the plain reduction
        new_op = HipElemwiseReduce(ew.op.scalar_op, (ew.outputs.index(x),), op.scalar_ops, op.acc_dtypes, op.out_dtypes)
        new = new_op.make_node(*ew.inputs)
        n_ew = len(ew.outputs)
        if [o.type for o in new.outputs] != [o.type for o in ew.outputs] + [red.outputs[0].type]:
            continue
        for o, no in zip(ew.outputs, new.outputs[:n_ew]):
            fgraph.replace(o, no)
        fgraph.replace(red.outputs[0], new.outputs[n_ew])
        count += 1
    return count


def codegen_identity(scalar_op):
    from .codegen import reduce_identity
    try:
        return reduce_identity(scalar_op, "int64")
    except Exception:
        return None


def optimize(fgraph, fuse=True, rowchain=True, inplace=True):
    """Full pipeline: clean up, lift, fuse, then in-place."""
    from ..tensor.opt import canonicalize
    canonicalize(fgraph)
    fgraph = lift_to_hip(fgraph)
    gof.merge_identical(fgraph)
    if fuse:
        fuse_elemwise(fgraph)
        if rowchain:
            from .rowchain import fuse_row_chains
            fuse_row_chains(fgraph)
        fuse_around_reductions(fgraph)
        fuse_reduction_of_stored_result(fgraph)
    if inplace:
        inplace_elemwise(fgraph)
    return fgraph


def fuse_around_reductions(fgraph):
    """The passes that follow elementwise fusion on a lifted graph: reductions take in their
    elementwise producers and consumers, siblings share a launch."""
    merge_sibling_reductions(fgraph)
    fuse_reduce_prologue(fgraph)
    gof.merge_identical(fgraph)
    merge_sibling_reductions(fgraph)
    gof.merge_identical(fgraph)
    share_equal_accumulators(fgraph)
    fuse_reduce_epilogue(fgraph)
    # a sum that reads results of a reduction over the same elements joins that reduction's pass
    from .hoist import hoist_result_operands, merge_chained_reductions
    if config.merge_dependent_reductions:
        if hoist_result_operands(fgraph):
            gof.merge_identical(fgraph)
        if merge_chained_reductions(fgraph):
            gof.merge_identical(fgraph)
            fuse_reduce_epilogue(fgraph)
    fuse_argmax_prologue(fgraph)
    gof.merge_identical(fgraph)
    fuse_elemwise(fgraph)          # producers that lost their other clients to an epilogue
    gof.merge_identical(fgraph)
    if merge_sibling_elemwise(fgraph):
        fuse_elemwise(fgraph)      # a producer whose clients all ended up in one kernel joins it
        gof.merge_identical(fgraph)
