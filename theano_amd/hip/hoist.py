"""Two rewrites that let a reduction share its pass over memory with the reduction its own
operands come from.

A gradient graph such as batch normalisation's holds ``sum(g * (x - mean))`` next to the
``sum(x)`` that ``mean`` itself is made of.  Both read ``x``, but the first cannot start before the
second has finished, so they stay two kernels and ``x`` is read twice.  Since ``mean`` is constant
along the reduced axes,

    sum(g * (x - mean)) = sum(g * x) - mean * sum(g)

and the sums on the right no longer need ``mean`` while they run: it moves from the per-element
prologue into the per-result epilogue (``hoist_result_operands``).  A reduction whose epilogue -
and only its epilogue - depends on another reduction over the same elements can then run in the
same kernel, the two epilogues chained (``merge_chained_reductions``).  The reference has no
counterpart: it keeps every CAReduce a node of its own (``theano/tensor/opt.py:7071-7470`` fuses
elementwise nodes only).

Only sums with float64 accumulators are rewritten, and only expressions that are of first degree in
the hoisted operands.  The terms of the expanded sums are far larger than the terms of the original
one when the mean is large against the spread (``g * x`` against ``g * (x - mean)``), so a product of
free factors must not be rounded to the operands' own type: a float32 product would put an error of
2**-24 |g x| into every term, |mean| / sigma times what the reference's ``g * (x - mean)`` carries.
Every product or quotient of free factors is therefore formed in float64 (the product of two float32
values is exact there; where both factors are float16 values widened to float32 the float32 product is
exact already and stays).  The difference of the two sums then carries a relative error of 2**-53 times
the ratio of their size to the result's, invisible at float32 (let alone float16) precision, where a
second-degree expansion (``sum((x - mean)**2)``) would cancel catastrophically.
"""
import numpy as np

from .. import gof
from .. import scalar as scal
from ..config import config
from ..gof import Constant
from ..tensor import basic as T
from .ops import HipArrayType, HipCAReduce, HipDimShuffle, HipElemwise, _is_host_scalar

_FLOATS = ("float32", "float64")
# operands of an epilogue: eight bytes each in the kernel's argument block of 4096 bytes
_MAX_EXTRAS = 32


def _depends(outputs, roots):
    """The scalar variables among the ancestors of ``outputs`` (inclusive) that depend on ``roots``."""
    dep = set(roots)
    for node in gof.io_toposort([], outputs):
        if any(i in dep for i in node.inputs):
            dep.update(node.outputs)
    return dep


class _NotSeparable(Exception):
    pass


def _times(a, b):
    return a if b is None else (b if a is None else scal.mul(a, b))


def _f64(v):
    return v if v.type.dtype == "float64" else scal.cast(v, "float64")


def _half_bits(v):
    """Is ``v`` a float16 value (possibly widened)?  Such a value has 11 significant bits."""
    while v.owner is not None and isinstance(v.owner.op, (scal.Cast, scal.Identity)) and (
            v.type.dtype in scal.float_dtypes and v.owner.inputs[0].type.dtype in scal.float_dtypes and
            np.dtype(v.type.dtype).itemsize >= np.dtype(v.owner.inputs[0].type.dtype).itemsize):
        v = v.owner.inputs[0]
    return v.type.dtype == "float16"


def _free_times(a, b):
    """The product of two free factors without a rounding: in float64, or in float32 where both are
    float16 values (22 significant bits)."""
    if a is None or b is None:
        return a if b is None else b
    if _half_bits(a) and _half_bits(b) and a.type.dtype == b.type.dtype == "float32":
        return scal.mul(a, b)
    return scal.mul(_f64(a), _f64(b))


def _terms(v, cset, dep, pure, memo):
    """``v`` as a list of terms ``(c, k, h, f)`` meaning ``k * c * h * f``: ``c`` one hoisted scalar or
    None (1), ``k`` a Python float, ``h`` an expression of host scalars and constants only or None, ``f`` an
    expression free of hoisted scalars or None.  Everything but ``f`` is left to the epilogue.
    ``dep``: the variables that depend on hoisted scalars; ``pure``: those made of host scalars only."""
    if v in memo:
        return memo[v]
    if v in cset:
        res = [(v, 1.0, None, None)]
    elif isinstance(v, Constant):
        if v.type.dtype not in scal.float_dtypes and v.type.dtype not in scal.int_dtypes:
            raise _NotSeparable()
        res = [(None, float(v.data), None, None)]
    elif v in pure:
        res = [(None, 1.0, v, None)]
    elif v not in dep:
        res = [(None, 1.0, None, v)]
    else:
        node, op = v.owner, v.owner.op
        ins = node.inputs
        if isinstance(op, (scal.Cast, scal.Identity)):
            # a change of float type is exact towards the wider type and the accumulators are float64
            if v.type.dtype not in _FLOATS or ins[0].type.dtype not in scal.float_dtypes:
                raise _NotSeparable()
            res = _terms(ins[0], cset, dep, pure, memo)
        elif isinstance(op, scal.Add):
            res = [t for i in ins for t in _terms(i, cset, dep, pure, memo)]
        elif isinstance(op, scal.Sub):
            res = _terms(ins[0], cset, dep, pure, memo) + [(c, -k, h, f) for c, k, h, f in
                                                          _terms(ins[1], cset, dep, pure, memo)]
        elif isinstance(op, scal.Neg):
            res = [(c, -k, h, f) for c, k, h, f in _terms(ins[0], cset, dep, pure, memo)]
        elif isinstance(op, scal.Mul):
            res = [(None, 1.0, None, None)]
            for i in ins:
                nxt = []
                for c1, k1, h1, f1 in res:
                    for c2, k2, h2, f2 in _terms(i, cset, dep, pure, memo):
                        if c1 is not None and c2 is not None:
                            raise _NotSeparable()          # second degree
                        nxt.append((c1 if c1 is not None else c2, k1 * k2, _times(h1, h2), _free_times(f1, f2)))
                res = nxt
        elif isinstance(op, scal.TrueDiv):
            den = ins[1]
            if den in dep or den.type.dtype not in scal.float_dtypes:
                raise _NotSeparable()
            res = []
            for c, k, h, f in _terms(ins[0], cset, dep, pure, memo):
                if isinstance(den, Constant):
                    res.append((c, k / float(den.data), h, f))
                elif den in pure:
                    res.append((c, k, scal.inv(den) if h is None else scal.true_div(h, den), f))
                else:
                    res.append((c, k, h, scal.inv(_f64(den)) if f is None else scal.true_div(_f64(f), _f64(den))))
        else:
            raise _NotSeparable()
        if v.type.dtype not in _FLOATS:
            raise _NotSeparable()
    memo[v] = res
    return res


def _canon(v):
    """``v`` without identity wrappers."""
    while v.owner is not None and isinstance(v.owner.op, scal.Identity):
        v = v.owner.inputs[0]
    return v


_RANK = {"float16": 0, "float32": 1, "float64": 2}


def _unique_accumulators(s_inputs, exprs, ops, acc_dts):
    """One Composite over ``s_inputs`` yielding ``exprs`` with equal (expression, op) pairs computed and
    accumulated once; returns (composite, ops, acc dtypes, position of each original in it).  Two sums
    of one expression that differ in their float accumulator type share the wider one: an accumulator
    wider than asked for is never farther from the exact sum."""
    comp = scal.Composite(s_inputs, exprs)
    ops, acc_dts = list(ops), list(acc_dts)
    uniq, where = [], []
    for s, o in enumerate(comp.outputs):
        for q, u in enumerate(uniq):
            same = _canon(comp.outputs[u]) is _canon(o) or (
                isinstance(o, Constant) and isinstance(comp.outputs[u], Constant) and
                o.type == comp.outputs[u].type and o.data == comp.outputs[u].data)
            if not same or ops[u] != ops[s]:
                continue
            if acc_dts[u] != acc_dts[s]:
                if not (isinstance(ops[s], scal.Add) and acc_dts[u] in _RANK and acc_dts[s] in _RANK):
                    continue
                if _RANK[acc_dts[s]] > _RANK[acc_dts[u]]:
                    acc_dts[u] = acc_dts[s]
            where.append(q)
            break
        else:
            where.append(len(uniq))
            uniq.append(s)
    if len(uniq) < len(exprs):
        comp = scal.Composite(comp.inputs, [comp.outputs[u] for u in uniq])
    return comp, [ops[u] for u in uniq], [acc_dts[u] for u in uniq], where


def _same_elements(a, b):
    """Do the reductions ``a`` and ``b`` walk the same elements?  Same axes, and a common device
    operand that spans the whole reduce domain of both (which fixes every extent at run time)."""
    if a.op.axis != b.op.axis:
        return False
    pats = []
    for n in (a, b):
        red_in = n.inputs[:len(n.inputs) - n.op.n_extra]
        nd = max(i.type.ndim for i in red_in)
        pats.append([all(bb) for bb in zip(*[i.type.broadcastable for i in red_in if i.type.ndim == nd])])
    if pats[0] != pats[1]:
        return False
    full = set(id(i) for i in a.inputs[:len(a.inputs) - a.op.n_extra]
               if isinstance(i.type, HipArrayType) and list(i.type.broadcastable) == pats[0])
    return any(id(i) in full for i in b.inputs[:len(b.inputs) - b.op.n_extra])


def _reduction_ancestors(var, limit=2000):
    out, stack, seen = [], [var], set()
    while stack and len(seen) < limit:
        v = stack.pop()
        if id(v) in seen or v.owner is None:
            continue
        seen.add(id(v))
        if isinstance(v.owner.op, HipCAReduce):
            out.append(v.owner)
        stack.extend(v.owner.inputs)
    return out


def hoist_result_operands(fgraph):
    """Moves operands that are constant along the reduced axes, and that come from a reduction over the
    same elements, out of a sum's prologue into its epilogue; returns the number of nodes rewritten."""
    count = 0
    for red in fgraph.toposort():
        op = red.op
        if not isinstance(op, HipCAReduce) or op.pre_scalar_op is None or red not in fgraph.apply_nodes:
            continue
        n_in = len(red.inputs) - op.n_extra
        red_in, extras = list(red.inputs[:n_in]), list(red.inputs[n_in:])
        nd = max(i.type.ndim for i in red_in)
        axis = op.axis if op.axis is not None else tuple(range(nd))
        # per-result operands: extent 1 along every reduced axis, the results' own extents along the others
        pattern = [all(bb) for bb in zip(*[i.type.broadcastable for i in red_in if i.type.ndim == nd])]
        hoist = [k for k, i in enumerate(red_in)
                 if isinstance(i.type, HipArrayType) and i.type.ndim == nd and i.type.dtype in _FLOATS and
                 all(i.type.broadcastable[d] == (d in axis or pattern[d]) for d in range(nd)) and
                 any(_same_elements(p, red) for p in _reduction_ancestors(i))]
        if not hoist:
            continue
        new = _hoisted(fgraph, red, hoist, axis)
        if new is None:
            continue
        for o, no in zip(red.outputs, new.outputs):
            fgraph.replace(o, no)
        count += 1
    return count


def _hoisted(fgraph, red, hoist, axis):
    op = red.op
    pre = op.pre_scalar_op
    n_in = len(red.inputs) - op.n_extra
    red_in, extras = list(red.inputs[:n_in]), list(red.inputs[n_in:])
    K = len(op.scalar_ops)
    cset = set(pre.inputs[k] for k in hoist)
    dep = _depends(pre.outputs, cset)
    host = [pre.inputs[k] for k in range(n_in) if _is_host_scalar(red_in[k])]
    data = [pre.inputs[k] for k in range(n_in) if k not in hoist and not _is_host_scalar(red_in[k])]
    pure = _depends(pre.outputs, host) - _depends(pre.outputs, data) - dep
    # per accumulator: untouched, or its terms
    plans = []
    for k in range(K):
        if pre.outputs[k] not in dep:
            plans.append(None)
            continue
        if not isinstance(op.scalar_ops[k], scal.Add) or op.acc_dtypes[k] != "float64":
            return None
        try:
            plans.append(_terms(pre.outputs[k], cset, dep, pure, {}))
        except _NotSeparable:
            return None
    # new accumulators: the untouched ones, then one sum per free expression
    acc_exprs, acc_ops, acc_dts = [], [], []
    slot_of_old = {}
    for k in range(K):
        if plans[k] is None:
            slot_of_old[k] = len(acc_exprs)
            acc_exprs.append(pre.outputs[k])
            acc_ops.append(op.scalar_ops[k])
            acc_dts.append(op.acc_dtypes[k])
    need_count = False
    for k in range(K):
        if plans[k] is None:
            continue
        cur = []
        for c, coef, h, f in plans[k]:
            if f is None:
                need_count = True
                cur.append((c, coef, h, None))
                continue
            cur.append((c, coef, h, len(acc_exprs)))
            acc_exprs.append(f)
            acc_ops.append(scal.add)
            acc_dts.append("float64")
        plans[k] = cur
    reach = _ancestors(acc_exprs)
    keep_in = [k for k in range(n_in) if pre.inputs[k] in reach]
    if any(k in hoist for k in keep_in) or not any(pre.inputs[k] in data for k in keep_in):
        return None
    new_pre, acc_ops, acc_dts, where = _unique_accumulators([pre.inputs[k] for k in keep_in], acc_exprs, acc_ops, acc_dts)
    if len(acc_ops) > 8:
        return None
    # the epilogue: every accumulator arrives in its own type; recombine, then whatever followed
    old_post_in = list(op.post_in_dtypes) if op.post_scalar_op is not None else list(op.out_dtypes)
    s_acc = [scal.Scalar(dt)() for dt in acc_dts]
    s_old_extras = [scal.Scalar(e.type.dtype)() for e in extras]
    new_extras, s_new_extras = list(extras), list(s_old_extras)
    count = None
    if need_count:
        full = [i for i in red_in if isinstance(i.type, HipArrayType) and not any(i.type.broadcastable[a] for a in axis)]
        if not full:
            return None
        for a in axis:
            se = scal.Scalar("float64")()
            new_extras.append(T.ShapeFloat(a, "float64")(full[0]))
            s_new_extras.append(se)
            count = se if count is None else scal.mul(count, se)
    results, wanted = [], set()
    for k in range(K):
        if plans[k] is None:
            results.append(scal.cast(s_acc[where[slot_of_old[k]]], old_post_in[k]))
            continue
        total = None
        for c, coef, h, slot in plans[k]:
            t = s_acc[where[slot]] if slot is not None else count
            if h is not None:
                t = scal.mul(scal.cast(h, "float64"), t)
                wanted.update(v for v in _ancestors([h]) if v in host)
            if c is not None:
                t = scal.mul(scal.cast(c, "float64"), t)
                wanted.add(c)
            if coef == -1.0:
                t = scal.neg(t)
            elif coef != 1.0:
                t = scal.mul(scal.constant(coef, dtype="float64"), t)
            total = t if total is None else scal.add(total, t)
        results.append(scal.cast(total, old_post_in[k]))
    # the prologue's own scalars stand for the operands that moved (or were copied) to the epilogue
    for k in range(n_in):
        if pre.inputs[k] in wanted:
            new_extras.append(red_in[k])
            s_new_extras.append(pre.inputs[k])
    if op.post_scalar_op is None:
        outs = [scal.cast(r, dt) for r, dt in zip(results, op.out_dtypes)]
    else:
        outs = op.post_scalar_op(*(results + s_old_extras), return_list=True)
    outs = [scal.identity(o) if (o in s_acc or o in s_new_extras) else o for o in outs]
    if len(new_extras) > _MAX_EXTRAS:
        return None
    new_post = scal.Composite(s_acc + s_new_extras, outs)
    new_op = HipCAReduce(tuple(acc_ops), op.axis, tuple(acc_dts), op.out_dtypes, new_pre, new_post, tuple(acc_dts),
                         len(new_extras))
    node = new_op.make_node(*([red_in[k] for k in keep_in] + new_extras))
    if [o.type for o in node.outputs] != [o.type for o in red.outputs]:
        return None
    return node


def _ancestors(outputs):
    seen, stack = set(), list(outputs)
    while stack:
        v = stack.pop()
        if v in seen:
            continue
        seen.add(v)
        if v.owner is not None:
            stack.extend(v.owner.inputs)
    return seen


# --------------------------------------------------------------------------
def merge_chained_reductions(fgraph):
    """``b``'s epilogue reads results of ``a``, nothing else of ``b`` depends on ``a``, and both walk the
    same elements: one kernel accumulates for both and runs ``a``'s epilogue, then ``b``'s on its values."""
    from .opt import _cheap, _depends_on, _scalar_constant, _TRIVIAL_OPS
    count = 0
    changed = True
    while changed:
        changed = False
        reds = [n for n in fgraph.toposort() if isinstance(n.op, HipCAReduce)]
        for bi, b in enumerate(reds):
            if b.op.post_scalar_op is None or not b.op.n_extra:
                continue
            nb = len(b.inputs) - b.op.n_extra
            for a in reds[:bi]:
                if not _same_elements(a, b):
                    continue
                if a.outputs[0].type.broadcastable != b.outputs[0].type.broadcastable:
                    continue
                if any(_depends_on(i, a) for i in b.inputs[:nb]):
                    continue
                if not any(_depends_on(e, a) for e in b.inputs[nb:]):
                    continue
                merged = _chain(fgraph, a, b, _cheap, _depends_on, _scalar_constant, _TRIVIAL_OPS)
                if merged is None:
                    continue
                for o, no in zip(list(a.outputs) + list(b.outputs), merged.outputs):
                    fgraph.replace(o, no)
                count += 1
                changed = True
                break
            if changed:
                break
    return count


def _chain(fgraph, a, b, _cheap, _depends_on, _scalar_constant, _TRIVIAL_OPS):
    na, nb = len(a.inputs) - a.op.n_extra, len(b.inputs) - b.op.n_extra
    inputs, s_inputs = [], []

    def scalar_for(v):
        for t, s in zip(inputs, s_inputs):
            if t is v:
                return s
        s = scal.Scalar(v.type.dtype)()
        inputs.append(v)
        s_inputs.append(s)
        return s

    pre_outs = []
    for n, k in ((a, na), (b, nb)):
        args = [scalar_for(v) for v in n.inputs[:k]]
        if n.op.pre_scalar_op is None:
            pre_outs.extend(scal.identity(x) for x in args)
        else:
            pre_outs.extend(n.op.pre_scalar_op(*args, return_list=True))
    if len(inputs) > config.max_fused_inputs:
        return None
    ops = list(a.op.scalar_ops + b.op.scalar_ops)
    acc_dts = list(a.op.acc_dtypes + b.op.acc_dtypes)
    pre, ops, acc_dts, where = _unique_accumulators(s_inputs, pre_outs, ops, acc_dts)
    if len(ops) > 8:
        return None
    # every accumulator reaches the epilogue in its own type and takes the type each epilogue expects there
    pia = list(a.op.post_in_dtypes) if a.op.post_scalar_op is not None else list(a.op.out_dtypes)
    pib = list(b.op.post_in_dtypes)
    s_acc = [scal.Scalar(dt)() for dt in acc_dts]
    Ka = len(a.op.scalar_ops)
    s_acc_a = [scal.cast(s_acc[where[k]], dt) for k, dt in enumerate(pia)]
    s_acc_b = [scal.cast(s_acc[where[Ka + k]], dt) for k, dt in enumerate(pib)]
    extras, s_extras = [], []

    def extra_for(v):
        for t, s in zip(extras, s_extras):
            if t is v:
                return s
        s = scal.Scalar(v.type.dtype)()
        extras.append(v)
        s_extras.append(s)
        return s

    a_ex = [extra_for(e) for e in a.inputs[na:]]
    if a.op.post_scalar_op is None:
        cur_a = [scal.cast(s, dt) for s, dt in zip(s_acc_a, a.op.out_dtypes)]
    else:
        cur_a = a.op.post_scalar_op(*(s_acc_a + a_ex), return_list=True)
    layout = None

    def value_of(v, depth=0):
        """Scalar expression of a per-result value of ``b``'s epilogue in terms of ``a``'s results."""
        c = _scalar_constant(v)
        if c is not None:
            return c
        if v.owner is a:
            return cur_a[a.outputs.index(v)]
        if not _depends_on(v, a):
            if not (_is_host_scalar(v) or isinstance(v.type, HipArrayType)):
                return None
            return extra_for(v)
        p = v.owner
        if isinstance(p.op, HipDimShuffle):
            kept = [o for o in p.op.new_order if o != "x"]
            if kept != sorted(kept) or depth > 8:
                return None
            return value_of(p.inputs[0], depth + 1)
        if (isinstance(p.op, HipElemwise) and len(p.outputs) == 1 and not p.op.inplace_pattern and depth <= 8 and
                _cheap(p.op.scalar_op, _TRIVIAL_OPS)):
            args = [value_of(i, depth + 1) for i in p.inputs]
            if all(x is not None for x in args):
                return p.op.scalar_op(*args)
        return None

    b_ex = []
    for e in b.inputs[nb:]:
        x = value_of(e)
        if x is None:
            return None
        b_ex.append(x)
    cur_b = b.op.post_scalar_op(*(s_acc_b + b_ex), return_list=True)
    if len(extras) > _MAX_EXTRAS:
        return None
    outs = [scal.identity(o) if (o in s_acc or o in s_extras) else o for o in cur_a + cur_b]
    post = scal.Composite(s_acc + s_extras, outs)
    op = HipCAReduce(tuple(ops), a.op.axis, tuple(acc_dts), a.op.out_dtypes + b.op.out_dtypes, pre, post,
                     tuple(acc_dts), len(extras))
    node = op.make_node(*(inputs + extras))
    if [o.type for o in node.outputs] != [o.type for o in list(a.outputs) + list(b.outputs)]:
        return None
    return node
