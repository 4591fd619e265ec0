"""Row chains: islands of elementwise nodes and last-axis reductions executed by
one kernel that keeps each row on chip.

The reference never fuses across a reduction (``theano/tensor/opt.py:7071-7313``
only merges Elemwise nodes); for row softmax it substitutes a hand-written
``Softmax`` op instead (``theano/tensor/nnet/nnet.py:411-600, 888-925``).  Here the
same effect is obtained for any such island: the sub-graph is turned into a
straight-line row program (load, elementwise steps, reductions, store), code is
generated for it and one launch replaces the whole island.  Results follow the
per-node semantics: elementwise steps use each scalar op's ``c_code``, every
reduction accumulates in the accumulator dtype of its node and is cast to the
node's output dtype before anything consumes it.
"""
import ctypes
import hashlib

import numpy as np

from .. import gof
from ..config import config
from .. import scalar as scal
from ..gof import Apply, Op
from ..scalar import Scalar, compute_ctype, storage_ctype
from . import codegen
from .ops import (HipArrayType, HipCAReduce, HipDimShuffle, HipElemwise, _is_host_scalar)
from .runtime import HipArray, call_flags, check, host_scalar_thx, lib, mark_reused, thx_array

FULL, ROW, COL, SCALAR = 0, 1, 2, 3
THX_ERR_UNSUPPORTED = 6


def _klass(var, nd, red=None):
    """Operand class of a rank-``nd`` variable by its broadcast pattern, for reductions over the
    axes ``red`` (default: the last one): ROW is one value per kept index, COL (last-axis chains
    only) one value per position along the reduced axis."""
    b = var.type.broadcastable
    n_red = 1 if red is None else len(red)
    if len(b) == nd - n_red:
        # the kept axes alone (a reduction's result before keepdims): one value per kept index
        return ROW if not any(b) else (SCALAR if all(b) else None)
    if len(b) != nd:
        return None
    if not any(b):
        return FULL
    if red is None or tuple(red) == (nd - 1,):
        if all(b):
            return SCALAR
        if b[-1] and not any(b[:-1]):
            return ROW
        if not b[-1] and all(b[:-1]):
            return COL
        return None
    if all(b[d] == (d in red) for d in range(nd)):
        return ROW          # also the keepdims form of a reduction over every axis
    return SCALAR if all(b) else None


def _chain_axes(nd, axis):
    """The reduced axes as a sorted tuple if a chain can run over them: the kept axes are adjacent
    and at least one reduced axis trails them (it is walked with unit stride)."""
    red = tuple(range(nd)) if axis is None else tuple(sorted(axis))
    if not red or len(set(red)) != len(red) or red[-1] != nd - 1:
        return None
    kept = [d for d in range(nd) if d not in red]
    if kept and kept != list(range(kept[0], kept[-1] + 1)):
        return None
    return red


def _row_shape(full, red, keepdims):
    if keepdims:
        return tuple(1 if d in red else n for d, n in enumerate(full))
    return tuple(n for d, n in enumerate(full) if d not in red)


def _tests_equality(scalar_op):
    """Does the scalar operation (or a Composite's inner graph) compare values with == or != ?"""
    if isinstance(scalar_op, (scal.EQ, scal.NEQ)):
        return True
    if isinstance(scalar_op, scal.Composite):
        return any(_tests_equality(n.op) for n in gof.io_toposort(scalar_op.inputs, scalar_op.outputs))
    return False


class RowProgram(object):
    """Straight-line program over per-element values and per-row scalars."""

    def __init__(self):
        self.in_kinds, self.in_dtypes = [], []
        self.steps = []        # ("ew", scalar_op, arg ids, out ids) | ("red", scalar_op, acc, out dtype, arg, out)
        self.var = {}          # id -> (per_element, dtype)
        self.outputs = []      # (var id, kind, dtype)
        self.axes = None       # reduced axes of the full shape; None: the last one
        self.held_passes = 0
        self._next = 0

    def new_var(self, per_element, dtype):
        i = self._next
        self._next += 1
        self.var[i] = (per_element, dtype)
        return i

    def add_input(self, kind, dtype):
        self.in_kinds.append(kind)
        self.in_dtypes.append(dtype)
        return self.new_var(kind in (FULL, COL), dtype)

    # -- code generation
    def source(self):
        lines, ops = [], []
        nm = lambda i: ("v%d" if self.var[i][0] else "s%d") % i
        elem = lambda i: ("v%d[ch][k]" if self.var[i][0] else "s%d") % i
        loaders = {FULL: "load_full", ROW: "load_row", COL: "load_col", SCALAR: "load_scalar"}
        for k, (kind, dt) in enumerate(zip(self.in_kinds, self.in_dtypes)):
            ct = compute_ctype(dt)
            decl = "%s v%d[X::NCH][X::VEC];" % (ct, k) if kind in (FULL, COL) else "%s s%d;" % (ct, k)
            lines.append("%s x.template %s<%d, %s, %s>(%s);" % (decl, loaders[kind], k, storage_ctype(dt), ct, nm(k)))
        for step in self.steps:
            if step[0] == "ew":
                _, op, args, outs = step
                node = op.make_node(*[Scalar(self.var[a][1])() for a in args])
                per_elem = any(self.var[o][0] for o in outs)
                for o in outs:
                    ct = compute_ctype(self.var[o][1])
                    lines.append("%s v%d[X::NCH][X::VEC];" % (ct, o) if self.var[o][0] else "%s s%d;" % (ct, o))
                code = op.c_code(node, [elem(a) for a in args], [elem(o) for o in outs])
                if per_elem:
                    lines.append("_Pragma(\"unroll\") for (int ch = 0; ch < X::NCH; ++ch) {\n"
                                 "_Pragma(\"unroll\") for (int k = 0; k < X::VEC; ++k) {\n%s\n}}" % code)
                else:
                    lines.append("{\n%s\n}" % code)
            else:
                _, op, acc_dt, out_dt, arg, out = step
                act, oct_ = compute_ctype(acc_dt), compute_ctype(out_dt)
                ident = codegen.reduce_identity(op, acc_dt)
                if ident is None:
                    raise NotImplementedError("reduction with %s has no identity element" % op)
                cnode = Apply(op, [Scalar(acc_dt)(), Scalar(acc_dt)()], [Scalar(acc_dt)()])
                ops.append("  struct Op%d { THX_DEV static void comb(%s& a, const %s& b) { %s } };" % (
                    out, act, act, op.c_code(cnode, ["a", "b"], ["a"])))
                lines.append("%s a%d = %s;" % (act, out, ident))
                lines.append("_Pragma(\"unroll\") for (int ch = 0; ch < X::NCH; ++ch) { if (x.valid(ch)) {\n"
                             "_Pragma(\"unroll\") for (int k = 0; k < X::VEC; ++k) { if (x.counts(ch, k)) { %s t = (%s)v%d[ch][k]; "
                             "Op%d::comb(a%d, t); } } } }" % (act, act, arg, out, out))
                lines.append("a%d = x.template allreduce<Op%d, %s>(a%d);" % (out, out, act, out))
                val = "a%d" % out
                if out_dt == "bool":
                    val = "(%s ? 1 : 0)" % val
                # the result takes the storage precision of the node's output before anything reads it
                lines.append("%s s%d = (%s)(%s)%s;" % (oct_, out, oct_, storage_ctype(out_dt), val))
        for k, (vid, kind, dt) in enumerate(self.outputs):
            ct = compute_ctype(self.var[vid][1])
            st = "store_full" if kind == FULL else "store_row"
            lines.append("x.template %s<%d, %s, %s>(%s);" % (st, k, storage_ctype(dt), ct, nm(vid)))
        body = "\n".join("    " + l for l in "\n".join(lines).splitlines())
        text = "  enum { NIN = %d, NOUT = %d };\n%s\n" % (len(self.in_kinds), len(self.outputs), "\n".join(ops))
        if self.axes is None:
            text += "  template <class X> THX_DEV static void row(X& x) {\n%s\n  }" % body
        held = self._held_lines()
        if held is not None and self.held_passes >= 2:   # one pass gains nothing from keeping the values
            text += "\n  template <class X> THX_DEV static void held(X& x) {\n%s\n  }" % "\n".join(
                "    " + l for l in "\n".join(held).splitlines())
        name = "C" + hashlib.sha1((text + repr(self.in_kinds) + repr(self.axes)).encode()).hexdigest()[:16]
        return "struct %s {\n%s\n};\n" % (name, text), name

    def _held_lines(self):
        """The island for the held form (kernels/thx_rowchain.h): full-shaped inputs stay on chip in
        their storage type and nothing per element is kept between two loops over them; every loop
        (one per group of independent reductions, one for the stores) recomputes the elementwise
        steps it needs.  None when an operand has no place in that form."""
        self.held_passes = 0       # loops over the held values
        if COL in self.in_kinds or FULL not in self.in_kinds:
            return None
        n_in = len(self.in_kinds)
        lines = []
        nm = lambda i: ("e%d" if self.var[i][0] else "s%d") % i
        full_in = [k for k, kind in enumerate(self.in_kinds) if kind == FULL]
        for k, (kind, dt) in enumerate(zip(self.in_kinds, self.in_dtypes)):
            ct, st = compute_ctype(dt), storage_ctype(dt)
            if kind == FULL:
                lines.append("typename X::template Held<%d, %s> h%d; x.template hold<%d, %s>(h%d);" % (k, st, k, k, st, k))
            else:
                lines.append("%s s%d; x.template %s<%d, %s, %s>(s%d); s%d = X::uni(s%d);" % (
                    ct, k, "load_row" if kind == ROW else "load_scalar", k, st, ct, k, k, k))
        producer = {}          # per-element variable -> its elementwise step
        for step in self.steps:
            if step[0] == "ew" and any(self.var[o][0] for o in step[3]):
                for o in step[3]:
                    producer[o] = step

        def closure(vid, steps, inputs, scalars):
            """Elementwise steps (in program order), held inputs and per-index scalars behind a
            per-element variable."""
            if not self.var[vid][0]:
                scalars.add(vid)
                return
            if vid < n_in:
                inputs.add(vid)
                return
            step = producer[vid]
            if any(step is t for t in steps):
                return
            for a in step[2]:
                closure(a, steps, inputs, scalars)
            steps.append(step)

        def loop(reds, stores):
            steps, inputs, scalars = [], set(), set()
            for r in reds:
                closure(r[4], steps, inputs, scalars)
            for n, (vid, kind, dt) in stores:
                closure(vid, steps, inputs, scalars)
            out = []
            if stores:
                out.append("typename X::Pos q = x.begin();")
            out.append("_Pragma(\"unroll\") for (int ch = 0; ch < X::NCH; ++ch) {")
            out.append("  if (x.valid(ch)) {")
            for k in sorted(inputs):
                st = storage_ctype(self.in_dtypes[k])
                out.append("    const thx::Vec<%s, X::VEC> r%d = x.template get<%d, %s>(h%d, ch);" % (st, k, k, st, k))
            for n, (vid, kind, dt) in stores:
                out.append("    thx::Vec<%s, X::VEC> o%d;" % (storage_ctype(dt), n))
            out.append("    _Pragma(\"unroll\") for (int j = 0; j < X::VEC; ++j) {")
            for k in sorted(inputs):
                ct = compute_ctype(self.in_dtypes[k])
                out.append("      %s e%d = (%s)r%d.v[j];" % (ct, k, ct, k))
            for _, op, args, outs in steps:
                node = op.make_node(*[Scalar(self.var[a][1])() for a in args])
                for o in outs:
                    out.append("      %s %s;" % (compute_ctype(self.var[o][1]), nm(o)))
                out.append("      {\n%s\n      }" % op.c_code(node, [nm(a) for a in args], [nm(o) for o in outs]))
            for r in reds:
                act = compute_ctype(r[2])
                out.append("      { %s t = (%s)%s; Op%d::comb(a%d, t); }" % (act, act, nm(r[4]), r[5], r[5]))
            for n, (vid, kind, dt) in stores:
                out.append("      o%d.v[j] = (%s)%s;" % (n, storage_ctype(dt), nm(vid)))
            out.append("    }")
            for n, (vid, kind, dt) in stores:
                out.append("    x.template put<%d, %s>(q, o%d);" % (n, storage_ctype(dt), n))
            out.append("  }")
            if stores:
                out.append("  x.next(q);")
            for r in reds:
                out.append("  X::pin(a%d);" % r[5])
            out.append("  X::pace(ch);")
            out.append("}")
            return ["{"] + ["  " + l for l in out] + ["}"], scalars

        pending, deferred, blocked = [], [], set()

        def scalar_step(step):
            _, op, args, outs = step
            node = op.make_node(*[Scalar(self.var[a][1])() for a in args])
            for o in outs:
                lines.append("%s s%d;" % (compute_ctype(self.var[o][1]), o))
            lines.append("{\n%s\n}" % op.c_code(node, [nm(a) for a in args], [nm(o) for o in outs]))
            for o in outs:
                lines.append("s%d = X::uni(s%d);" % (o, o))

        def flush():
            """One loop for the reductions collected so far, then the per-index steps that waited for
            their results."""
            if pending:
                self.held_passes += 1
                for r in pending:
                    lines.append("%s a%d = %s;" % (compute_ctype(r[2]), r[5], codegen.reduce_identity(r[1], r[2])))
                text, _ = loop(pending, [])
                lines.extend(text)
                for k in full_in:
                    lines.append("x.template fence<%d, %s>(h%d);" % (k, storage_ctype(self.in_dtypes[k]), k))
                for _, op, acc_dt, out_dt, arg, out in pending:
                    act, oct_ = compute_ctype(acc_dt), compute_ctype(out_dt)
                    lines.append("a%d = x.template allreduce<Op%d, %s>(a%d);" % (out, out, act, out))
                    val = "a%d" % out
                    if out_dt == "bool":
                        val = "(%s ? 1 : 0)" % val
                    lines.append("%s s%d = X::uni((%s)(%s)%s);" % (oct_, out, oct_, storage_ctype(out_dt), val))
            for step in deferred:
                scalar_step(step)
            del pending[:], deferred[:]
            blocked.clear()

        for step in self.steps:
            if step[0] == "ew":
                _, op, args, outs = step
                if any(self.var[o][0] for o in outs):
                    continue           # per element: recomputed inside the loops that need it
                if blocked.intersection(args):
                    deferred.append(step)       # reads a reduction that later ones may still join
                    blocked.update(outs)
                else:
                    scalar_step(step)
            else:
                if codegen.reduce_identity(step[1], step[2]) is None:
                    return None
                # max / min of a computed floating-point value that a later step tests for equality (the gradient
                # of max does: eq(max, value)) needs the very same bits in both places, which a second evaluation
                # in another loop does not promise; values held as they were read always qualify
                if (isinstance(step[1], (scal.Maximum, scal.Minimum)) and step[4] >= n_in and
                        self.var[step[4]][1] in scal.continuous_dtypes and
                        any(t[0] == "ew" and _tests_equality(t[1]) for t in self.steps[self.steps.index(step) + 1:])):
                    return None
                steps, inputs, scalars = [], set(), set()
                closure(step[4], steps, inputs, scalars)
                if blocked.intersection(scalars):
                    flush()
                pending.append(step)
                blocked.add(step[5])
        flush()
        stores = [(n, o) for n, o in enumerate(self.outputs) if o[1] == FULL]
        if stores:
            self.held_passes += 1
            text, _ = loop([], stores)
            lines.extend(text)
        for n, (vid, kind, dt) in enumerate(self.outputs):
            if kind != FULL:
                lines.append("x.template store_row<%d, %s, %s>(%s);" % (n, storage_ctype(dt), compute_ctype(self.var[vid][1]), nm(vid)))
        return lines


_handles = {}


class HipRowChain(Op):
    """One launch for a whole elementwise + row-reduction island."""

    __props__ = ("signature",)

    def __init__(self, program, out_types, fallback):
        self.program = program
        self.src, self.name = program.source()
        self.signature = (self.name, tuple(program.in_kinds), tuple(str(t) for t in out_types), program.axes)
        self.out_types = list(out_types)
        self.fallback = fallback   # (inner input variables, inner output variables) of the original island

    def __str__(self):
        n_red = sum(1 for s in self.program.steps if s[0] == "red")
        over = "" if self.program.axes is None else ", axes %s" % (self.program.axes,)
        return "HipRowChain{%d steps, %d reductions%s}" % (len(self.program.steps), n_red, over)

    def make_node(self, *inputs):
        return Apply(self, list(inputs), [t() for t in self.out_types])

    def __getstate__(self):
        # the compiled form of the island (device handles inside) is rebuilt on first use
        d = dict(self.__dict__)
        d.pop("_fallback_function", None)
        return d

    def infer_shape(self, node, shapes):
        full = None
        for s, k in zip(shapes, self.program.in_kinds):
            if k == FULL:
                full = tuple(s)
        out = []
        red = self._red(len(full))
        for (vid, kind, dt), t in zip(self.program.outputs, self.out_types):
            out.append(full if kind == FULL else _row_shape(full, red, t.ndim == len(full)))
        return out

    def _red(self, nd):
        return (nd - 1,) if self.program.axes is None else self.program.axes

    def _handle(self):
        h = _handles.get(self.signature)
        if h is None:
            p = self.program
            dts = list(p.in_dtypes) + [dt for _, _, dt in p.outputs]
            kinds = list(p.in_kinds) + [k for _, k, _ in p.outputs]
            codes = (ctypes.c_int32 * len(dts))(*[scal.dtype_code(d) for d in dts])
            kk = (ctypes.c_int32 * len(kinds))(*kinds)
            handle = ctypes.c_void_p()
            check(lib.thx_rowchain_new(self.src.encode(), self.name.encode(), len(p.in_kinds), len(p.outputs), codes, kk,
                                       ctypes.byref(handle)))
            if p.axes is not None:
                check(lib.thx_rowchain_set_axes(handle, len(p.axes), (ctypes.c_int32 * len(p.axes))(*p.axes)))
            h = _handles[self.signature] = handle
        return h

    def perform(self, node, inputs, output_storage):
        p = self.program
        cache = node.tag.get("thx")
        if cache is None:
            cache = node.tag["thx"] = (self._handle(), (thx_array * len(inputs))(), (thx_array * len(p.outputs))(),
                                       [np.dtype(dt) for _, _, dt in p.outputs])
        handle, ins, outs, out_dt = cache
        full = None
        for v, k in zip(inputs, p.in_kinds):
            if k == FULL:
                full = v.shape
                break
        nd = len(full)
        red = self._red(nd)
        layout = tuple((v.shape, v.strides) for v in inputs if type(v) is HipArray)
        refused = node.tag.setdefault("thx_refused", set())
        if len(refused) > 256:          # a function called with ever new shapes: start over
            refused.clear()
        if layout in refused:           # turned away before with these shapes and strides
            results = self._run_fallback(inputs)
        else:
            last = node.tag.get("thx_last")
            if last is None:
                last = node.tag["thx_last"] = [None] * len(inputs)
            for k, v in enumerate(inputs):
                if type(v) is HipArray:
                    v.as_thx(ins[k])
                elif last[k] is not v:          # the same host array as last time: its descriptor stands
                    host_scalar_thx(v, nd, ins[k])
                    last[k] = v
            results = []
            for k, ((vid, kind, dt), t) in enumerate(zip(p.outputs, self.out_types)):
                shape = full if kind == FULL else _row_shape(full, red, t.ndim == nd)
                arr = HipArray._new_contiguous(tuple(shape), out_dt[k])
                arr.as_thx(outs[k])
                results.append(arr)
            mark_reused(node, ins, outs)
            rc = lib.thx_rowchain_call(handle, ins, outs, call_flags(node))
            if rc == THX_ERR_UNSUPPORTED:
                refused.add(layout)
                del results
                results = self._run_fallback(inputs)
            elif rc:
                check(rc)
        for k, arr in enumerate(results):
            output_storage[k][0] = arr

    def _run_fallback(self, inputs):
        """Shapes or strides the one-kernel form does not take (reduce domains too long for the
        registers and LDS of one block, rows that are not contiguous, too few kept indices): the island
        runs as reductions that compute their elementwise producers and consumers on the fly plus the
        elementwise kernels in between, compiled the first time this is needed like any function
        (same rewrites after row chains, same reuse marks, intermediate results dropped after their
        last use)."""
        f = getattr(self, "_fallback_function", None)
        if f is None:
            from . import opt
            from ..compile import Function, In, Out
            fg = gof.FunctionGraph(*self.fallback)
            opt.fuse_around_reductions(fg)
            opt.fuse_reduction_of_stored_result(fg)
            opt.inplace_elemwise(fg)
            f = self._fallback_function = Function(fg, [In(v) for v in fg.inputs],
                                                   [Out(o, device=True) for o in fg.outputs], False, [])
        return f.call_trusted(inputs)


# --------------------------------------------------------------------------
def _eligible(node, nd, red):
    op = node.op
    last = red == (nd - 1,)
    if isinstance(op, HipElemwise):
        if len(node.outputs) != 1 or op.inplace_pattern:
            return False
        if _klass(node.outputs[0], nd, red) not in (FULL, ROW):
            return False
        for i in node.inputs:
            if isinstance(i.type, HipArrayType):
                k = _klass(i, nd, red)
                if k is None or (k == COL and not last):
                    return False
            elif not _is_host_scalar(i):
                return False
        return True
    if isinstance(op, HipCAReduce):
        return (len(op.scalar_ops) == 1 and op.pre_scalar_op is None and op.post_scalar_op is None and
                len(node.inputs) == 1 and node.inputs[0].type.ndim == nd and
                _chain_axes(nd, op.axis) == red and
                _klass(node.inputs[0], nd, red) == FULL and
                # float16 accumulators: maxima and minima only, which pick one of the values whatever the
                # arithmetic's width (the row max of a float16 softmax then stays in the chain's one kernel)
                (op.acc_dtypes[0] != "float16" or isinstance(op.scalar_ops[0], (scal.Maximum, scal.Minimum))))
    if isinstance(op, HipDimShuffle):
        x = node.inputs[0]
        kept = iter(range(nd - len(red)))
        keepdims = tuple("x" if d in red else next(kept) for d in range(nd))
        return (x.type.ndim == nd - len(red) and not any(x.type.broadcastable) and
                tuple(op.new_order) == keepdims and x.owner is not None and
                isinstance(x.owner.op, (HipCAReduce, HipElemwise)))
    return False


def fuse_row_chains(fgraph):
    """Replace every island that contains a last-axis reduction by one
    HipRowChain node."""
    count = 0
    changed = True
    while changed:
        changed = False
        for seed in fgraph.toposort():
            if not isinstance(seed.op, HipCAReduce) or seed not in fgraph.apply_nodes:
                continue
            nd = seed.inputs[0].type.ndim
            red = _chain_axes(nd, seed.op.axis) if nd >= 1 else None
            if red is None or (red != (nd - 1,) and not config.held_chains) or not _eligible(seed, nd, red):
                continue
            island = _grow(fgraph, seed, nd, red)
            if island is None:
                continue
            if _replace(fgraph, island, nd, red):
                count += 1
                changed = True
                break
    return count


def _grow(fgraph, seed, nd, red):
    island = {seed}
    frontier = [seed]
    while frontier:
        n = frontier.pop()
        neigh = [i.owner for i in n.inputs if i.owner is not None]
        for o in n.outputs:
            neigh.extend(c for c, _ in fgraph.clients.get(o, []) if c != "output")
        for m in neigh:
            if m in island or m not in fgraph.apply_nodes or not _eligible(m, nd, red):
                continue
            if isinstance(m.op, HipDimShuffle) and m.inputs[0].owner not in island:
                # reached from a consumer: the keepdims view joins together with its reduction
                prod = m.inputs[0].owner
                if prod not in fgraph.apply_nodes or not _eligible(prod, nd, red):
                    continue
                island.add(prod)
                frontier.append(prod)
            island.add(m)
            frontier.append(m)
    # a DimShuffle only belongs with its reduction; drop strays whose producer never joined
    for m in list(island):
        if isinstance(m.op, HipDimShuffle) and m.inputs[0].owner not in island:
            island.discard(m)
    n_red = sum(1 for m in island if isinstance(m.op, HipCAReduce))
    n_ew = sum(1 for m in island if isinstance(m.op, HipElemwise))
    if n_red == 0 or n_red + n_ew < 2:
        return None
    # worth one kernel only if something inside consumes a reduction result: a lone reduction with
    # elementwise producers is served (for any row length) by the prologue-fused reduction kernels
    if not any(isinstance(m.op, HipElemwise) and any(
            i.owner in island and isinstance(i.owner.op, (HipCAReduce, HipDimShuffle)) for i in m.inputs)
            for m in island):
        return None
    # the island must not feed itself through outside nodes
    produced = set(id(o) for m in island for o in m.outputs)
    ext_inputs = [i for m in island for i in m.inputs if id(i) not in produced]
    stack, seen = [i for i in ext_inputs], set()
    while stack:
        v = stack.pop()
        if id(v) in seen or v.owner is None:
            continue
        seen.add(id(v))
        if v.owner in island:
            return None
        stack.extend(v.owner.inputs)
    return island


def _replace(fgraph, island, nd, red):
    order = [n for n in fgraph.toposort() if n in island]
    produced = set(id(o) for m in island for o in m.outputs)
    prog = RowProgram()
    if red != (nd - 1,):
        prog.axes = red
    ext_inputs, ids = [], {}

    def var_id(v):
        if id(v) in ids:
            return ids[id(v)]
        # an external operand
        if isinstance(v.type, HipArrayType):
            k = _klass(v, nd, red)
        else:
            k = SCALAR
        if k is None:
            raise ValueError("unsupported operand")
        ids[id(v)] = prog.add_input(k, v.type.dtype)
        ext_inputs.append(v)
        return ids[id(v)]

    # inputs first so that their ids are 0 .. n_in - 1
    for n in order:
        for i in n.inputs:
            if id(i) not in produced and not isinstance(i, gof.Constant):
                try:
                    var_id(i)
                except ValueError:
                    return False
    if not any(k == FULL for k in prog.in_kinds):
        return False
    from .opt import _scalar_constant
    for n in order:
        op = n.op
        if isinstance(op, HipElemwise):
            s_in, args = [], []
            s_args = []
            for i in n.inputs:
                c = _scalar_constant(i) if id(i) not in produced else None
                if c is not None:
                    s_args.append(c)
                    continue
                if isinstance(i, gof.Constant) and id(i) not in ids:
                    return False
                s = Scalar(i.type.dtype)()
                s_in.append(s)
                s_args.append(s)
                args.append(var_id(i))
            sop = scal.Composite(s_in, [op.scalar_op(*s_args)]) if len(s_in) != len(n.inputs) else op.scalar_op
            per_elem = any(prog.var[a][0] for a in args)
            if per_elem != (_klass(n.outputs[0], nd, red) == FULL):
                return False
            out = prog.new_var(per_elem, n.outputs[0].type.dtype)
            ids[id(n.outputs[0])] = out
            prog.steps.append(("ew", sop, args, [out]))
        elif isinstance(op, HipCAReduce):
            arg = var_id(n.inputs[0])
            out = prog.new_var(False, op.out_dtypes[0])
            ids[id(n.outputs[0])] = out
            prog.steps.append(("red", op.scalar_ops[0], op.acc_dtypes[0], op.out_dtypes[0], arg, out))
        else:  # keepdims DimShuffle: same per-row value
            ids[id(n.outputs[0])] = ids[id(n.inputs[0])]
    # outputs: island variables used outside
    outs = []
    for n in order:
        for o in n.outputs:
            users = fgraph.clients.get(o, [])
            if any(c == "output" or c not in island for c, _ in users):
                outs.append(o)
    if not outs:
        return False
    out_types = []
    for o in outs:
        kind = FULL if (o.type.ndim == nd and _klass(o, nd, red) == FULL) else ROW
        prog.outputs.append((ids[id(o)], kind, o.type.dtype))
        out_types.append(o.type)
    if len(ext_inputs) + len(outs) > 48:
        return False
    if prog.axes is not None:
        # worth holding the values only for a full-sized result that is computed from reductions of them
        # (statistics alone are one streaming pass of the merged reduction kernels, which is faster)
        prog.source()
        if prog.held_passes < 2 or not any(kind == FULL for _, kind, _ in prog.outputs):
            return False
    # fallback: a private copy of the island
    memo = dict((v, v.type()) for v in ext_inputs)
    inner_in = [memo[v] for v in ext_inputs]
    memo = gof.clone_get_equiv(ext_inputs, outs, copy_inputs=False, memo=memo)
    inner_out = [memo[o] for o in outs]
    new_node = HipRowChain(prog, out_types, (inner_in, inner_out)).make_node(*ext_inputs)
    for o, no in zip(outs, new_node.outputs):
        fgraph.replace(o, no)
    return True
