"""``function``: compile a graph into a callable that runs on the GPU.

The counterpart of ``theano.function`` (``theano/compile/function.py:74``,
``FunctionMaker`` ``theano/compile/function_module.py:1428``) reduced to this
path: clone the graph, run the HIP rewrite pipeline (lift, fuse), order the
nodes, and execute them one ``perform`` call each, releasing intermediate
results after their last use (the loop of ``theano/gof/vm.py:237-305``).
"""
import numpy as np

from . import gof
from .config import config
from .gof import Constant, FunctionGraph, Variable
from .tensor.type import TensorType, as_tensor_variable


class In(object):
    """An input with options (``theano/compile/io.py:40-216``).  ``strict``: the argument must already have
    the input's dtype and rank (no conversion); ``allow_downcast``: conversions that lose precision are
    accepted; ``mutable`` / ``borrow``: permission for the function to overwrite the argument - what
    ``accept_inplace`` graphs do to the arguments their operations destroy, with or without it, as in the
    reference.  Default values and per-input updates (``value=``, ``update=``) belong to shared variables
    here: ``shared(...)`` with ``function(updates=...)``."""

    def __init__(self, variable, name=None, value=None, update=None, mutable=None, strict=False, allow_downcast=None,
                 autoname=True, implicit=None, borrow=None, shared=False):
        if value is not None or update is not None or implicit or shared:
            raise NotImplementedError("In(value=, update=, implicit=, shared=): use a shared variable and "
                                      "function(updates=...)")
        if strict and allow_downcast:
            raise ValueError("In(strict=True) excludes allow_downcast")
        self.variable = variable
        self.name = name or (variable.name if autoname else None)
        self.borrow = bool(borrow) if borrow is not None else bool(mutable)
        self.mutable = bool(mutable) if mutable is not None else self.borrow
        self.strict = bool(strict)
        self.allow_downcast = allow_downcast


class Out(object):
    """``device=True`` leaves the result in GPU memory (a ``HipArray``)."""

    def __init__(self, variable, borrow=False, device=False):
        self.variable = variable
        self.borrow = borrow
        self.device = device


class SharedVariable(Variable):
    """A variable with persistent device storage, an implicit input of every
    function that uses it (``theano/compile/sharedvalue.py``)."""

    def __init__(self, type, value, name=None):
        Variable.__init__(self, type, None, None, name)
        self.container = [value]

    def get_value(self, borrow=False, return_internal_type=False):
        v = self.container[0]
        return v if return_internal_type else v.to_numpy()

    strict, allow_downcast = False, None

    def set_value(self, value, borrow=False):
        self.container[0] = self.type.filter(value, strict=self.strict, allow_downcast=self.allow_downcast)

    def clone(self):
        return self  # shared variables are never copied into a function graph


def shared(value, name=None, strict=False, allow_downcast=None, **kwargs):
    """Device-resident shared variable holding ``value`` (``theano.shared``, ``theano/compile/sharedvalue.py:238-300``;
    the device constructor's keywords ``broadcastable=``, ``borrow=`` and ``target=`` of
    ``theano/gpuarray/type.py:650-700``: the value is always copied to this library's GPU).  ``strict`` and
    ``allow_downcast`` govern later ``set_value`` calls as they govern ``filter``."""
    broadcastable = kwargs.pop("broadcastable", None)
    kwargs.pop("borrow", None)
    kwargs.pop("target", None)
    if kwargs:
        raise TypeError("shared() got unexpected keyword arguments %s" % sorted(kwargs))
    from .hip.ops import HipArrayType, HipArrayVariable
    from .hip.runtime import HipArray
    if isinstance(value, HipArray):
        dtype, shape = str(value.dtype), value.shape
    else:
        value = np.asarray(value)
        dtype, shape = str(value.dtype), value.shape
    if broadcastable is None:
        broadcastable = (False,) * len(shape)
    t = HipArrayType(dtype, broadcastable)

    class _Shared(SharedVariable, HipArrayVariable):
        pass
    sv = _Shared(t, t.filter(value), name=name)
    sv.strict, sv.allow_downcast = bool(strict), allow_downcast
    return sv


class UnusedInputError(Exception):
    """A symbolic input passed to ``function`` is not needed (``theano/compile/function_module.py:34-40``)."""


class NanGuardError(FloatingPointError):
    """A node produced NaN or infinity under ``mode='nan_guard'``."""


class CheckModeError(RuntimeError):
    """``mode='check'`` found an overwritten argument or a result that depends on the rewrites."""


def _guarded(perform):
    """``perform`` followed by a scan of every floating-point result for NaN and infinity: the check of
    ``NanGuardMode`` (``theano/compile/nanguardmode.py:230-300``), after each node as there."""
    def run(node, inputs, outs):
        perform(node, inputs, outs)
        for k, cell in enumerate(outs):
            v = cell[0]
            if v is None or not hasattr(v, "dtype") or np.dtype(v.dtype).kind not in "fc":
                continue
            host = v.to_numpy() if hasattr(v, "to_numpy") else np.asarray(v)
            if host.size and not np.isfinite(host).all():
                what = "NaN" if np.isnan(host).any() else "Inf"
                raise NanGuardError("%s in output %d of %s (inputs: %s)" % (
                    what, k, node, ", ".join("%s%s" % (getattr(i, "dtype", type(i).__name__),
                                                     tuple(getattr(i, "shape", ()))) for i in inputs)))
    return run


class CheckedFunction(object):
    """What ``function(..., mode='check')`` returns: the host-side counterpart of the in-place and
    aliasing checks of ``DebugMode`` (``BadDestroyMap`` / ``BadOptimization``,
    ``theano/compile/debugmode.py:130-330``).  Every call
    (1) runs the same graph compiled without fusion, row chains and in-place operation, one kernel per
        node, on the arguments;
    (2) runs the optimised function;
    (3) raises ``CheckModeError`` if an argument's contents changed (an in-place kernel wrote into an
        array it does not own), or a result or the new value of a shared variable differs between the
        two beyond ``config.check_mode_tolerance`` (integers and booleans: at all).
    Meant for debugging: it costs two runs and copies of every argument and result."""

    def __init__(self, primary, reference, n_updates):
        self.primary, self.reference, self.n_updates = primary, reference, n_updates
        self.maker = primary
        self.fgraph = primary.fgraph

    def toposort(self):
        return self.primary.toposort()

    @staticmethod
    def _host(v):
        return v.to_numpy() if hasattr(v, "to_numpy") else np.array(v)

    def __call__(self, *args):
        before = [self._host(a) for a in args]
        ref = self.reference(*args)
        ref = list(ref) if isinstance(ref, (list, tuple)) else [ref]
        got = self.primary(*args)
        for k, (a, b) in enumerate(zip(args, before)):
            now = self._host(a)
            if now.shape != b.shape or not np.array_equal(now, b, equal_nan=now.dtype.kind in "fc"):
                raise CheckModeError("argument %d (%s) was overwritten by the call" % (k, self.primary.in_specs[k].name))
        outs = list(got) if isinstance(got, (list, tuple)) else [got]
        news = [sv.container[0] for sv in self.primary.update_targets]
        names = ["output %d" % k for k in range(len(outs))] + ["update of %s" % sv for sv in self.primary.update_targets]
        for name, g, r in zip(names, outs + news, ref):
            g, r = self._host(g), self._host(r)
            if g.shape != r.shape or g.dtype != r.dtype:
                raise CheckModeError("%s: %s%s with the rewrites, %s%s without" % (name, g.dtype, g.shape, r.dtype, r.shape))
            if g.dtype.kind in "fc":
                rtol, atol = config.check_mode_tolerance.get(str(g.dtype), (0.0, 0.0))
                ok = np.isclose(g, r, rtol=rtol, atol=atol, equal_nan=True)
            else:
                ok = g == r
            if not np.all(ok):
                bad = tuple(np.argwhere(~np.asarray(ok))[0])
                raise CheckModeError("%s differs between the optimised function and one kernel per node: %d of %d "
                                     "values, first at %s: %r against %r" % (name, int((~ok).sum()), ok.size, bad,
                                                                            g[bad], r[bad]))
        return got


class Function(object):
    """Callable produced by ``function``."""

    def __init__(self, fgraph, in_specs, out_specs, single_output, shared_inputs, update_targets=(), nan_guard=False,
                 writeback=()):
        self.nan_guard = nan_guard
        self.update_targets = list(update_targets)
        # positions of the arguments that take the trailing (hidden) results after each call: what the
        # caller's in-place operations overwrote
        self.writeback = list(writeback)
        self.fgraph = fgraph
        self.maker = self  # so that f.maker.fgraph reads as with the reference
        self.in_specs = in_specs
        self.out_specs = out_specs
        self.single_output = single_output
        self.shared_inputs = shared_inputs
        self.nodes = fgraph.toposort()
        self._prepare()

    def _mark_reuse(self):
        """For every kernel node, the positions of the full-sized inputs that a later kernel of
        this function reads again (``node.tag['reused_in']``) and of the outputs that a later
        kernel reads (``node.tag['reused_out']``).  The ops pass them on as THX_REUSED, which
        keeps those arrays out of non-temporal accesses so that the last-level cache can serve
        the next read (a batch-norm pass over 100 MB of activations after the statistics pass,
        a reduction over an elementwise result that is also an output)."""
        from .hip.ops import HipArrayType

        def root(v):   # the array a chain of views looks at
            while v.owner is not None and getattr(v.owner.op, "view_map", None):
                v = v.owner.inputs[v.owner.op.view_map[0][0]]
            return v

        def big(v):
            return isinstance(v.type, HipArrayType) and v.type.ndim > 0 and not any(v.type.broadcastable)

        kernels = [n for n in self.nodes
                   if type(n.op).__name__ in ("HipElemwise", "HipElemwiseReduce", "HipCAReduce", "HipRowChain", "HipMaxAndArgmax")]
        later = set()
        for node in reversed(kernels):
            node.tag["reused_in"] = tuple(k for k, i in enumerate(node.inputs) if big(i) and id(root(i)) in later)
            node.tag["reused_out"] = tuple(k for k, o in enumerate(node.outputs) if big(o) and id(o) in later)
            later |= set(id(root(i)) for i in node.inputs if big(i))

    def _prepare(self):
        from .hip.opt import DeviceConstant
        from .hip.runtime import HipArray
        # storage cells
        self.storage = {}
        for v in self.fgraph.inputs:
            self.storage[v] = [None]
        self.constants = []
        for node in self.nodes:
            for i in node.inputs:
                if i not in self.storage:
                    if isinstance(i, DeviceConstant):
                        self.storage[i] = [None]
                        self.constants.append(i)
                    elif isinstance(i, Constant):
                        self.storage[i] = [np.asarray(i.data)]
                    elif isinstance(i, SharedVariable):
                        self.storage[i] = i.container
                    else:
                        raise gof.InconsistencyError("%s is used but never computed" % i)
            for o in node.outputs:
                self.storage[o] = [None]
        for o in self.fgraph.outputs:
            if o not in self.storage:
                if isinstance(o, Constant):
                    self.storage[o] = [np.asarray(o.data)]
                elif isinstance(o, SharedVariable):
                    self.storage[o] = o.container
        # last use of every computed variable, for early release
        keep = set(id(o) for o in self.fgraph.outputs)
        last = {}
        for k, node in enumerate(self.nodes):
            for i in node.inputs:
                last[id(i)] = k
        self.release = [[] for _ in self.nodes]
        computed = set()
        for node in self.nodes:
            for o in node.outputs:
                computed.add(id(o))
        by_id = dict((id(v), v) for v in self.storage)
        for vid, k in last.items():
            if vid in computed and vid not in keep:
                self.release[k].append(self.storage[by_id[vid]])
        for k, node in enumerate(self.nodes):
            for o in node.outputs:
                if id(o) not in last and id(o) not in keep:
                    self.release[k].append(self.storage[o])
        self._mark_reuse()
        static = self._shape_only_nodes()
        for k, node in enumerate(self.nodes):      # what such nodes computed is kept between calls
            held = [self.storage[o] for s in static for o in s.outputs]
            self.release[k] = [c for c in self.release[k] if not any(c is h for h in held)]
        self.thunks = []
        for node in self.nodes:
            node.op.prepare_node(node)
            self.thunks.append((_guarded(node.op.perform) if self.nan_guard else node.op.perform, node,
                                [self.storage[i] for i in node.inputs],
                                [self.storage[o] for o in node.outputs], node in static,
                                self.release[len(self.thunks)]))
        self._static_key = None
        self._input_cells = [self.storage[v] for v in self.fgraph.inputs]
        self._constants_ready = False
        self._HipArray = HipArray
        self._last_shape = {}

    def _shape_only_nodes(self):
        """Host nodes whose results depend on nothing but the shapes of the function's arguments: the
        extents ``mean`` divides by (``ShapeFloat``) and host DimShuffles of them.  They run when the
        argument shapes differ from the previous call's and keep their results otherwise: a
        batch-normalisation function holds a dozen of them, each a few microseconds of host time
        that a 20 us kernel does not hide."""
        from .tensor.basic import ShapeFloat
        from .tensor.elemwise import DimShuffle
        from .tensor import views as V
        from .hip.ops import HipDimShuffle, HipElemwise, HipCAReduce, HipMaxAndArgmax, HostToHip, HipToHost
        inputs = set(id(v) for v in self.fgraph.inputs)
        pure = {}

        def shape_pure(v):
            """Is the shape of ``v`` a function of the arguments' shapes alone?"""
            if id(v) in pure:
                return pure[id(v)]
            if v.owner is None:
                res = id(v) in inputs
            else:
                op = v.owner.op
                if isinstance(op, (V.Subtensor, V.IncSubtensor, V.Reshape, V.Alloc)) and len(v.owner.inputs) > (
                        2 if isinstance(op, V.IncSubtensor) else 1):
                    res = False             # extents or indices that are run-time values
                elif isinstance(op, (HostToHip, HipToHost, DimShuffle, HipElemwise, HipCAReduce, HipMaxAndArgmax,
                                     V.Subtensor, V.IncSubtensor, V.Reshape, V.Alloc, V.Rebroadcast)) or (
                                         type(op).__name__ == "HipRowChain"):
                    res = all(shape_pure(i) for i in v.owner.inputs if hasattr(i.type, "ndim"))
                else:
                    res = False
            pure[id(v)] = res
            return res

        static = set()
        for node in self.nodes:
            if isinstance(node.op, ShapeFloat) and shape_pure(node.inputs[0]):
                static.add(node)
            elif (type(node.op) is DimShuffle and node.inputs[0].owner is not None and
                  node.inputs[0].owner in static):
                static.add(node)
        outs = set(id(o) for o in self.fgraph.outputs)
        return set(n for n in static if not any(id(o) in outs for o in n.outputs))

    def _upload_constants(self):
        for c in self.constants:
            self.storage[c][0] = self._HipArray.from_numpy(np.asarray(c.data))
        self._constants_ready = True

    def __call__(self, *args):
        if len(args) != len(self.in_specs):
            raise TypeError("function takes %d arguments, got %d" % (len(self.in_specs), len(args)))
        if not self._constants_ready:
            self._upload_constants()
        HipArray = self._HipArray
        for spec, var, a in zip(self.in_specs, self.fgraph.inputs, args):
            if type(a) is np.ndarray and a.dtype == var.type.numpy_dtype and a.shape == self._last_shape.get(var):
                self.storage[var][0] = a  # same dtype and shape as a value that already passed the full check
                continue
            if isinstance(a, HipArray) and isinstance(var.type, TensorType):
                # device-resident argument for a host-typed input: checked like a host value
                if a.dtype != var.type.numpy_dtype or len(a.shape) != var.type.ndim:
                    raise TypeError("Bad input argument %s: expected %s, got %s" % (spec.name, var.type, a))
                for d, b in enumerate(var.type.broadcastable):
                    if b and a.shape[d] != 1:
                        raise TypeError("Non-unit value on shape on a broadcastable dimension.", a.shape,
                                        var.type.broadcastable)
                self.storage[var][0] = a
            else:
                try:
                    v = self.storage[var][0] = var.type.filter(a, strict=spec.strict, allow_downcast=spec.allow_downcast)
                    if type(v) is np.ndarray:
                        self._last_shape[var] = v.shape
                except TypeError as e:
                    raise TypeError("Bad input argument to theano function with name \"%s\": %s" % (spec.name, e))
        return self._run(args)

    def call_trusted(self, args):
        """The call without the checks of the arguments: for values that already passed them as operands
        of the node this function stands in for (a row chain running its island unfused)."""
        if not self._constants_ready:
            self._upload_constants()
        storage = self.storage
        for var, a in zip(self.fgraph.inputs, args):
            storage[var][0] = a
        return self._run(args)

    def _run(self, args):
        HipArray = self._HipArray
        # the shapes of the values the nodes will read (the filtered arguments: a list has become an array),
        # never those of the raw arguments; a value without a shape never matches
        key = tuple([getattr(c[0], "shape", None) for c in self._input_cells])
        same = key == self._static_key and None not in key
        self._static_key = None                 # stays unset if a node raises half-way
        for perform, node, ins, outs, static, release in self.thunks:
            if static and same:
                continue
            perform(node, [c[0] for c in ins], outs)
            for cell in release:
                cell[0] = None
        self._static_key = key
        results = [self.storage[o][0] for o in self.fgraph.outputs]
        if self.writeback:
            n_keep = len(results) - len(self.writeback)
            self._write_back(args, results[n_keep:])
            results = results[:n_keep]
        if self.update_targets:
            n_out = len(results) - len(self.update_targets)
            new_values = results[n_out:]
            results = results[:n_out]
            held = set(id(s.container[0].buffer) for s in self.shared_inputs)
            held |= set(id(a.buffer) for a in args if isinstance(a, HipArray))
            for sv, val in zip(self.update_targets, new_values):
                if id(val.buffer) in held:   # a view of a shared variable or of an argument: take a private copy
                    val = val.copy()
                sv.container[0] = val
        for v in self.fgraph.inputs:
            self.storage[v][0] = None
        for o in self.fgraph.outputs:
            if o.owner is not None:
                self.storage[o][0] = None
        if self.single_output:
            return results[0]
        return results

    def capture(self, *args):
        """Record one call of this function on device-resident arguments as a HIP graph: returns
        ``(results, graph)``; every ``graph.launch()`` runs the function's kernels again on the same argument
        arrays and writes the same result arrays, at the cost of one launch for the whole sequence.  For
        functions of several small kernels, where the host's work per launch exceeds the kernels' run time.
        The arguments and results must be device arrays (``Out(v, device=True)``): a transfer would wait for
        the device in the middle of the recording.  The graph keeps the arguments and the current values of the
        shared variables alive; a ``set_value`` after the recording is not seen by replays.  The function is run once first, so that its kernels are
        loaded and the shapes it depends on are known; calls that the function makes differently from one
        run to the next (a row chain turned away at run time, say) are recorded as this call made them."""
        from .hip.ops import HipToHost
        from .hip.runtime import capture
        if self.update_targets or self.writeback:
            raise ValueError("capture: a function with updates or in-place arguments changes state on the host")
        if not all(isinstance(a, self._HipArray) for a in args):
            raise TypeError("capture: every argument must be a device array")
        if any(isinstance(n.op, HipToHost) for n in self.nodes):
            raise TypeError("capture: the function copies results to the host; ask for device results, "
                            "Out(v, device=True)")
        self(*args)                         # loads the kernels, warms the pool, runs the shape-only nodes
        with capture() as c:
            results = self(*args)
        # a replay reads the argument arrays and the arrays the shared variables held at this moment
        # (a later set_value puts a new array into the variable, which the recording does not see)
        c.graph.hold(*args)
        c.graph.hold(*[s.container[0] for s in self.shared_inputs])
        return results, c.graph

    def _write_back(self, args, values):
        """Store each hidden result into the argument its operation overwrites: a device argument takes a
        device copy (whatever its strides), a writable host array of the input's dtype takes the values;
        an argument that had to be converted on the way in was copied then, and stays as it is - as with
        the reference, whose ``filter`` makes that copy."""
        from .hip.views import copy_into
        for k, val in zip(self.writeback, values):
            a = args[k]
            if isinstance(a, self._HipArray):
                if a.shape != val.shape:
                    raise ValueError("in-place result has shape %s, argument %d has %s" % (val.shape, k, a.shape))
                if val.size and not val.buffer.fake:
                    copy_into(val, a)
            elif type(a) is np.ndarray and a.dtype == val.dtype and a.shape == val.shape and a.flags.writeable:
                a[...] = val.to_numpy()

    def toposort(self):
        return list(self.nodes)


def function(inputs, outputs=None, mode=None, updates=None, givens=None, no_default_updates=False, accept_inplace=False,
             name=None, rebuild_strict=True, allow_input_downcast=None, profile=None, on_unused_input=None, *,
             fuse=True, rowchain=True, inplace=True):
    """Compile ``outputs`` as a function of ``inputs``: the arguments of ``theano.function`` in its order
    (``theano/compile/function.py:74-77``), then this package's own switches, by keyword only.
    ``no_default_updates`` and ``rebuild_strict`` are accepted for that order's sake (shared variables here have
    no default updates, and replacements in ``givens`` must keep the type); ``profile`` must stay unset -
    ``theano_amd.hip.runtime.profile`` times the kernels of any call.  ``on_unused_input``: 'raise' (the
    default, None), 'warn' or 'ignore'.

    ``inputs``: variables or ``In`` instances.  A host-typed input may be given
    a ``HipArray`` at call time, which skips the upload.  ``outputs``: a
    variable, ``Out`` or a list of those; ``Out(v, device=True)`` leaves the
    result on the GPU.  ``updates``: pairs (or a dict) of shared variable and
    the expression whose value replaces its content after each call, as in
    ``theano.function`` (``theano/compile/pfunc.py:60-230``).  ``givens``: pairs (or a
    dict) of a variable and the expression of the same type that stands for it in this
    function, e.g. ``{x: data[i * n:(i + 1) * n]}`` with ``data`` shared and ``i`` an
    input (``theano/compile/pfunc.py:365-420``).  Every op must
    have a HIP implementation.  ``fuse=False``
    keeps one kernel per graph node; ``rowchain=False`` keeps elementwise /
    row-reduction islands as separate fused kernels; ``inplace=False`` gives
    every elementwise result a buffer of its own.  ``mode``: None, ``'nan_guard'`` (every node's
    floating-point results are scanned for NaN / infinity, ``NanGuardError``) or ``'check'`` (see
    ``CheckedFunction``: arguments must come back unchanged and results must not depend on fusion or
    in-place operation).  ``allow_input_downcast``: arguments of plain (non-``In``) inputs may be converted
    with loss of precision, e.g. float64 values for a float32 input.  ``accept_inplace``: the graph may hold operations that overwrite an operand
    (``theano.tensor.inplace``); without it such a graph is refused, as in the reference
    (``theano/compile/function_module.py:183-190``) - see ``_functional_form`` for how they run."""
    from .hip import opt as hip_opt
    from .hip.ops import HipArrayType, as_hip_variable

    in_specs = [i if isinstance(i, In) else In(i, allow_downcast=allow_input_downcast) for i in inputs]
    if outputs is None:
        outputs = []
    single = not isinstance(outputs, (list, tuple))
    out_list = [outputs] if single else list(outputs)
    out_specs = [o if isinstance(o, Out) else Out(o) for o in out_list]
    out_vars = []
    for spec in out_specs:
        v = spec.variable
        if not isinstance(v, Variable):
            v = as_tensor_variable(v)
        if spec.device and isinstance(v.type, TensorType):
            v = as_hip_variable(v)
        out_vars.append(v)
    # updates: new values of shared variables, computed with the outputs and stored after the call
    # (theano/compile/pfunc.py:60-230); each must have the type of the variable it replaces
    update_targets = []
    if updates:
        pairs = list(updates.items()) if isinstance(updates, dict) else list(updates)
        for sv, new in pairs:
            if not isinstance(sv, SharedVariable):
                raise TypeError("update target must be a shared variable", sv)
            if sv in update_targets:
                raise ValueError("this shared variable already has an update expression", sv)
            if not isinstance(new, Variable):
                new = as_tensor_variable(new)
            if isinstance(new.type, TensorType):
                new = as_hip_variable(new)
            if new.type != sv.type:
                raise TypeError("an update must have the same type as the original shared variable "
                                "(shared_var=%s, shared_var.type=%s, update_val=%s, update_val.type=%s)"
                                % (sv, sv.type, new, new.type))
            update_targets.append(sv)
            out_vars.append(new)
    if givens:
        pairs = list(givens.items()) if isinstance(givens, dict) else list(givens)
        swap = {}
        for var, rep in pairs:
            if not isinstance(rep, Variable):
                rep = as_tensor_variable(rep)
            vt, rt = var.type, rep.type
            if vt != rt:        # also a device-typed variable for a host-typed one: as_tensor_variable(shared) converts
                raise TypeError("Cannot use a shared variable or expression of type %s as a replacement for a "
                                "variable of type %s in givens" % (rt, vt))
            swap[var] = rep
        memo = gof.clone_get_equiv([], out_vars, copy_inputs=False, memo=dict(swap))
        out_vars = [memo[v] for v in out_vars]
    in_vars = [s.variable for s in in_specs]
    shared_inputs = [v for v in gof.graph_inputs(out_vars) if isinstance(v, SharedVariable)]
    used = set(id(v) for v in gof.graph_inputs(out_vars))
    if on_unused_input is None:
        on_unused_input = "raise"
    if on_unused_input not in ("raise", "warn", "ignore"):
        raise ValueError("Invalid value for keyword on_unused_input of theano.function: '%s'.\nValid values are "
                         "'raise', 'warn', and 'ignore'." % on_unused_input)
    if profile:
        raise NotImplementedError("function(profile=...): use theano_amd.hip.runtime.profile() around the calls")
    if on_unused_input != "ignore":
        for k, v in enumerate(in_vars):
            if id(v) not in used:
                msg = ("theano.function was asked to create a function computing outputs given certain inputs, but "
                       "the provided input variable at index %i is not part of the computational graph needed to "
                       "compute the outputs: %s.\n" % (k, v))
                if on_unused_input == "warn":
                    import warnings
                    warnings.warn(msg + "To make this warning into an error, you can pass the parameter "
                                  "on_unused_input='raise' to theano.function. To disable it completely, use "
                                  "on_unused_input='ignore'.", stacklevel=2)
                else:
                    raise UnusedInputError(msg + "To make this error into a warning, you can pass the parameter "
                                           "on_unused_input='warn' to theano.function. To disable it completely, "
                                           "use on_unused_input='ignore'.")
    # clone everything except shared variables
    memo = dict((s, s) for s in shared_inputs)
    memo = gof.clone_get_equiv(in_vars, out_vars, copy_inputs=True, memo=memo)
    c_in = [memo[v] for v in in_vars]
    c_out = [memo[v] for v in out_vars]
    fgraph = _SharedAwareGraph(c_in, c_out, shared_inputs)
    if mode not in (None, "nan_guard", "check"):
        raise ValueError("mode must be None, 'nan_guard' or 'check'", mode)
    destroyers = [n for n in fgraph.toposort() if getattr(n.op, "destroy_map", None)]
    writeback = []
    if destroyers:
        if not accept_inplace:
            raise TypeError("Graph must not contain inplace operations", destroyers[0], destroyers[0].op)
        fgraph, writeback = _functional_form(fgraph, destroyers, shared_inputs)
        if writeback and mode == "check":
            raise ValueError("mode='check' verifies that a call leaves its arguments alone; this graph overwrites "
                             "argument %d in place" % writeback[0])
    fgraph = hip_opt.optimize(fgraph, fuse=fuse, rowchain=rowchain, inplace=inplace)
    primary = Function(fgraph, in_specs, out_specs, single, shared_inputs, update_targets, nan_guard=mode == "nan_guard",
                       writeback=writeback)
    if mode != "check":
        return primary
    # the same outputs and new shared values, as plain results of a function without the rewrites
    ref_outs = [Out(v, device=spec.device) for v, spec in zip(out_vars, out_specs)]
    ref_outs += [Out(v, device=True) for v in out_vars[len(out_specs):]]
    reference = function(in_specs, ref_outs, givens=None, fuse=False, rowchain=False, inplace=False,
                         on_unused_input="ignore", accept_inplace=accept_inplace)
    return CheckedFunction(primary, reference, len(update_targets))


def _functional_form(fgraph, destroyers, shared_inputs):
    """Graphs with the user's in-place elementwise operations (``theano.tensor.inplace``), made safe to
    reorder and fuse: every such node is replaced by the same scalar operation writing a buffer of its
    own, so that whatever else reads the overwritten variable reads its old value - the order the
    reference's DestroyHandler forces (``theano/gof/destroyhandler.py``).  Where the overwritten variable
    is an argument of the function the new result becomes one more (hidden, device) output that
    ``Function`` stores into the argument after the call; an intermediate result that is overwritten
    cannot be observed and needs nothing.  As in the reference, constants and shared variables are
    protected and one variable takes one destroyer.  Returns the rebuilt graph and, per hidden output in
    order, the position of the argument that receives it."""
    from .hip.ops import as_hip_variable
    from .tensor.elemwise import Elemwise

    def root(v):
        seen_view = False
        while v.owner is not None and getattr(v.owner.op, "view_map", None):
            v = v.owner.inputs[v.owner.op.view_map[0][0]]
            seen_view = True
        return v, seen_view

    shared = set(id(v) for v in shared_inputs)
    taken = set()
    origin = {}       # id(result written over an argument's buffer) -> position of that argument
    final = {}        # position of an argument -> the last result written over it (chains of in-place nodes)
    for node in destroyers:
        if not isinstance(node.op, Elemwise):
            raise NotImplementedError("in-place operation %s" % node.op)
        new = Elemwise(node.op.scalar_op, name=node.op.name).make_node(*node.inputs)
        for o, idxs in node.op.destroy_map.items():
            victim, through_view = root(node.inputs[idxs[0]])
            if isinstance(victim, Constant) or id(victim) in shared:
                raise gof.InconsistencyError("Trying to destroy a protected Variable.", victim)
            if id(victim) in taken:
                raise gof.InconsistencyError("Multiple destroyers of %s" % victim)
            taken.add(id(victim))
            pos = fgraph.inputs.index(victim) if victim in fgraph.inputs else origin.get(id(victim))
            if pos is not None:
                if through_view:
                    raise NotImplementedError("in-place operation on a view of a function argument (%s)" % node.op)
                origin[id(new.outputs[o])] = pos
                final[pos] = new.outputs[o]
        for o, no in zip(node.outputs, new.outputs):
            fgraph.replace(o, no)
    writeback = sorted(final)
    if writeback:
        fgraph = fgraph.rebuild(list(fgraph.outputs) + [as_hip_variable(final[pos]) for pos in writeback])
    return fgraph, writeback


class _SharedAwareGraph(FunctionGraph):
    """FunctionGraph that accepts shared variables as undeclared inputs."""

    def __init__(self, inputs, outputs, shared_inputs):
        self._shared = set(id(s) for s in shared_inputs)
        FunctionGraph.__init__(self, inputs, outputs, clone_graph=False)

    def rebuild(self, outputs):
        g = _SharedAwareGraph.__new__(_SharedAwareGraph)
        g._shared = self._shared
        FunctionGraph.__init__(g, self.inputs, outputs, clone_graph=False)
        return g

    def _import_var(self, var):
        if var.owner is None and id(var) in self._shared:
            self.variables.add(var)
            self.clients.setdefault(var, [])
            return
        FunctionGraph._import_var(self, var)
