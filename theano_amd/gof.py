"""Minimal symbolic-graph core carrying Theano's Op / Type / Apply protocol.

Only what the fused Elemwise / CAReduce path needs is here: typed variables,
apply nodes, ops identified by ``__props__``, a function graph with client
tracking and replacement, and a small optimizer driver.  The contract mirrored
is the one documented for Theano ops (``doc/extending/op.txt``: ``make_node``
:50-65, ``perform`` and output-storage reuse :67-109, ``__props__`` :151,
``infer_shape`` :218, ``grad`` :292) and implemented in ``theano/gof/graph.py``
(``Apply`` :50, ``Variable`` :270, ``Constant`` :559), ``theano/gof/op.py:793``
and ``theano/gof/fg.py``.
"""


class MethodNotDefined(NotImplementedError):
    """Raised by optional Op methods that an op does not provide."""


# --------------------------------------------------------------------------
# types and variables
class Type(object):
    """Description of the values a Variable may hold."""

    Variable = None  # set after Variable is defined
    Constant = None

    def filter(self, data, strict=False, allow_downcast=None):
        raise MethodNotDefined("filter", type(self))

    def make_variable(self, name=None):
        return self.Variable(self, name=name)

    def make_constant(self, value, name=None):
        return self.Constant(self, self.filter(value), name=name)

    def __call__(self, name=None):
        return self.make_variable(name)

    def __ne__(self, other):
        return not (self == other)


class Variable(object):
    """A typed node of the graph: either an input (``owner is None``) or the
    ``index``-th output of the Apply node ``owner``."""

    def __init__(self, type, owner=None, index=None, name=None):
        self.type = type
        self.owner = owner
        self.index = index
        self.name = name
        self.tag = {}

    def __str__(self):
        if self.name is not None:
            return self.name
        if self.owner is not None:
            if len(self.owner.outputs) == 1:
                return "%s.out" % self.owner.op
            return "%s.%d" % (self.owner.op, self.index)
        return "<%s>" % self.type

    __repr__ = __str__

    def clone(self):
        v = self.__class__(self.type, None, None, self.name)
        v.tag = dict(self.tag)
        return v


class Constant(Variable):
    """A Variable with a fixed value (``theano/gof/graph.py:559``)."""

    def __init__(self, type, data, name=None):
        Variable.__init__(self, type, None, None, name)
        self.data = data

    def clone(self):
        c = self.__class__(self.type, self.data, self.name)
        c.tag = dict(self.tag)
        return c

    def signature(self):
        return (self.type, repr(self.data))

    def __str__(self):
        if self.name is not None:
            return self.name
        s = str(self.data)
        return "Constant{%s}" % (s if len(s) < 24 else s[:20] + "...")

    __repr__ = __str__


Type.Variable = Variable
Type.Constant = Constant


class Apply(object):
    """One application of an Op to inputs, producing outputs."""

    def __init__(self, op, inputs, outputs):
        self.op = op
        self.inputs = list(inputs)
        self.outputs = list(outputs)
        self.tag = {}
        for i, o in enumerate(self.outputs):
            if o.owner is None:
                o.owner = self
                o.index = i
            elif o.owner is not self:
                raise ValueError("output already owned by another Apply")

    @property
    def nin(self):
        return len(self.inputs)

    @property
    def nout(self):
        return len(self.outputs)

    def default_output(self):
        do = getattr(self.op, "default_output", None)
        if do is None:
            if len(self.outputs) == 1:
                return self.outputs[0]
            raise AttributeError("%s has several outputs and no default_output" % self.op)
        return self.outputs[do]

    out = property(default_output)

    def clone_with_new_inputs(self, inputs, strict=True):
        """Re-apply the op; when input types changed and ``strict`` is False the
        node is rebuilt through ``make_node`` so output types follow."""
        remake = any(new.type != old.type for old, new in zip(self.inputs, inputs))
        if remake and not strict:
            return self.op.make_node(*inputs)
        if remake:
            raise TypeError("clone_with_new_inputs: input types changed")
        node = Apply(self.op, inputs, [o.clone() for o in self.outputs])
        node.tag = dict(self.tag)
        return node

    def __str__(self):
        return "%s(%s)" % (self.op, ", ".join(str(i) for i in self.inputs))

    __repr__ = __str__


# --------------------------------------------------------------------------
# ops
class Op(object):
    """Base class of every operation.

    Subclasses list their defining attributes in ``__props__``; equality, hash
    and ``str`` derive from it (``theano/gof/utils.py:162-210``), which is what
    lets a merge pass and the kernel caches recognise identical ops.
    """

    __props__ = ()
    default_output = None
    view_map = {}
    destroy_map = {}

    def _props(self):
        return tuple(getattr(self, p) for p in self.__props__)

    def __eq__(self, other):
        return type(self) is type(other) and self._props() == other._props()

    def __ne__(self, other):
        return not (self == other)

    def __hash__(self):
        return hash((type(self), self._props()))

    def __str__(self):
        if not self.__props__:
            return type(self).__name__
        return "%s{%s}" % (type(self).__name__, ", ".join("%s=%s" % (p, getattr(self, p)) for p in self.__props__))

    __repr__ = __str__

    # -- graph construction
    def make_node(self, *inputs):
        raise MethodNotDefined("make_node", type(self))

    def __call__(self, *inputs, **kwargs):
        return_list = kwargs.pop("return_list", False)
        node = self.make_node(*inputs, **kwargs)
        if self.default_output is not None:
            rval = node.outputs[self.default_output]
            return [rval] if return_list else rval
        if return_list or len(node.outputs) != 1:
            return list(node.outputs)
        return node.outputs[0]

    # -- execution
    def perform(self, node, inputs, output_storage):
        """Compute outputs from ``inputs`` into ``output_storage`` (a list of
        one-element lists; ``output_storage[i][0]`` may hold a previous result
        that the op is free to reuse)."""
        raise MethodNotDefined("perform", type(self))

    def prepare_node(self, node):
        """Hook run once before the first ``perform`` of ``node``."""

    # -- shape and gradient
    def infer_shape(self, node, input_shapes):
        raise MethodNotDefined("infer_shape", type(self))

    def L_op(self, inputs, outputs, output_grads):
        return self.grad(inputs, output_grads)

    def grad(self, inputs, output_grads):
        raise MethodNotDefined("grad", type(self))

    def R_op(self, inputs, eval_points):
        """Forward-mode derivative: the op's Jacobian times ``eval_points``, one variable (or None) per output
        (``theano/gof/op.py:PureOp.R_op``); an op that has none says so."""
        raise MethodNotDefined("R_op", type(self))

    def connection_pattern(self, node):
        return [[True] * len(node.outputs) for _ in node.inputs]


# --------------------------------------------------------------------------
# graph walks
def ancestors(outputs, blockers=None):
    """All variables reachable from ``outputs`` going up, each once."""
    seen, order = set(), []
    stack = list(outputs)
    blockers = set(id(b) for b in (blockers or ()))
    while stack:
        v = stack.pop()
        if id(v) in seen:
            continue
        seen.add(id(v))
        order.append(v)
        if v.owner is not None and id(v) not in blockers:
            stack.extend(v.owner.inputs)
    return order


def graph_inputs(outputs, blockers=None):
    return [v for v in ancestors(outputs, blockers) if v.owner is None]


def io_toposort(inputs, outputs):
    """Apply nodes needed for ``outputs``, stopping at ``inputs``, in an order
    where every node follows the producers of its inputs."""
    stop = set(id(i) for i in inputs)
    order, state = [], {}
    stack = [(o.owner, False) for o in reversed(outputs) if o.owner is not None and id(o) not in stop]
    while stack:
        node, expanded = stack.pop()
        if node is None or state.get(id(node)) == 2:
            continue
        if expanded:
            state[id(node)] = 2
            order.append(node)
            continue
        if state.get(id(node)) == 1:
            continue
        state[id(node)] = 1
        stack.append((node, True))
        for i in reversed(node.inputs):
            if i.owner is not None and id(i) not in stop and state.get(id(i.owner)) != 2:
                stack.append((i.owner, False))
    return order


def clone_get_equiv(inputs, outputs, copy_inputs=True, memo=None):
    """Clone the sub-graph between ``inputs`` and ``outputs``; returns the map
    from original variables / nodes to their clones."""
    memo = {} if memo is None else memo
    for i in inputs:
        if i not in memo:
            memo[i] = i.clone() if copy_inputs else i
    for node in io_toposort(inputs, outputs):
        for i in node.inputs:
            if i not in memo:  # a free variable or constant not listed in inputs
                memo[i] = i
        new_node = node.clone_with_new_inputs([memo[i] for i in node.inputs])
        memo[node] = new_node
        for o, no in zip(node.outputs, new_node.outputs):
            if o not in memo:       # a variable the caller mapped to something else keeps that mapping
                memo[o] = no
    for o in outputs:
        if o not in memo:
            memo[o] = o.clone() if (copy_inputs and o.owner is None and not isinstance(o, Constant)) else o
    return memo


def clone(inputs, outputs, copy_inputs=True):
    memo = clone_get_equiv(inputs, outputs, copy_inputs)
    return [memo[i] for i in inputs], [memo[o] for o in outputs]


# --------------------------------------------------------------------------
# function graph
class InconsistencyError(Exception):
    pass


class FunctionGraph(object):
    """A closed sub-graph with explicit inputs and outputs that records, for
    every variable, the (node, input index) pairs that consume it, so that
    rewrites can ask "who uses this?" and replace variables in place
    (``theano/gof/fg.py``).  The string 'output' stands for the graph's own
    use of an output variable."""

    import_log = None   # a list while a rewriter wants to know which nodes a replacement brings in

    def __init__(self, inputs, outputs, clone_graph=True):
        if clone_graph:
            inputs, outputs = clone(inputs, outputs)
        self.inputs = list(inputs)
        self.outputs = list(outputs)
        self.clients = {}
        self.apply_nodes = set()
        self.variables = set()
        for i in self.inputs:
            self.variables.add(i)
            self.clients.setdefault(i, [])
        for idx, o in enumerate(self.outputs):
            self._import_var(o)
            self.clients.setdefault(o, []).append(("output", idx))

    # -- bookkeeping
    def _import_var(self, var):
        if var in self.variables:
            return
        if var.owner is None:
            if not isinstance(var, Constant) and var not in self.inputs:
                raise InconsistencyError("undeclared input %s" % var)
            self.variables.add(var)
            self.clients.setdefault(var, [])
            return
        # post-order walk over the producers that are not part of the graph yet
        stack = [(var.owner, False)]
        while stack:
            node, expanded = stack.pop()
            if node in self.apply_nodes:
                continue
            if expanded:
                self._import_node(node)
                continue
            stack.append((node, True))
            for i in node.inputs:
                if i in self.variables:
                    continue
                if i.owner is None:
                    self._import_var(i)
                else:
                    stack.append((i.owner, False))

    def _import_node(self, node):
        """Adds a node whose inputs are all part of the graph (or become so here)."""
        if node in self.apply_nodes:
            return
        for i in node.inputs:
            if i not in self.variables:
                self._import_var(i)
        self.apply_nodes.add(node)
        if self.import_log is not None:
            self.import_log.append(node)
        for o in node.outputs:
            self.variables.add(o)
            self.clients.setdefault(o, [])
        for idx, i in enumerate(node.inputs):
            self.clients.setdefault(i, []).append((node, idx))

    def _prune(self, var):
        """Drop the producer of ``var`` if nothing uses any of its outputs."""
        node = var.owner
        if node is None or node not in self.apply_nodes:
            return
        if any(self.clients.get(o) for o in node.outputs):
            return
        self.apply_nodes.discard(node)
        for o in node.outputs:
            self.variables.discard(o)
            self.clients.pop(o, None)
        for idx, i in enumerate(node.inputs):
            cl = self.clients.get(i, [])
            for k, (n, j) in enumerate(cl):
                if n is node and j == idx:
                    del cl[k]
                    break
            self._prune(i)

    # -- rewriting
    def replace(self, var, new_var):
        if var is new_var:
            return
        if var.type != new_var.type:
            raise TypeError("replace: %s (%s) by %s (%s)" % (var, var.type, new_var, new_var.type))
        if var not in self.variables:
            return
        self._import_var(new_var)
        for node, idx in list(self.clients.get(var, [])):
            if node == "output":
                self.outputs[idx] = new_var
            else:
                node.inputs[idx] = new_var
            self.clients[new_var].append((node, idx))
        self.clients[var] = []
        self._prune(var)

    def replace_all(self, pairs):
        for var, new_var in pairs:
            self.replace(var, new_var)

    def toposort(self):
        return io_toposort(self.inputs, self.outputs)

    def rebuild(self, outputs):
        """A new graph over the same inputs computing ``outputs``."""
        return FunctionGraph(self.inputs, outputs, clone_graph=False)

    def n_clients(self, var):
        return len(self.clients.get(var, []))

    def __str__(self):
        return "[%s]" % ", ".join(str(o) for o in self.outputs)


# --------------------------------------------------------------------------
# optimizer drivers
class LocalOptimizer(object):
    """A rewrite tried on one node: ``transform`` returns False/None or the
    list of replacement outputs."""

    tracks = None  # op classes the rewrite cares about, None = any

    def transform(self, fgraph, node):
        raise MethodNotDefined("transform", type(self))


class FromFunctionLocalOptimizer(LocalOptimizer):
    def __init__(self, fn, tracks=None):
        self.fn = fn
        self.tracks = tuple(tracks) if tracks is not None else None
        self.__name__ = fn.__name__

    def transform(self, fgraph, node):
        if self.tracks is not None and not isinstance(node.op, self.tracks):
            return False
        return self.fn(fgraph, node)

    def __str__(self):
        return self.__name__


def local_optimizer(tracks=None):
    def deco(fn):
        return FromFunctionLocalOptimizer(fn, tracks)
    return deco


def apply_local(fgraph, opts, order="in_to_out", max_passes=64):
    """Apply local rewrites over the whole graph until nothing changes.  Within a
    pass, the nodes a replacement brings in and the consumers of the replaced value
    are visited right away (a chain of rewrites that feed one another does not cost
    one pass per link); a pass that changes nothing ends the loop."""
    changed_any = False
    budget = None
    for _ in range(max_passes):
        changed = False
        nodes = fgraph.toposort()
        if order == "out_to_in":
            nodes.reverse()
        if budget is None:
            budget = 32 * len(nodes) + 512      # rewrites that undo each other must not spin
        nodes.reverse()                          # a stack: the next node is at the end
        while nodes and budget > 0:
            node = nodes.pop()
            if node not in fgraph.apply_nodes:
                continue
            for opt in opts:
                repl = opt.transform(fgraph, node)
                if not repl:
                    continue
                if isinstance(repl, dict):
                    pairs = list(repl.items())
                else:
                    pairs = list(zip(node.outputs, repl))
                fgraph.import_log = fresh = []
                touched = []
                for old, new in pairs:
                    if new is not None:
                        fgraph.replace(old, new)
                        touched.extend(c for c, _ in fgraph.clients.get(new, []) if c != "output")
                fgraph.import_log = None
                again = [n for n in fresh + touched + [node] if n in fgraph.apply_nodes]
                if order == "out_to_in":
                    again.reverse()
                nodes.extend(reversed(again))
                changed = True
                budget -= 1
                break
        changed_any = changed_any or changed
        if not changed:
            break
        if budget <= 0:
            import warnings
            warnings.warn("graph rewriting stopped early: the rewrites keep replacing each other's results")
            break
    return changed_any


def merge_identical(fgraph):
    """Merge nodes that apply equal ops to identical inputs, and equal
    constants (the job of Theano's MergeOptimizer, ``theano/gof/opt.py``)."""
    changed = True
    while changed:
        changed = False
        consts, seen = {}, {}
        for node in fgraph.toposort():
            for idx, i in enumerate(list(node.inputs)):
                if isinstance(i, Constant):
                    try:
                        sig = i.signature()
                    except Exception:
                        continue
                    first = consts.setdefault(sig, i)
                    if first is not i:
                        fgraph.replace(i, first)
                        changed = True
            if getattr(node.op, "destroy_map", None):
                continue
            key = (node.op, tuple(id(i) for i in node.inputs))
            try:
                prev = seen.get(key)
            except TypeError:
                continue
            if prev is None:
                seen[key] = node
            elif prev is not node:
                for o, po in zip(node.outputs, prev.outputs):
                    fgraph.replace(o, po)
                changed = True
    return fgraph
