"""Reverse-mode differentiation over the graph: ``grad(cost, wrt)``.

A reduced form of ``theano/gradient.py`` (``grad`` :414, ``_populate_grad_dict``
:977-1430): walk the nodes between ``wrt`` and ``cost`` from the cost down,
ask every op for ``L_op(inputs, outputs, output_grads)`` and accumulate the
terms per variable.
"""
import numpy as np

from . import gof
from . import scalar as scal
from .config import config
from .scalar import DisconnectedType


class DisconnectedInputError(ValueError):
    pass


class NullTypeGradError(TypeError):
    """The gradient asked for runs through a term an op declared not implemented or undefined."""


class NullType(gof.Type):
    """Type of the placeholder an ``L_op`` returns for a gradient it cannot give
    (``theano/gof/null_type.py``): no value, only a reason."""

    def __init__(self, why_null="(no default value given)"):
        self.why_null = why_null

    def filter(self, data, strict=False, allow_downcast=None):
        raise ValueError("No values may be assigned to a NullType")

    def __eq__(self, other):
        return type(self) == type(other)

    def __hash__(self):
        return hash(type(self))

    def __str__(self):
        return "NullType"


def grad_not_implemented(op, x_pos, x, comment=""):
    """What an ``L_op`` returns for input ``x_pos`` when that gradient is not implemented
    (``theano/gradient.py:1995-2034``); asking for it raises NullTypeGradError."""
    return NullType("This variable is Null because the grad method for input %s (%s) of the %s op is not "
                    "implemented. %s" % (x_pos, x, op, comment))()


def grad_undefined(op, x_pos, x, comment=""):
    """Same, for a gradient that is mathematically undefined (``theano/gradient.py:2037-2074``)."""
    return NullType("This variable is Null because the grad method for input %s (%s) of the %s op is "
                    "mathematically undefined. %s" % (x_pos, x, op, comment))()


def grad(cost, wrt, consider_constant=None, disconnected_inputs="raise", add_names=True, known_grads=None,
         return_disconnected="zero", null_gradients="raise"):
    """Symbolic gradient of the 0-d ``cost`` with respect to ``wrt`` (a variable, a list or a tuple of
    variables), with the arguments of ``theano.grad`` (``theano/gradient.py:414-628``):

    ``consider_constant``: expressions nothing is propagated through.  ``disconnected_inputs``: what happens
    when an element of ``wrt`` is not part of the graph of the cost, or only reaches it through operands an op
    declares unconnected (``connection_pattern``) - ``'raise'`` DisconnectedInputError, ``'warn'`` or
    ``'ignore'``; in the last two cases ``return_disconnected`` says what comes back: ``'zero'``, ``'None'`` or
    ``'Disconnected'`` (a variable of DisconnectedType).  A variable that reaches the cost only through
    integer-valued results is connected, with a gradient of zeros.  ``known_grads``: gradients given for
    variables of the graph (``cost`` may then be None).  ``null_gradients``: ``'raise'`` NullTypeGradError for a
    gradient an op declared undefined or not implemented, or ``'return'`` the NullType variable.
    ``add_names``: a named cost and a named variable name their gradient ``(dcost/dvar)``."""
    import warnings
    from .tensor import basic as T
    from .tensor.type import as_tensor_variable

    if disconnected_inputs not in ("ignore", "warn", "raise"):
        raise ValueError("Invalid value for keyword 'disconnected_inputs', valid values are 'ignore', 'warn' and "
                         "'raise'.")
    if return_disconnected not in ("zero", "None", "Disconnected"):
        raise ValueError("Invalid value for keyword 'return_disconnected', valid values are 'zero', 'None' and "
                         "'Disconnected'.")
    if null_gradients not in ("raise", "return"):
        raise ValueError("Invalid value for keyword 'null_gradients', valid values are 'raise' and 'return'.")
    if cost is None and known_grads is None:
        raise AssertionError("cost and known_grads can't both be None.")
    if cost is not None and isinstance(cost.type, NullType):
        raise ValueError("Can't differentiate a NaN cost. cost is NaN because " + cost.type.why_null)
    as_tuple = isinstance(wrt, tuple)
    single = not isinstance(wrt, (list, tuple))
    wrt_list = [wrt] if single else list(wrt)
    for w in wrt_list:
        if not isinstance(w, gof.Variable):
            raise TypeError("Expected Variable, got %s of type %s" % (w, type(w)))
    constant = set(id(v) for v in (consider_constant or ()))
    grads = {}
    if cost is not None:
        if cost.type.ndim != 0:
            raise TypeError("cost must be a scalar.")
        # an integer-valued cost has zero gradients everywhere (theano/gradient.py:_float_ones_like)
        grads[cost] = (T.ones_like(cost) if cost.type.dtype in scal.continuous_dtypes
                       else T.ones_like(cost, dtype=config.floatX))
    for var, g in (known_grads or {}).items():
        g = as_tensor_variable(g) if not isinstance(g, gof.Variable) else g
        if not isinstance(g.type, (NullType, DisconnectedType)) and g.type.dtype not in scal.continuous_dtypes:
            raise TypeError("Gradients must always be NullType, DisconnectedType, or continuous, but grad was given "
                            "a known_grad of type " + str(g.type))
        grads[var] = g
    outputs = list(grads.keys())

    # nodes on a path from wrt to the outputs; nothing is computed "from" an expression held constant
    order = gof.io_toposort([], outputs)
    depends = set(id(w) for w in wrt_list)
    for node in order:
        if any(id(i) in depends for i in node.inputs):
            for o in node.outputs:
                if id(o) not in constant:       # a gradient may arrive at such an expression, none goes through it
                    depends.add(id(o))
    # variables with a path to an output (one whose gradient is not given as disconnected) along which every op
    # declares its operand connected
    connected = set(id(o) for o in outputs if not isinstance(grads[o].type, DisconnectedType))
    for node in reversed(order):
        hit = [k for k, o in enumerate(node.outputs) if id(o) in connected and id(o) not in constant]
        if not hit:
            continue
        pattern = node.op.connection_pattern(node)
        for k, i in enumerate(node.inputs):
            if any(pattern[k][o] for o in hit):
                connected.add(id(i))

    for node in reversed(order):
        if not any(id(o) in depends for o in node.outputs):
            continue
        ograds = []
        live = False
        null = None
        for o in node.outputs:
            g = grads.get(o) if id(o) not in constant else None
            if g is None or isinstance(g.type, DisconnectedType):
                ograds.append(DisconnectedType()())
            else:
                live = True
                ograds.append(g)
                if isinstance(g.type, NullType):
                    null = g
        if not live:
            continue
        if null is not None:
            # nothing can be said about what lies behind an unknown gradient
            for i in node.inputs:
                if id(i) in depends:
                    grads[i] = null
            continue
        if len(node.outputs) == 1 and getattr(node.outputs[0].type, "dtype", "float32") not in scal.continuous_dtypes:
            # integer-valued results carry no gradient to their inputs
            continue
        # replace missing output grads by zeros for ops that cannot take placeholders
        ograds = [T.zeros_like(o) if isinstance(g.type, DisconnectedType) and len(node.outputs) > 1 else g
                  for o, g in zip(node.outputs, ograds)]
        # the gradient of a floating-point result enters the op in that result's own dtype
        # (theano/gradient.py:1107-1115): what flows back to a float32 variable stays float32
        ograds = [g.astype(o.type.dtype) if (hasattr(g.type, "dtype") and getattr(o.type, "dtype", None) is not None and
                                             o.type.dtype not in scal.discrete_dtypes and g.type.dtype != o.type.dtype)
                  else g for o, g in zip(node.outputs, ograds)]
        try:
            igrads = node.op.L_op(node.inputs, node.outputs, ograds)
        except gof.MethodNotDefined:
            raise NotImplementedError("%s does not define a gradient" % node.op)
        if len(igrads) != len(node.inputs):
            raise ValueError("%s.L_op returned %d gradients for %d inputs" % (node.op, len(igrads), len(node.inputs)))
        for i, g in zip(node.inputs, igrads):
            if g is None or isinstance(g.type, DisconnectedType):
                continue
            if id(i) not in depends:
                continue
            if isinstance(g.type, NullType):
                grads[i] = g
                continue
            if i in grads and isinstance(grads[i].type, NullType):
                continue
            if g.type.dtype not in scal.continuous_dtypes:
                continue
            if hasattr(i.type, "broadcastable") and g.type.broadcastable != i.type.broadcastable:
                g = _match_broadcast(g, i)
            grads[i] = g if i not in grads or isinstance(grads[i].type, DisconnectedType) else T.add(grads[i], g)

    result = []
    for w in wrt_list:
        g = grads.get(w)
        if g is not None and isinstance(g.type, NullType):
            if null_gradients == "raise":
                raise NullTypeGradError("tensor.grad encountered a NaN. " + g.type.why_null)
            result.append(g)
            continue
        if g is None or isinstance(g.type, DisconnectedType):
            float_zeros = lambda: T.zeros_like(                                             # noqa: E731
                w, dtype=w.type.dtype if w.type.dtype in scal.continuous_dtypes else config.floatX)
            if id(w) in connected and g is None:
                g = float_zeros()               # reaches the cost, through integer-valued results only
            else:
                message = ("grad method was asked to compute the gradient with respect to a variable that is not "
                           "part of the computational graph of the cost, or is used only by a non-differentiable "
                           "operator: %s" % w)
                if disconnected_inputs == "raise":
                    raise DisconnectedInputError(message)
                if disconnected_inputs == "warn":
                    warnings.warn(message, stacklevel=2)
                g = (float_zeros() if return_disconnected == "zero" else None if return_disconnected == "None"
                     else DisconnectedType()())
        elif add_names and cost is not None and cost.name is not None and w.name is not None:
            g.name = "(d%s/d%s)" % (cost.name, w.name)
        result.append(g)
    if single:
        return result[0]
    return tuple(result) if as_tuple else result


def Lop(f, wrt, eval_points, consider_constant=None, disconnected_inputs="raise"):
    """L operator: eval_points times the Jacobian of ``f`` with respect to
    ``wrt`` (``theano/gradient.py:348-411``): reverse mode seeded with
    ``eval_points`` as the gradients of ``f``."""
    fs = list(f) if isinstance(f, (list, tuple)) else [f]
    eps = list(eval_points) if isinstance(eval_points, (list, tuple)) else [eval_points]
    if len(fs) != len(eps):
        raise ValueError("Lop needs one evaluation point per element of f")
    return grad(None, wrt, known_grads=dict(zip(fs, eps)), consider_constant=consider_constant,
                disconnected_inputs=disconnected_inputs)


def Rop(f, wrt, eval_points, disconnected_outputs="raise", return_disconnected="zero"):
    """R operator: the Jacobian of ``f`` with respect to ``wrt`` times
    ``eval_points`` (``theano/gradient.py:155-345``).  Forward mode: every node
    between ``wrt`` and ``f`` is asked for ``R_op(inputs, eval_points)``;
    graph inputs outside ``wrt`` contribute zeros."""
    from .tensor import basic as T
    from .tensor.type import as_tensor_variable

    single = not isinstance(f, (list, tuple))
    fs = [f] if single else list(f)
    wrt = list(wrt) if isinstance(wrt, (list, tuple)) else [wrt]
    eval_points = list(eval_points) if isinstance(eval_points, (list, tuple)) else [eval_points]
    if len(wrt) != len(eval_points):
        raise ValueError("Rop needs one evaluation point per element of wrt")
    eval_points = [as_tensor_variable(e) for e in eval_points]
    for k, (w, e) in enumerate(zip(wrt, eval_points)):
        if w.type.ndim != e.type.ndim:
            raise ValueError("Element %d of wrt/eval_point have mismatched dimensionality: %d versus %d"
                             % (k, w.type.ndim, e.type.ndim))
    point_of = dict((id(w), e) for w, e in zip(wrt, eval_points))
    seen = {}

    for node in gof.io_toposort([], fs):
        if any(id(o) in point_of for o in node.outputs) and all(id(o) in point_of for o in node.outputs):
            continue
        local = []
        for inp in node.inputs:
            if id(inp) in point_of:
                pt = point_of[id(inp)]
            elif inp.owner is None:
                pt = T.zeros_like(inp) if hasattr(inp.type, "broadcastable") else None
            else:
                pt = seen[id(inp.owner)][inp.owner.outputs.index(inp)]
            if pt is not None and hasattr(inp.type, "dtype") and pt.type.dtype != inp.type.dtype:
                pt = T.cast(pt, inp.type.dtype)
            local.append(pt)
        try:
            seen[id(node)] = node.op.R_op(node.inputs, local)
        except gof.MethodNotDefined:
            raise NotImplementedError("%s does not define R_op" % node.op)

    result = []
    for out in fs:
        if id(out) in point_of:
            result.append(point_of[id(out)])
            continue
        r = seen[id(out.owner)][out.owner.outputs.index(out)] if out.owner is not None else None
        if r is None:
            message = ("Rop method was asked to compute the gradient with respect to a variable that is not part of "
                       "the computational graph of variables in wrt, or is used only by a non-differentiable "
                       "operator: %s" % out)
            if disconnected_outputs == "raise":
                raise DisconnectedInputError(message)
            if disconnected_outputs == "warn":
                import warnings
                warnings.warn(message, stacklevel=2)
            elif disconnected_outputs != "ignore":
                raise ValueError("Invalid value for keyword 'disconnected_inputs', valid values are 'ignore', 'warn' "
                                 "and 'raise'.")
            how = return_disconnected.lower()
            if how not in ("zero", "none", "disconnected"):
                raise ValueError("Invalid value for keyword 'return_disconnected', valid values are 'zero', 'None' "
                                 "and 'Disconnected'.")
            r = T.zeros_like(out) if how == "zero" else None if how == "none" else DisconnectedType()()
        result.append(r)
    return result[0] if single else result


def _match_broadcast(g, var):
    """Make the gradient's static broadcast pattern equal to the variable's."""
    from .tensor import basic as T
    gb, vb = g.type.broadcastable, var.type.broadcastable
    if len(gb) != len(vb):
        raise ValueError("gradient of %s has rank %d, the variable has rank %d" % (var, len(gb), len(vb)))
    to_sum = [k for k, (a, b) in enumerate(zip(gb, vb)) if b and not a]
    if to_sum:
        g = T.sum(g, axis=to_sum, keepdims=True)
    if g.type.broadcastable != vb:
        # the gradient is broadcastable where the variable is not: expand it
        g = T.second(var, g)
    return g


def numeric_grad(f, pts, eps=None):
    """Central finite differences of the scalar function ``f`` at the list of
    float64 arrays ``pts`` (the check used by ``verify_grad``,
    ``theano/gradient.py:1435-1800``)."""
    pts = [np.array(p, dtype="float64") for p in pts]
    out = []
    for k, p in enumerate(pts):
        g = np.zeros_like(p)
        flat, gflat = p.reshape(-1), g.reshape(-1)
        for j in range(flat.size):
            old = flat[j]
            h = eps or 1e-6 * max(1.0, abs(old))
            flat[j] = old + h
            fp = f(*pts)
            flat[j] = old - h
            fm = f(*pts)
            flat[j] = old
            gflat[j] = (fp - fm) / (2 * h)
        out.append(g)
    return out


# ---- verify_grad (theano/gradient.py:1420-1830) ---------------------------------------------------
TYPE_EPS = {"float64": 1e-7, "float32": 3e-4, "float16": 1e-1}       # finite-difference steps, per dtype


class GradientError(Exception):
    """A gradient was computed, but it is not the finite-difference one."""

    def __init__(self, arg, err_pos, shape, val1, val2, abs_err, rel_err, abs_tol, rel_tol):
        Exception.__init__(self)
        self.arg, self.err_pos, self.shape, self.val1, self.val2 = arg, err_pos, shape, val1, val2
        self.abs_err, self.rel_err, self.abs_tol, self.rel_tol = abs_err, rel_err, abs_tol, rel_tol

    def __str__(self):
        return ("GradientError: numeric gradient and analytic gradient exceed tolerance:\n"
                "        At position %i of argument %i with shape %s,\n"
                "            val1 = %f      ,  val2 = %f\n"
                "            abs. error = %f,  abs. tolerance = %f\n"
                "            rel. error = %f,  rel. tolerance = %f\n%s" % (
                    self.err_pos, self.arg, self.shape, self.val1, self.val2, self.abs_err, self.abs_tol,
                    self.rel_err, self.rel_tol, ", ".join(str(a) for a in self.args)))


def _one_sided_grad(f, pts, eps):
    """Forward differences of the scalar function ``f`` with one step size for every element, computed in
    the widest dtype among ``pts`` (``numeric_grad.__init__``, ``theano/gradient.py:1437-1530``)."""
    wide = max((p.dtype for p in pts), key=lambda d: d.itemsize)
    pts = [np.array(p, dtype=wide) for p in pts]
    f0 = float(f(*pts))
    out = []
    for p in pts:
        g = np.zeros(p.shape, wide)
        flat, gflat = p.reshape(-1), g.reshape(-1)
        for j in range(flat.size):
            old = flat[j]
            flat[j] = old + eps
            gflat[j] = (float(f(*pts)) - f0) / eps
            flat[j] = old
        out.append(g)
    return out


def _abs_rel_err(a, b):
    """|a - b| and |a - b| / max(|a| + |b|, 1e-8) (``numeric_grad.abs_rel_err``, :1532-1557)."""
    a, b = np.asarray(a, "float64"), np.asarray(b, "float64")
    abs_err = abs(a - b)
    return abs_err, abs_err / np.maximum(abs(a) + abs(b), 1e-8)


def _max_err(analytic, numeric, abs_tol, rel_tol):
    """The element where min(abs_err / abs_tol, rel_err / rel_tol) is largest over all arguments: (argument,
    flat position, abs_err, rel_err) there (``numeric_grad.max_err``, :1579-1611)."""
    best = None
    for k, (a, b) in enumerate(zip(analytic, numeric)):
        if np.shape(a) != np.shape(b):
            raise ValueError("argument element %i has wrong shape %s" % (k, (np.shape(a), np.shape(b))))
        abs_err, rel_err = _abs_rel_err(a, b)
        if not np.all(np.isfinite(abs_err)):
            raise ValueError("abs_err not finite", repr(abs_err))
        if not np.all(np.isfinite(rel_err)):
            raise ValueError("rel_err not finite", repr(rel_err))
        if abs_err.size == 0:
            continue
        scaled = np.minimum(abs_err / abs_tol, rel_err / rel_tol).reshape(-1)
        j = int(scaled.argmax())
        if best is None or scaled[j] > best[0]:
            best = (scaled[j], k, j, abs_err.reshape(-1)[j], rel_err.reshape(-1)[j])
    if best is None:
        return 0, 0, 0.0, 0.0
    return best[1:]


_GRAD_TOL = {"float16": 5e-2, "float32": 1e-2, "float64": 1e-4}      # absolute and relative, per dtype


class _GradientCheck(object):
    """The device functions one gradient check needs: the cost ``sum(direction * fun(*args))`` with the
    direction a shared array that each round replaces, and the symbolic gradient of that cost."""

    def __init__(self, fun, values, mode, direction_dtype):
        from . import compile as C
        from .tensor import basic as T
        from .tensor.type import TensorType
        self.values = values
        args = [TensorType(str(v.dtype), tuple(n == 1 for n in v.shape))(name="input %i" % k)
                for k, v in enumerate(values)]
        result = fun(*args)
        if isinstance(result, (list, tuple)):
            raise NotImplementedError("verify_grad checks functions of one result; this one returns %d" % len(result))

        def compiled(outputs):
            return C.function([C.In(a, allow_downcast=True) for a in args], outputs, on_unused_input="ignore",
                              accept_inplace=True, mode=mode)

        shape = np.shape(compiled(result)(*self.fresh()))
        self.dtype = direction_dtype or ("float32" if result.type.dtype == "float32" and direction_dtype is False
                                         else "float64")
        self.shape = shape
        self.direction = C.shared(np.ones(shape, self.dtype), name="random_projection",
                                  broadcastable=tuple(result.type.broadcastable))
        cost = T.sum(self.direction * result)
        self.cost = compiled(cost)
        self.gradient = compiled(grad(cost, args, disconnected_inputs="ignore"))

    def fresh(self):
        return [v.copy() for v in self.values]

    def new_direction(self, rng):
        draw = rng.random_sample if hasattr(rng, "random_sample") else rng.random
        self.direction.set_value(np.asarray(draw(self.shape) + 0.5, dtype=self.dtype))

    def worst(self, step, abs_tol, rel_tol):
        """(argument, flat position, analytic value, numeric value, abs error, rel error) of the element that
        is farthest outside the tolerances."""
        numeric = _one_sided_grad(self.cost, self.fresh(), step)
        analytic = self.gradient(*self.fresh())
        k, j, abs_err, rel_err = _max_err(analytic, numeric, abs_tol, rel_tol)
        return (k, j, np.shape(analytic[k]), np.asarray(analytic[k]).reshape(-1)[j], numeric[k].reshape(-1)[j],
                abs_err, rel_err)


def verify_grad(fun, pt, n_tests=2, rng=None, eps=None, out_type=None, abs_tol=None, rel_tol=None, mode=None,
                cast_to_output_type=False, no_debug_ref=True):
    """Check the symbolic gradient of ``fun`` (a function of symbolic tensors returning one tensor, or an
    op) at the list of floating-point arrays ``pt`` against forward differences, with the reference's
    acceptance rule (``theano/gradient.py:1625-1800``): the result is projected on a random direction
    with entries in [0.5, 1.5) to make a scalar cost, ``n_tests`` times; an element whose absolute *and*
    relative error both exceed the tolerances (defaults 5e-2 / 1e-2 / 1e-4 for float16 / 32 / 64, the
    loosest among ``pt``) raises ``GradientError``.  The functions run on the device."""
    if not isinstance(pt, (list, tuple)):
        raise TypeError("verify_grad: the point must be a list of arrays, one per argument")
    if rng is None:
        raise TypeError("verify_grad: pass a seeded numpy.random.RandomState (or Generator) as rng")
    values = [np.array(p) for p in pt]
    kinds = [str(v.dtype) for v in values]
    for k, dt in enumerate(kinds):
        if dt not in TYPE_EPS:
            raise TypeError("verify_grad can work only with floating point inputs, but input %i has dtype \"%s\"."
                            % (k, dt))
    loosest = max(_GRAD_TOL[dt] for dt in kinds)
    abs_tol = loosest if abs_tol is None else abs_tol
    rel_tol = loosest if rel_tol is None else rel_tol
    step = max(TYPE_EPS[dt] for dt in kinds) if eps is None else eps
    check = _GradientCheck(fun, values, mode, out_type or (False if cast_to_output_type else None))
    try:
        for _round in range(n_tests):
            check.new_direction(rng)
            k, j, shape, ana, num, abs_err, rel_err = check.worst(step, abs_tol, rel_tol)
            if abs_err > abs_tol and rel_err > rel_tol:
                raise GradientError(k, j, shape, ana, num, abs_err, rel_err, abs_tol, rel_tol)
    except Exception as e:
        e.args += ("verify_grad was checking at", pt, "with step", step, "and out_type", out_type)
        raise


verify_grad.E_grad = GradientError


# ---- identity operations that change the gradient only (theano/gradient.py:2022-2300) -----------------
class _GradView(gof.Op):
    """The value of the operand, unchanged; the subclasses say what flows back through it.  Compiled
    functions never run these nodes: ``local_remove_grad_views`` takes them out before the graph is
    lifted (the reference does the same, ``theano/tensor/opt.py:local_grad_clip`` and
    ``theano/compile/ops.py`` ``local_useless_*`` for ViewOp), so they cost nothing in the forward pass."""
    view_map = {0: [0]}
    __props__ = ()

    def make_node(self, x):
        from .tensor.type import as_tensor_variable
        if not isinstance(x, gof.Variable):
            x = as_tensor_variable(x)
        return gof.Apply(self, [x], [x.type()])

    def perform(self, node, inputs, output_storage):
        output_storage[0][0] = inputs[0]

    def infer_shape(self, node, shapes):
        return shapes

    def __eq__(self, other):
        return type(self) is type(other)

    def __hash__(self):
        return hash(type(self))

    def __str__(self):
        return type(self).__name__


class ZeroGrad(_GradView):
    """Gradients flow back through as zeros (:2057-2092)."""

    def L_op(self, inputs, outputs, gout):
        return [g.zeros_like() for g in gout]

    def R_op(self, inputs, eval_points):
        if eval_points[0] is None:
            return [None]
        return [eval_points[0].zeros_like()]


class ConsiderConstant(ZeroGrad):
    """The deprecated spelling of ZeroGrad (:2022-2054)."""


class DisconnectedGrad(_GradView):
    """Nothing flows back: the operand is disconnected from the cost through this path (:2133-2173)."""

    def L_op(self, inputs, outputs, gout):
        return [DisconnectedType()() for _ in gout]

    def R_op(self, inputs, eval_points):
        return [None]

    def connection_pattern(self, node):
        return [[False]]


class UndefinedGrad(_GradView):
    """Asking for a gradient through this raises (:2095-2130)."""

    def L_op(self, inputs, outputs, gout):
        return [grad_undefined(self, i, x) for i, x in enumerate(inputs)]

    def R_op(self, inputs, eval_points):
        return [None]

    def connection_pattern(self, node):
        return [[True]]


class GradClip(_GradView):
    """The gradient is clipped to [clip_lower_bound, clip_upper_bound] on the way back (:2176-2232).  The
    bounds take no part in equality, as in the reference: they do not change what the node computes."""

    def __init__(self, clip_lower_bound, clip_upper_bound):
        self.clip_lower_bound, self.clip_upper_bound = clip_lower_bound, clip_upper_bound
        if not self.clip_upper_bound >= self.clip_lower_bound:
            raise ValueError("clip_upper_bound must be at least clip_lower_bound")

    def L_op(self, inputs, outputs, gout):
        from .tensor import basic as T
        return [T.clip(g, self.clip_lower_bound, self.clip_upper_bound) for g in gout]


class GradScale(_GradView):
    """The gradient is multiplied by ``multiplier`` on the way back (:2235-2275)."""

    def __init__(self, multiplier):
        self.multiplier = multiplier

    def L_op(self, inputs, outputs, gout):
        return [self.multiplier * g for g in gout]


consider_constant_, zero_grad_, undefined_grad_, disconnected_grad_ = (ConsiderConstant(), ZeroGrad(), UndefinedGrad(),
                                                                     DisconnectedGrad())


def consider_constant(x):
    """Deprecated: ``zero_grad`` or ``disconnected_grad``."""
    import warnings
    warnings.warn("consider_constant() is deprecated, use zero_grad() or disconnected_grad() instead.", stacklevel=2)
    return consider_constant_(x)


def zero_grad(x):
    """``x``, with zeros for the gradient of everything behind it."""
    return zero_grad_(x)


def undefined_grad(x):
    """``x``; taking a gradient through it raises NullTypeGradError."""
    return undefined_grad_(x)


def disconnected_grad(x):
    """``x``, with nothing behind it reachable from the cost through this path."""
    return disconnected_grad_(x)


def grad_clip(x, lower_bound, upper_bound):
    """``x`` in the forward pass; its gradient clipped elementwise to [lower_bound, upper_bound]."""
    return GradClip(lower_bound, upper_bound)(x)


def grad_scale(x, multiplier):
    """``x`` in the forward pass; its gradient multiplied by ``multiplier``."""
    return GradScale(multiplier)(x)
