"""Device source for the functors the kernel templates are instantiated with.

From a ScalarOp (usually a ``Composite``) and operand dtypes this emits the
struct described in ``csrc/kernels/thx_elemwise.h`` / ``thx_reduce.h``: operand
registers, loads, the per-element statements and stores.  The role is that of
``_generate_op_string`` (``theano/gpuarray/elemwise.py:153-200``) and of the
kernel bodies assembled in ``GpuCAReduceCuda`` (``:969-1093``): everything
per-element comes from ``scalar_op.c_code``.
"""
import hashlib

import numpy as np

from .. import scalar as scal
from ..gof import Apply
from ..scalar import Scalar, c_literal, compute_ctype, storage_ctype


def _scalar_node(op, in_dtypes):
    return op.make_node(*[Scalar(dt)() for dt in in_dtypes])


def _indent(text, n):
    pad = " " * n
    return "\n".join(pad + l if l.strip() else l for l in text.splitlines())


def _name(prefix, text):
    return prefix + hashlib.sha1(text.encode()).hexdigest()[:16]


def _regs(dtypes, names):
    return "  template <int V> struct Regs { %s };\n" % " ".join(
        "thx::Vec<%s, V> %s;" % (storage_ctype(dt), nm) for dt, nm in zip(dtypes, names))


def elemwise_functor(scalar_op, in_dtypes, out_dtypes=None, red=None):
    """(source, functor name, output dtypes) for an n-ary elementwise op.

    ``red = (name of a reduction functor, indices of the outputs it reads)``: the functor names
    that reduction (``Red``) and feeds it, element by element, the results a thread holds
    (``red_lanes``); the source of the reduction functor must precede this one's."""
    node = _scalar_node(scalar_op, in_dtypes)
    odt = [o.type.dtype for o in node.outputs]
    if out_dtypes is not None and list(out_dtypes) != odt:
        raise TypeError("scalar op gives %s, node expects %s" % (odt, list(out_dtypes)))
    nin, nout = len(in_dtypes), len(odt)
    ins = ["i%d" % k for k in range(nin)]
    outs = ["o%d" % k for k in range(nout)]
    stmt = scalar_op.c_code(node, ins, outs)
    params = ", ".join(["const %s %s" % (compute_ctype(dt), nm) for dt, nm in zip(in_dtypes, ins)] +
                       ["%s& %s" % (compute_ctype(dt), nm) for dt, nm in zip(odt, outs)])
    body = []
    body.append("  enum { NIN = %d, NOUT = %d, NOPS = %d };" % (nin, nout, nin + nout))
    body.append(_regs(list(in_dtypes) + odt, ins + outs).rstrip("\n"))
    body.append("  template <int V, class A> THX_DEV static void load(const A& a, Regs<V>& r) { %s }" % " ".join(
        "a.template ld<%d>(r.%s);" % (k, nm) for k, nm in enumerate(ins)))
    body.append("  THX_DEV static void apply(%s) {\n%s\n  }" % (params, _indent(stmt, 4)))
    call = ", ".join(["(%s)r.%s.v[k]" % (compute_ctype(dt), nm) for dt, nm in zip(in_dtypes, ins)] +
                     ["t_%s" % nm for nm in outs])
    decl = " ".join("%s t_%s;" % (compute_ctype(dt), nm) for dt, nm in zip(odt, outs))
    back = " ".join("r.%s.v[k] = (%s)t_%s;" % (nm, storage_ctype(dt), nm) for dt, nm in zip(odt, outs))
    body.append("  template <int V> THX_DEV static void compute(Regs<V>& r) {\n#pragma unroll\n"
                "    for (int k = 0; k < V; ++k) { %s apply(%s); %s }\n  }" % (decl, call, back))
    body.append("  template <int V, class A> THX_DEV static void store(const A& a, const Regs<V>& r) { %s }" % " ".join(
        "a.template st<%d>(r.%s);" % (nin + k, nm) for k, nm in enumerate(outs)))
    if red is not None:
        rname, which = red
        feed = ", ".join("(%s)r.%s.v[k]" % (compute_ctype(odt[w]), outs[w]) for w in which)
        body.append("  typedef %s Red;" % rname)
        body.append("  template <int V, class AccT> THX_DEV static void red_lanes(AccT* acc, const Regs<V>& r) {\n"
                    "#pragma unroll\n    for (int k = 0; k < V; ++k) { typename Red::Acc t; Red::pre(%s, t); "
                    "Red::comb(acc[k], t); }\n  }" % feed)
    text = "\n".join(body)
    name = _name("F", text)
    return "struct %s {\n%s\n};\n" % (name, text), name, odt


# --------------------------------------------------------------------------
def reduce_identity(scalar_op, dtype):
    """Identity element of a reduction op for an accumulator of ``dtype``: the
    op's own, or the extreme value for max / min
    (``theano/tensor/elemwise.py:1470-1488``).  None when the op has none."""
    if isinstance(scalar_op, scal.Minimum):
        big = True
    elif isinstance(scalar_op, scal.Maximum):
        big = False
    else:
        if scalar_op.identity is None:
            return None
        return c_literal(scalar_op.identity, dtype)
    if dtype in scal.complex_dtypes:
        raise NotImplementedError("maximum / minimum of complex numbers (theano/scalar/basic.py:1635, 1674)")
    if dtype in scal.float_dtypes:
        return c_literal(np.inf if big else -np.inf, dtype)
    if dtype == "bool":
        return c_literal(1 if big else 0, dtype)
    info = np.iinfo(dtype)
    return c_literal(info.max if big else info.min, dtype)


def acc_struct_bytes(acc_dtypes):
    """sizeof of a struct holding one field per accumulator dtype."""
    off, align = 0, 1
    for dt in acc_dtypes:
        sz = np.dtype("float32" if dt == "float16" else dt).itemsize
        off = (off + sz - 1) // sz * sz + sz
        align = max(align, sz)
    return (off + align - 1) // align * align


def _narrow_stores(pre_stmt, narrow):
    """The prologue's closing stores ``v.aK = (acc type)pK;`` written so that they convert to whatever
    type field K has in the struct at hand (``Acc``, or ``Part`` with its float32 fields)."""
    import re
    return re.sub(r"v\.a(\d+) = \([a-z0-9_]+\)(p\d+|i0);", r"v.a\1 = (decltype(v.a\1))\2;", pre_stmt)


def _half_products(pre_op, in_dtypes, narrow):
    """For each narrowed sum k whose per-element value is a float16 input widened to float32, its square, or
    the product of two such inputs: ``{k: (a, b)}`` with the input positions (``b`` None for a plain sum).
    Those sums are formed two elements at a time straight from the packed halves (``thx::half_dot``); a
    product of two float16 values is exact in float32, so nothing is lost against widening first."""
    if not isinstance(pre_op, scal.Composite):
        return {}

    def source(v):
        """Position of the float16 input that ``v`` is a widened copy of, or None."""
        while v.owner is not None and isinstance(v.owner.op, (scal.Cast, scal.Identity)) and (
                v.type.dtype == "float32" and v.owner.inputs[0].type.dtype in ("float16", "float32")):
            v = v.owner.inputs[0]
        if v in pre_op.inputs:
            k = pre_op.inputs.index(v)
            return k if in_dtypes[k] == "float16" else None
        return None

    found = {}
    for k, (out, nw) in enumerate(zip(pre_op.outputs, narrow)):
        if nw != "float32" or out.type.dtype != "float32":
            continue
        a = source(out)
        if a is not None:
            found[k] = (a, None)
            continue
        v = out
        while v.owner is not None and isinstance(v.owner.op, scal.Identity):
            v = v.owner.inputs[0]
        if v.owner is None:
            continue
        if isinstance(v.owner.op, scal.Mul) and len(v.owner.inputs) == 2:
            a, b = source(v.owner.inputs[0]), source(v.owner.inputs[1])
            if a is not None and b is not None:
                found[k] = (a, b)
        elif isinstance(v.owner.op, scal.Sqr):
            a = source(v.owner.inputs[0])
            if a is not None:
                found[k] = (a, a)
    return found


def comb_part_src(scalar_ops, acc_dtypes, narrow):
    """Statements merging two ``Part`` values: addition in the partial type (``narrow[k]``, a dtype name) in
    the narrowed fields, the reduction's own op in its accumulator type in the others."""
    out = []
    for k, (op, dt, nw) in enumerate(zip(scalar_ops, acc_dtypes, narrow)):
        dt = nw if nw else dt
        cnode = Apply(op, [Scalar(dt)(), Scalar(dt)()], [Scalar(dt)()])
        out.append(op.c_code(cnode, ["a.a%d" % k, "b.a%d" % k], ["a.a%d" % k]))
    return out


def reduce_functor(scalar_ops, acc_dtypes, in_dtypes, out_dtypes, pre_op=None, post_op=None, extra_dtypes=(),
                   post_in_dtypes=None, extra_is_array=None, half_data=False):
    """(source, name, sizeof(Acc)) for K simultaneous reductions.

    Per element, ``pre_op`` (nin = len(in_dtypes), nout = K; default: the single
    input itself) yields K values, each cast to its accumulator dtype and
    folded with ``scalar_ops[k]``.  ``post_op`` (nin = K + len(extra_dtypes))
    maps the K results, each first cast to ``post_in_dtypes`` (the dtype the
    unfused reduction would have produced), and the extra operands (a host
    scalar's value, or where ``extra_is_array[j]`` the element of a device array
    at the result's index) to the outputs; the default casts result k to
    ``out_dtypes[k]``."""
    K = len(scalar_ops)
    nin, nout = len(in_dtypes), len(out_dtypes)
    ins = ["i%d" % k for k in range(nin)]
    acc_c = [compute_ctype(dt) for dt in acc_dtypes]
    lines = ["  enum { NIN = %d, NOUT = %d, NEX = %d };" % (nin, nout, len(extra_dtypes))]
    lines.append("  struct Acc { %s };" % " ".join("%s a%d;" % (c, k) for k, c in enumerate(acc_c)))
    lines.append(_regs(in_dtypes, ins).rstrip("\n"))
    init = []
    for k, (op, dt) in enumerate(zip(scalar_ops, acc_dtypes)):
        ident = reduce_identity(op, dt)
        if ident is None:
            raise NotImplementedError("reduction with %s has no identity element" % op)
        init.append("a.a%d = %s;" % (k, ident))
    lines.append("  THX_DEV static void init(Acc& a) { %s }" % " ".join(init))
    lines.append("  template <int V, class A> THX_DEV static void load(const A& a, Regs<V>& r) { %s }" % " ".join(
        "a.template ld<%d>(r.%s);" % (k, nm) for k, nm in enumerate(ins)))
    # prologue
    if pre_op is None:
        if nin != 1 or K != 1:
            raise ValueError("a reduction without prologue takes one input and one accumulator")
        pre_stmt = "v.a0 = (%s)i0;" % acc_c[0]
        value_dtypes = ["float32" if in_dtypes[0] == "float16" else in_dtypes[0]]
    else:
        pnode = _scalar_node(pre_op, in_dtypes)
        if len(pnode.outputs) != K:
            raise ValueError("prologue yields %d values for %d reductions" % (len(pnode.outputs), K))
        tmp = ["p%d" % k for k in range(K)]
        value_dtypes = ["float32" if o.type.dtype == "float16" else o.type.dtype for o in pnode.outputs]
        pre_stmt = " ".join("%s %s;" % (compute_ctype(o.type.dtype), t) for o, t in zip(pnode.outputs, tmp))
        pre_stmt += "\n" + pre_op.c_code(pnode, ins, tmp) + "\n"
        pre_stmt += " ".join("v.a%d = (%s)%s;" % (k, acc_c[k], t) for k, t in enumerate(tmp))
    # float32 partial sums per vector for float64 sums over float16 data (see ``half_data``)
    # ... and 32-bit partial sums per vector for 64-bit sums over 8- and 16-bit integers: the at most 16 elements
    # of a vector cannot overflow them, and a 64-bit addition per vector replaces one per element
    def partial_dtype(op, acc, val):
        if not isinstance(op, scal.Add):
            return None
        if half_data and acc == "float64" and val == "float32":
            return "float32"
        if acc == "int64" and val in ("bool", "int8", "int16", "uint8", "uint16"):
            return "int32"
        if acc == "uint64" and val in ("bool", "uint8", "uint16"):
            return "uint32"
        return None
    narrow = [partial_dtype(op, acc, val) for op, acc, val in zip(scalar_ops, acc_dtypes, value_dtypes)]
    if any(narrow):
        part_c = {"float32": "thx_f32", "int32": "int", "uint32": "unsigned int"}
        lines[1] += "\n  struct Part { %s };" % " ".join(
            "%s a%d;" % (part_c[nw] if nw else c, k) for k, (c, nw) in enumerate(zip(acc_c, narrow)))
    lines.append("  template <class AccT> THX_DEV static void pre(%s, AccT& v) {\n%s\n  }" % (
        ", ".join("const %s %s" % (compute_ctype(dt), nm) for dt, nm in zip(in_dtypes, ins)),
        _indent(pre_stmt if not any(narrow) else _narrow_stores(pre_stmt, narrow), 4)))
    # combine: the reduction op applied to two accumulator-typed values
    comb = []
    for k, (op, dt) in enumerate(zip(scalar_ops, acc_dtypes)):
        cnode = Apply(op, [Scalar(dt)(), Scalar(dt)()], [Scalar(dt)()])
        comb.append(op.c_code(cnode, ["a.a%d" % k, "b.a%d" % k], ["a.a%d" % k]))
    lines.append("  THX_DEV static void comb(Acc& a, const Acc& b) {\n%s\n  }" % _indent("\n".join(comb), 4))
    call = ", ".join("(%s)r.%s.v[k]" % (compute_ctype(dt), nm) for dt, nm in zip(in_dtypes, ins))
    if any(narrow):
        # the elements of one vector meet in a Part (float32 where narrowed) before the accumulator sees them
        comb_part = comb_part_src(scalar_ops, acc_dtypes, narrow)
        lines.append("  THX_DEV static void comb_part(Part& a, const Part& b) {\n%s\n  }" % _indent("\n".join(comb_part), 4))
        call0 = call.replace(".v[k]", ".v[0]")
        widen = " ".join("w.a%d = (%s)t.a%d;" % (k, acc_c[k], k) for k in range(K))
        # sums of float16 inputs and of their pairwise products come from the packed halves, two elements per
        # instruction; the per-element form of those fields above is then dead code the compiler drops
        dots = _half_products(pre_op, in_dtypes, narrow) if pre_op is not None else {}
        packed = " ".join("t.a%d = thx::half_%s;" % (k, "sum<V>(r.%s)" % ins[a] if b is None else
                                                     "dot<V>(r.%s, r.%s)" % (ins[a], ins[b]))
                          for k, (a, b) in sorted(dots.items()))
        packed = "    if constexpr (V %% 2 == 0) { %s }\n" % packed if packed else ""
        if pre_op is None and narrow[0] in ("int32", "uint32"):
            # the narrow integers themselves are summed: four or two of them per instruction
            packed = ("    if constexpr ((V * sizeof(%s)) %% 4 == 0) { t.a0 = (decltype(t.a0))thx::packed_isum<V>(r.%s); }\n"
                      % (storage_ctype(in_dtypes[0]), ins[0]))
        lines.append("  template <int V> THX_DEV static void accum(Acc& s, const Regs<V>& r) {\n"
                     "    Part t; pre(%s, t);\n#pragma unroll\n"
                     "    for (int k = 1; k < V; ++k) { Part u; pre(%s, u); comb_part(t, u); }\n%s"
                     "    Acc w; %s comb(s, w);\n  }" % (call0, call, packed, widen))
    else:
        lines.append("  template <int V> THX_DEV static void accum(Acc& s, const Regs<V>& r) {\n#pragma unroll\n"
                     "    for (int k = 0; k < V; ++k) { Acc t; pre(%s, t); comb(s, t); }\n  }" % call)
    lines.append("  template <int V> THX_DEV static void accum_lanes(Acc* s, const Regs<V>& r) {\n#pragma unroll\n"
                 "    for (int k = 0; k < V; ++k) { Acc t; pre(%s, t); comb(s[k], t); }\n  }" % call)
    lines.append("  THX_DEV static Acc shfl_xor(const Acc& a, int m) { Acc r; %s return r; }" % " ".join(
        "r.a%d = thx::shfl_xor_t(a.a%d, m);" % (k, k) for k in range(K)))
    # epilogue
    if post_op is None:
        if nout != K:
            raise ValueError("a reduction without epilogue has one output per accumulator")
        post = []
        for k, dt in enumerate(out_dtypes):
            val = "a.a%d" % k
            if dt == "bool":
                val = "(%s ? 1 : 0)" % val
            post.append("((%s*)o.ptr[%d])[idx] = (%s)%s;" % (storage_ctype(dt), k, storage_ctype(dt), val))
        post_stmt = "\n".join(post)
    else:
        post_in = list(post_in_dtypes) if post_in_dtypes is not None else list(acc_dtypes)
        qnode = _scalar_node(post_op, post_in + list(extra_dtypes))
        if [o.type.dtype for o in qnode.outputs] != list(out_dtypes):
            raise TypeError("epilogue gives %s, node expects %s" % ([o.type.dtype for o in qnode.outputs],
                                                                      list(out_dtypes)))
        tmp = ["q%d" % k for k in range(nout)]
        post_stmt = " ".join("%s %s;" % (compute_ctype(dt), t) for dt, t in zip(out_dtypes, tmp))
        # each reduction result takes the storage precision of the unfused node's output first
        args = []
        for k, dt in enumerate(post_in):
            post_stmt += "\n%s r%d = (%s)(%s)%s;" % (compute_ctype(dt), k, compute_ctype(dt), storage_ctype(dt),
                                                     "(a.a%d ? 1 : 0)" % k if dt == "bool" else "a.a%d" % k)
            args.append("r%d" % k)
        for j, dt in enumerate(extra_dtypes):
            # read in the storage type, used in the arithmetic type (float16 computes as float, as every kernel
            # operand does: the scalar ops' code is written for that)
            if extra_is_array is not None and extra_is_array[j]:
                args.append("((%s)(((const %s*)o.ex[%d])[idx * o.exs[%d]]))" % (compute_ctype(dt), storage_ctype(dt), j, j))
            else:
                args.append("((%s)(*(const %s*)&o.ex[%d]))" % (compute_ctype(dt), storage_ctype(dt), j))
        post_stmt += "\n" + post_op.c_code(qnode, args, tmp) + "\n"
        post_stmt += "\n".join("((%s*)o.ptr[%d])[idx] = (%s)%s;" % (storage_ctype(dt), k, storage_ctype(dt), t)
                               for k, (dt, t) in enumerate(zip(out_dtypes, tmp)))
    lines.append("  template <class O> THX_DEV static void post(const O& o, long long idx, const Acc& a) {\n%s\n  }"
                 % _indent(post_stmt, 4))
    # any / all: the slices of a split reduction settle the result with one atomic add each (thx_reduce.h)
    if K <= 3 and all(dt == "bool" and isinstance(op, (scal.OR, scal.AND)) for op, dt in zip(scalar_ops, acc_dtypes)):
        pack = " | ".join("((unsigned long long)(%sa.a%d ? 1 : 0) << %d)" % ("" if isinstance(op, scal.OR) else "!", k, 16 * k)
                          for k, op in enumerate(scalar_ops))
        unpack = " ".join("a.a%d = ((w >> %d) & 0xffffull) %s 0;" % (k, 16 * k, "!=" if isinstance(op, scal.OR) else "==")
                          for k, op in enumerate(scalar_ops))
        lines.append("  THX_DEV static unsigned long long ticket_pack(const Acc& a) { return %s; }" % pack)
        lines.append("  THX_DEV static Acc ticket_unpack(unsigned long long w) { Acc a; %s return a; }" % unpack)
    text = "\n".join(lines)
    name = _name("R", text)
    return "struct %s {\n%s\n};\n" % (name, text), name, acc_struct_bytes(acc_dtypes)


def argmax_functor(in_dtypes, value_dtype, pre_op=None, packed=False):
    """(source, name, sizeof(Acc)) of the reduction behind ``MaxAndArgmax``.

    The inputs are ``in_dtypes`` followed by one int64 position operand (the
    library's index operand: the element's position within the reduced
    dimensions).  ``pre_op`` (default: the single input itself) gives the value;
    the accumulator is the pair (value, position).  Merging keeps the greater
    value, a NaN before any number, and on equal values (or two NaNs) the smaller
    position - so the result is NumPy's first occurrence whatever order partial
    results meet in.

    ``packed`` (values of at most 32 bits, fewer than 2^31 reduced elements per
    result): the pair travels as one unsigned 64-bit key - the value mapped to an
    order-preserving unsigned 32-bit number (every NaN to the largest) in the high
    half, the complemented position in the low half - so merging is a single
    64-bit maximum instead of a cascade of comparisons and selects."""
    nin = len(in_dtypes)
    ins = ["i%d" % k for k in range(nin)]
    vt = compute_ctype(value_dtype)
    st = storage_ctype(value_dtype)
    if packed and np.dtype(value_dtype).itemsize > 4:
        raise ValueError("packed keys hold values of at most 32 bits")
    lines = ["  enum { NIN = %d, NOUT = 2, NEX = 0 };" % (nin + 1)]
    if packed:
        lines.append("  struct Acc { unsigned long long key; };")
    else:
        lines.append("  struct Acc { %s val; long long idx; };" % vt)
    lines.append(_regs(list(in_dtypes) + ["int64"], ins + ["ix"]).rstrip("\n"))
    if value_dtype in scal.float_dtypes:
        lowest = c_literal(-np.inf, value_dtype)
    elif value_dtype == "bool":
        lowest = c_literal(0, value_dtype)
    else:
        lowest = c_literal(np.iinfo(value_dtype).min, value_dtype)
    if packed:
        lines.append("  THX_DEV static void init(Acc& a) { a.key = 0ull; }")
    else:
        lines.append("  THX_DEV static void init(Acc& a) { a.val = %s; a.idx = 0x7fffffffffffffffLL; }" % lowest)
    lines.append("  template <int V, class A> THX_DEV static void load(const A& a, Regs<V>& r) { %s a.template ld<%d>(r.ix); }"
                 % (" ".join("a.template ld<%d>(r.%s);" % (k, nm) for k, nm in enumerate(ins)), nin))
    if pre_op is None:
        if nin != 1:
            raise ValueError("without prologue the reduction takes one input")
        value_stmt = "const %s val = (%s)i0;" % (vt, vt)
    else:
        pnode = _scalar_node(pre_op, in_dtypes)
        if len(pnode.outputs) != 1 or pnode.outputs[0].type.dtype != value_dtype:
            raise TypeError("prologue must yield one %s value" % value_dtype)
        value_stmt = "%s p0;\n%s\nconst %s val = (%s)p0;" % (vt, pre_op.c_code(pnode, ins, ["p0"]), vt, vt)
    if packed:
        if value_dtype in scal.float_dtypes:        # float16 widens exactly to float32
            # adding +0 turns -0 into +0: the two compare equal, so they must share one key
            to_key = ("const float f = (float)val + 0.0f;\nunsigned int b = __float_as_uint(f);\n"
                      "b = (f != f) ? 0xffffffffu : (b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u));")
            from_key = ("const unsigned int k = (unsigned int)(a.key >> 32);\n"
                        "const %s val = (%s)(k == 0xffffffffu ? __uint_as_float(0x7fc00000u) : "
                        "__uint_as_float((k >> 31) ? (k ^ 0x80000000u) : ~k));" % (st, st))
        elif value_dtype in scal.int_dtypes:
            to_key = "const unsigned int b = (unsigned int)(int)val ^ 0x80000000u;"
            from_key = "const %s val = (%s)(int)((unsigned int)(a.key >> 32) ^ 0x80000000u);" % (st, st)
        else:                                        # unsigned integers and bool
            to_key = "const unsigned int b = (unsigned int)val;"
            from_key = "const %s val = (%s)(unsigned int)(a.key >> 32);" % (st, st)
        pre_stmt = "%s\n%s\nv.key = ((unsigned long long)b << 32) | (unsigned int)~(unsigned int)ix;" % (value_stmt, to_key)
        comb = "    if (b.key > a.key) a.key = b.key;"
        shfl = "Acc r; r.key = thx::shfl_xor_t(a.key, m); return r;"
        post = ("%s\n((%s*)o.ptr[0])[idx] = val;\n"
                "((long long*)o.ptr[1])[idx] = (long long)(unsigned int)~(unsigned int)a.key;" % (from_key, st))
        size = 8
    else:
        pre_stmt = "%s\nv.val = val;\nv.idx = ix;" % value_stmt
        nan_a, nan_b = ("a.val != a.val", "b.val != b.val") if value_dtype in scal.float_dtypes else ("false", "false")
        comb = ("    const bool an = %s, bn = %s;\n"
                "    const bool take = bn ? (!an || b.idx < a.idx)\n"
                "                         : (!an && (b.val > a.val || (b.val == a.val && b.idx < a.idx)));\n"
                "    if (take) a = b;" % (nan_a, nan_b))
        shfl = "Acc r; r.val = thx::shfl_xor_t(a.val, m); r.idx = thx::shfl_xor_t(a.idx, m); return r;"
        post = "((%s*)o.ptr[0])[idx] = (%s)a.val;\n((long long*)o.ptr[1])[idx] = a.idx;" % (st, st)
        size = 16
    lines.append("  THX_DEV static void pre(%s, const long long ix, Acc& v) {\n%s\n  }" % (
        ", ".join("const %s %s" % (compute_ctype(dt), nm) for dt, nm in zip(in_dtypes, ins)), _indent(pre_stmt, 4)))
    lines.append("  THX_DEV static void comb(Acc& a, const Acc& b) {\n%s\n  }" % comb)
    call = ", ".join(["(%s)r.%s.v[k]" % (compute_ctype(dt), nm) for dt, nm in zip(in_dtypes, ins)] + ["r.ix.v[k]"])
    lines.append("  template <int V> THX_DEV static void accum(Acc& s, const Regs<V>& r) {\n#pragma unroll\n"
                 "    for (int k = 0; k < V; ++k) { Acc t; pre(%s, t); comb(s, t); }\n  }" % call)
    lines.append("  template <int V> THX_DEV static void accum_lanes(Acc* s, const Regs<V>& r) {\n#pragma unroll\n"
                 "    for (int k = 0; k < V; ++k) { Acc t; pre(%s, t); comb(s[k], t); }\n  }" % call)
    lines.append("  THX_DEV static Acc shfl_xor(const Acc& a, int m) { %s }" % shfl)
    lines.append("  template <class O> THX_DEV static void post(const O& o, long long idx, const Acc& a) {\n%s\n  }"
                 % _indent(post, 4))
    text = "\n".join(lines)
    name = _name("A", text)
    return "struct %s {\n%s\n};\n" % (name, text), name, size
