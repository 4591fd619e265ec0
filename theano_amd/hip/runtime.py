"""ctypes binding of libthx_hip.so and the device array type built on it.

The library is the only execution path: importing this module fails if the
shared object has not been built, and every call that needs the GPU raises
when no device is present.  ``HipArray`` plays the role pygpu's ``GpuArray``
plays for the reference (``theano/gpuarray/type.py:129-517``): a strided view
(shape, byte strides, offset) over a reference-counted device buffer.
"""
import ctypes
import os

import numpy as np

from .. import scalar as scal

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(os.path.dirname(_HERE), "csrc", "libthx_hip.so")

THX_MAX_ND = 8
THX_BROADCAST = 1
THX_DRY_RUN = 2
THX_HOST_SCALAR = 0x100
THX_INDEX = 0x200
THX_REUSED = 0x400


class thx_array(ctypes.Structure):
    _fields_ = [("base", ctypes.c_void_p), ("offset_bytes", ctypes.c_int64), ("nd", ctypes.c_int32),
                ("dtype", ctypes.c_int32), ("shape", ctypes.c_int64 * THX_MAX_ND),
                ("strides_bytes", ctypes.c_int64 * THX_MAX_ND)]


class HipRuntimeError(RuntimeError):
    pass


_EXC = {1: HipRuntimeError, 2: ValueError, 3: TypeError, 4: HipRuntimeError, 5: MemoryError,
        6: NotImplementedError, 7: ValueError}


def _load():
    if not os.path.exists(_LIB_PATH):
        raise ImportError("libthx_hip.so is missing (%s). Build it with `python -m theano_amd.csrc.build`; "
                          "there is no other execution path." % _LIB_PATH)
    lib = ctypes.CDLL(_LIB_PATH)
    vp, sz, i32, i64 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int32, ctypes.c_int64
    P = ctypes.POINTER
    sigs = {
        "thx_init": ([ctypes.c_int], ctypes.c_int),
        "thx_device_info": ([ctypes.c_char_p, sz, P(ctypes.c_int), P(i64)], ctypes.c_int),
        "thx_last_error": ([], ctypes.c_char_p),
        "thx_last_plan": ([], ctypes.c_char_p),
        "thx_alloc": ([sz, P(vp)], ctypes.c_int),
        "thx_free": ([vp], ctypes.c_int),
        "thx_pool_trim": ([], ctypes.c_int),
        "thx_h2d": ([vp, vp, sz], ctypes.c_int),
        "thx_d2h": ([vp, vp, sz], ctypes.c_int),
        "thx_d2d": ([vp, vp, sz], ctypes.c_int),
        "thx_fill_bytes": ([vp, ctypes.c_int, sz], ctypes.c_int),
        "thx_sync": ([], ctypes.c_int),
        "thx_set_cache_dir": ([ctypes.c_char_p], ctypes.c_int),
        "thx_cache_stats": ([P(i64), P(i64), P(i64)], ctypes.c_int),
        "thx_elemwise_new": ([ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int, P(i32), P(vp)], ctypes.c_int),
        "thx_elemwise_call": ([vp, P(thx_array), P(thx_array), ctypes.c_int], ctypes.c_int),
        "thx_elemwise_free": ([vp], ctypes.c_int),
        "thx_elemwise_attach_reduce": ([vp, vp, P(i32)], ctypes.c_int),
        "thx_elemwise_reduce_call": ([vp, P(thx_array), P(thx_array), P(thx_array), ctypes.c_int], ctypes.c_int),
        "thx_reduce_call_static": ([vp, P(thx_array), P(ctypes.c_uint8), P(thx_array), ctypes.c_int], ctypes.c_int),
        "thx_reduce_new": ([ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, P(i32),
                            ctypes.c_int, P(vp)], ctypes.c_int),
        "thx_reduce_call": ([vp, P(thx_array), P(ctypes.c_uint8), P(thx_array), ctypes.c_int], ctypes.c_int),
        "thx_reduce_free": ([vp], ctypes.c_int),
        "thx_rowchain_new": ([ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int, P(i32), P(i32), P(vp)],
                             ctypes.c_int),
        "thx_rowchain_call": ([vp, P(thx_array), P(thx_array), ctypes.c_int], ctypes.c_int),
        "thx_rowchain_set_axes": ([vp, ctypes.c_int, P(i32)], ctypes.c_int),
        "thx_rowchain_free": ([vp], ctypes.c_int),
        "thx_profile_begin": ([], ctypes.c_int),
        "thx_profile_end": ([ctypes.c_char_p, sz], ctypes.c_int),
        "thx_timer_start": ([], ctypes.c_int),
        "thx_timer_stop": ([P(ctypes.c_float)], ctypes.c_int),
        "thx_capture_begin": ([], ctypes.c_int),
        "thx_capture_end": ([P(vp)], ctypes.c_int),
        "thx_graph_launch": ([vp], ctypes.c_int),
        "thx_graph_free": ([vp], ctypes.c_int),
        "thx_scratch_reserve": ([sz], ctypes.c_int),
        "thx_scratch_state": ([P(i64), P(i64), P(i64)], ctypes.c_int),
    }
    for name, (argtypes, restype) in sigs.items():
        fn = getattr(lib, name, None)
        if fn is None:
            continue
        fn.argtypes = argtypes
        fn.restype = restype
    return lib


lib = _load()
_default_cache = os.environ.get("THX_CACHE_DIR") or os.path.join(os.path.dirname(_HERE), "_kcache")
lib.thx_set_cache_dir(_default_cache.encode())


def check(rc):
    if rc != 0:
        msg = lib.thx_last_error().decode(errors="replace")
        raise _EXC.get(rc, HipRuntimeError)(msg)


_initialised = False
_dry = False
_fake_next = [0x7f0000000000]


def set_dry_run(flag):
    """In dry-run mode nothing touches a GPU: arrays get placeholder addresses
    and every kernel call only validates, plans and compiles (filling the
    on-disk code-object cache).  Used to check and pre-build kernels on a
    machine without a device; results are meaningless."""
    global _dry
    _dry = bool(flag)


def dry_run():
    return _dry


def call_flags(node=None):
    """Flags of a kernel call."""
    return THX_BROADCAST | (THX_DRY_RUN if _dry else 0)


def mark_reused(node, ins, outs):
    """OR THX_REUSED into the descriptors of the operands that a later kernel of the same
    function reads (positions recorded in ``node.tag`` when the function was compiled)."""
    for k in node.tag.get("reused_in", ()):
        ins[k].dtype |= THX_REUSED
    for k in node.tag.get("reused_out", ()):
        outs[k].dtype |= THX_REUSED


def init(device=None):
    """Bind the library to a GPU; raises HipRuntimeError when none is visible."""
    global _initialised
    if _dry:
        return
    if not _initialised:
        from ..config import config
        check(lib.thx_init(config.device if device is None else device))
        _initialised = True


def device_info():
    init()
    buf = ctypes.create_string_buffer(128)
    cus, hbm = ctypes.c_int(), ctypes.c_int64()
    check(lib.thx_device_info(buf, 128, ctypes.byref(cus), ctypes.byref(hbm)))
    return {"arch": buf.value.decode(), "compute_units": cus.value, "hbm_bytes": hbm.value}


def sync():
    check(lib.thx_sync())


def last_plan():
    return lib.thx_last_plan().decode()


def cache_stats():
    a, b, c = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
    lib.thx_cache_stats(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
    return {"compiled": a.value, "disk_hits": b.value, "mem_hits": c.value}


class profile(object):
    """Context manager collecting per-kernel HIP-event timings:
    ``with profile() as p: ...`` then ``p.kernels`` maps plan name to
    (launches, total milliseconds)."""

    def __enter__(self):
        init()
        check(lib.thx_profile_begin())
        self.kernels = {}
        return self

    def __exit__(self, *exc):
        buf = ctypes.create_string_buffer(1 << 20)
        check(lib.thx_profile_end(buf, 1 << 20))
        for line in buf.value.decode().splitlines():
            name, n, ms = line.rsplit("\t", 2)
            self.kernels[name] = (int(n), float(ms))
        return False


def timer_start():
    check(lib.thx_timer_start())


def timer_stop():
    ms = ctypes.c_float()
    check(lib.thx_timer_stop(ctypes.byref(ms)))
    return ms.value


# --------------------------------------------------------------------------
_capture_keep = None      # while a capture is open: the buffers allocated inside it, which its graph owns


class Graph(object):
    """A recorded sequence of launches (``capture``): ``launch()`` replays it on the library's stream.  The
    graph owns every buffer that was allocated while it was recorded - replays write to those addresses -
    and ``hold(...)`` adds the arrays it only reads (arguments, shared variables' values as of the
    recording), so that nothing a replay touches returns to the pool while the graph is alive."""

    def __init__(self, handle, buffers):
        self._handle, self._buffers = handle, list(buffers)

    def hold(self, *arrays):
        self._buffers.extend(arrays)
        return self

    def launch(self):
        check(lib.thx_graph_launch(self._handle))

    def __del__(self):
        try:
            if self._handle is not None:
                lib.thx_graph_free(self._handle)
                self._handle = None
        except Exception:
            pass


def scratch_state():
    """(bytes of the reduction scratch buffer, superseded buffers still held for recorded sequences,
    recorded sequences alive)."""
    a, b, c = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
    check(lib.thx_scratch_state(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)))
    return a.value, b.value, c.value


def scratch_reserve(nbytes):
    init()
    check(lib.thx_scratch_reserve(int(nbytes)))


class capture(object):
    """``with capture() as c: ...`` records what the library launches inside the block instead of running it;
    ``c.graph`` is the replayable result.  Nothing inside may wait for the device (no ``to_numpy``, no host
    arguments or results), and the same calls should have run once before, so that their kernels are loaded."""

    def __enter__(self):
        global _capture_keep
        if _dry:
            raise HipRuntimeError("nothing is launched in dry-run mode: there is nothing to capture")
        if _capture_keep is not None:
            raise HipRuntimeError("a capture is already open")
        init()
        check(lib.thx_capture_begin())
        _capture_keep = []
        self.graph = None
        return self

    def __exit__(self, et, ev, tb):
        global _capture_keep
        kept, _capture_keep = _capture_keep, None
        if et is not None:
            lib.thx_capture_end(None)
            return False
        h = ctypes.c_void_p()
        check(lib.thx_capture_end(ctypes.byref(h)))
        self.graph = Graph(h, kept)
        return False


class _Buffer(object):
    """One pooled device allocation, released when the last view dies."""

    __slots__ = ("ptr", "nbytes", "fake")

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        self.fake = _dry
        if _dry:
            self.ptr = _fake_next[0]
            _fake_next[0] += (self.nbytes + 4095) // 4096 * 4096 + 4096
            return
        init()
        p = ctypes.c_void_p()
        check(lib.thx_alloc(max(int(nbytes), 1), ctypes.byref(p)))
        self.ptr = p.value
        if _capture_keep is not None:
            _capture_keep.append(self)

    def __del__(self):
        try:
            if self.ptr and not self.fake:
                lib.thx_free(self.ptr)
                self.ptr = None
        except Exception:
            pass


def _c_strides(shape, itemsize):
    strides, acc = [], itemsize
    for s in reversed(shape):
        strides.append(acc)
        acc *= max(int(s), 1)
    return tuple(reversed(strides))


_CODE_OF = dict((np.dtype(name), scal.dtype_code(name)) for name in scal.all_dtypes)


class HipArray(object):
    """A strided view of device memory."""

    __slots__ = ("buffer", "offset", "shape", "strides", "dtype", "code")

    def __init__(self, buffer, offset, shape, strides, dtype):
        self.buffer = buffer
        self.offset = int(offset)
        self.shape = tuple(int(s) for s in shape)
        self.strides = tuple(int(s) for s in strides)
        self.dtype = np.dtype(dtype)
        self.code = _CODE_OF[self.dtype]

    @classmethod
    def _raw(cls, buffer, offset, shape, strides, dtype, code):
        """A view from fields that are already of the right kind (tuples of ints, a np.dtype)."""
        self = cls.__new__(cls)
        self.buffer = buffer
        self.offset = offset
        self.shape = shape
        self.strides = strides
        self.dtype = dtype
        self.code = code
        return self

    @classmethod
    def _new_contiguous(cls, shape, dtype):
        """``empty`` for callers that already hold a tuple of ints and a np.dtype."""
        self = cls.__new__(cls)
        n = dtype.itemsize
        strides = []
        for s in reversed(shape):
            strides.append(n)
            n *= s if s > 1 else 1
        strides.reverse()
        total = dtype.itemsize
        for s in shape:
            total *= s
        self.buffer = _Buffer(total)
        self.offset = 0
        self.shape = shape
        self.strides = tuple(strides)
        self.dtype = dtype
        self.code = _CODE_OF[dtype]
        return self

    @classmethod
    def _new_fortran(cls, shape, dtype):
        """Column-major counterpart of ``_new_contiguous``."""
        self = cls._new_contiguous(tuple(reversed(shape)), dtype)
        self.shape = shape
        self.strides = tuple(reversed(self.strides))
        return self

    # -- construction
    @classmethod
    def empty(cls, shape, dtype):
        dtype = np.dtype(dtype)
        shape = tuple(int(s) for s in shape)
        if len(shape) > THX_MAX_ND:
            raise TypeError("arrays of rank %d exceed the limit of %d" % (len(shape), THX_MAX_ND))
        n = 1
        for s in shape:
            n *= s
        return cls(_Buffer(n * dtype.itemsize), 0, shape, _c_strides(shape, dtype.itemsize), dtype)

    @classmethod
    def from_numpy(cls, a):
        a = np.asarray(a)
        if a.dtype not in _CODE_OF:
            raise TypeError("dtype %s is not supported on the device" % a.dtype)
        if _dry:                       # shapes only: nothing is copied, so nothing needs to exist
            return cls.empty(a.shape, a.dtype)
        if a.ndim > 1 and a.flags.f_contiguous and not a.flags.c_contiguous:
            return cls.from_numpy(a.T).transpose()      # column-major arrays keep their layout
        a = np.asarray(a, order="C")
        out = cls.empty(a.shape, a.dtype)
        if a.nbytes and not out.buffer.fake:
            check(lib.thx_h2d(out.buffer.ptr, a.ctypes.data, a.nbytes))
        return out

    # -- properties
    @property
    def ndim(self):
        return len(self.shape)

    @property
    def size(self):
        n = 1
        for s in self.shape:
            n *= s
        return n

    @property
    def nbytes(self):
        return self.size * self.dtype.itemsize

    @property
    def ptr(self):
        return self.buffer.ptr + self.offset

    @property
    def c_contiguous(self):
        expect = self.dtype.itemsize
        for s, st in zip(reversed(self.shape), reversed(self.strides)):
            if s > 1 and st != expect:
                return False
            expect *= max(s, 1)
        return True

    @property
    def scaled_contiguous(self):
        """The layout of a C-contiguous array with every stride multiplied by one non-zero factor: a
        contiguous array, or a view that keeps its dimensions in order (``x[0, :, 0, 0]``, ``x[::2]``)."""
        expect = 0
        for s, st in zip(reversed(self.shape), reversed(self.strides)):
            if s > 1:
                if not expect:
                    if st == 0 or st % self.dtype.itemsize:
                        return False
                    expect = st
                if st != expect:
                    return False
                expect *= s
        return True

    @property
    def is_fortran(self):
        """Column-major contiguous and not row-major contiguous (NumPy's
        ``PyArray_ISFORTRAN``)."""
        shape, strides = self.shape, self.strides
        if len(shape) < 2 or (strides[-1] == self.dtype.itemsize and shape[-1] > 1):
            return False
        expect = self.dtype.itemsize
        for s, st in zip(shape, strides):
            if s > 1 and st != expect:
                return False
            expect *= max(s, 1)
        return not self.c_contiguous

    def __repr__(self):
        return "HipArray(shape=%s, dtype=%s, strides=%s)" % (self.shape, self.dtype, self.strides)

    # -- views
    def view(self, shape, strides, offset=None):
        return HipArray(self.buffer, self.offset if offset is None else offset, shape, strides, self.dtype)

    def transpose(self, *axes):
        if not axes:
            axes = tuple(reversed(range(self.ndim)))
        return self.view([self.shape[a] for a in axes], [self.strides[a] for a in axes])

    def copy(self):
        """A C-contiguous device copy."""
        out = HipArray.empty(self.shape, self.dtype)
        if self.size and not out.buffer.fake:
            if self.c_contiguous:
                check(lib.thx_d2d(out.ptr, self.ptr, self.nbytes))
            else:
                from .views import copy_into
                copy_into(self, out)
        return out

    # -- transfers
    def to_numpy(self):
        """Copy to host; strided views are copied as the byte span they cover
        and re-viewed on the host."""
        out = np.empty(self.shape, self.dtype)
        if self.buffer.fake:
            out.fill(0)
            return out
        if self.size == 0:
            return out
        if self.c_contiguous:
            check(lib.thx_d2h(out.ctypes.data, self.ptr, out.nbytes))
            return out
        lo = hi = 0
        for s, st in zip(self.shape, self.strides):
            if st < 0:
                lo += (s - 1) * st
            else:
                hi += (s - 1) * st
        span = hi - lo + self.dtype.itemsize
        raw = np.empty(span, np.uint8)
        check(lib.thx_d2h(raw.ctypes.data, self.ptr + lo, span))
        view = np.ndarray(self.shape, self.dtype, buffer=raw, offset=-lo, strides=self.strides)
        out[...] = view
        return out

    def __array__(self, dtype=None, copy=None):
        a = self.to_numpy()
        return a if dtype is None else a.astype(dtype)

    def as_thx(self, out=None):
        a = out if out is not None else thx_array()
        a.base = self.buffer.ptr
        a.offset_bytes = self.offset
        n = len(self.shape)
        a.nd = n
        a.dtype = self.code
        a.shape[:n] = self.shape
        a.strides_bytes[:n] = self.strides
        return a


def host_scalar_thx(value, nd, out=None):
    """Descriptor of a one-element host array passed by value (as a kernel
    argument) instead of through device memory."""
    a = out if out is not None else thx_array()
    a.base = value.ctypes.data
    a.offset_bytes = 0
    a.nd = nd
    a.dtype = _CODE_OF[value.dtype] | THX_HOST_SCALAR
    for i in range(nd):
        a.shape[i] = 1
        a.strides_bytes[i] = 0
    return a
