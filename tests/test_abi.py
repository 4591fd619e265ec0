"""The C-ABI library loads, exports every symbol the public header declares,
and its planner + hipRTC path compiles every kernel family for gfx950 without
a GPU (dry run)."""
import ctypes
import os
import re

import numpy as np
import pytest

import theano_amd as th
from theano_amd import hip, tensor as T
from theano_amd.hip import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "thx_hip.h")).read()
    names = set(re.findall(r"\b(thx_[a-z0-9_]+)\s*\(", header))
    assert len(names) >= 24
    lib = ctypes.CDLL(runtime._LIB_PATH)
    missing = [n for n in sorted(names) if not hasattr(lib, n)]
    assert not missing, missing


def test_fixed_scratch_array_is_visible_to_the_runtime(tmp_path):
    """hipGetSymbolAddress finds a device variable by name in the library's gfx950 code object, so the
    fixed scratch array of thx_reduce_call_static must be a global symbol there, of the size the
    header states (a local one makes thx_init abort on a GPU)."""
    import subprocess
    readelf, objcopy = "/opt/rocm/llvm/bin/llvm-readelf", "/opt/rocm/llvm/bin/llvm-objcopy"
    if not (os.path.exists(readelf) and os.path.exists(objcopy)):
        pytest.skip("no llvm binutils")
    fat = str(tmp_path / "fat.bin")
    subprocess.run([objcopy, "-O", "binary", "--only-section=.hip_fatbin", runtime._LIB_PATH, fat], check=True)
    data = open(fat, "rb").read()
    starts = [m.start() for m in re.finditer(b"\x7fELF", data)]
    header = open(os.path.join(ROOT, "include", "thx_hip.h")).read()
    size = int(re.search(r"#define\s+THX_STATIC_SCRATCH_BYTES\s+(\d+)", header).group(1))
    found = []
    for k, s in enumerate(starts):
        co = str(tmp_path / ("co%d.elf" % k))
        open(co, "wb").write(data[s:starts[k + 1] if k + 1 < len(starts) else len(data)])
        out = subprocess.run([readelf, "-s", co], capture_output=True, text=True).stdout
        found += [l.split() for l in out.splitlines() if l.strip().endswith("scratch") and "OBJECT" in l]
    assert found and all(f[2] == str(size) and f[4] == "GLOBAL" for f in found), found


def test_error_codes_map_to_exceptions():
    e = ctypes.c_void_p()
    dt = (ctypes.c_int32 * 2)(99, 10)
    rc = runtime.lib.thx_elemwise_new(b"struct F{};", b"F", 1, 1, dt, ctypes.byref(e))
    assert rc == 3
    with pytest.raises(TypeError):
        runtime.check(rc)
    assert b"dtype" in runtime.lib.thx_last_error()


def test_dimension_mismatch_is_reported_before_any_launch(dry_run):
    x, y = T.fmatrix(), T.fmatrix()
    f = th.function([x, y], x + y)
    with pytest.raises(ValueError, match="Input dimension mis-match"):
        f(np.zeros((2, 3), "float32"), np.zeros((3, 2), "float32"))
    with pytest.raises(ValueError, match="Input dimension mis-match"):
        f(np.zeros((2, 3), "float32"), np.zeros((1, 3), "float32"))  # extent 1 without the broadcast flag
    with pytest.raises(TypeError):
        f(np.zeros((2, 3), "float64"), np.zeros((2, 3), "float32"))
    with pytest.raises(TypeError):
        f(np.zeros((2, 3, 1), "float32"), np.zeros((2, 3), "float32"))


def test_c_level_shape_check(dry_run):
    # the library itself refuses mismatching extents, broadcast flag or not
    from theano_amd.hip.ops import HipElemwise
    from theano_amd import scalar as scal
    a = runtime.HipArray.empty((4, 5), "float32")
    b = runtime.HipArray.empty((4, 6), "float32")
    o = runtime.HipArray.empty((4, 5), "float32")
    x, y = T.fmatrix(), T.fmatrix()
    node = HipElemwise(scal.add).make_node(x, y)
    handle, _, _ = node.op._handle(node)
    ins = (runtime.thx_array * 2)()
    a.as_thx(ins[0]); b.as_thx(ins[1])
    outs = (runtime.thx_array * 1)()
    o.as_thx(outs[0])
    rc = runtime.lib.thx_elemwise_call(handle, ins, outs, runtime.THX_BROADCAST | runtime.THX_DRY_RUN)
    assert rc == 2 and b"mis-match" in runtime.lib.thx_last_error()


def test_a_host_scalar_without_an_address_is_refused(dry_run):
    # the planner itself reads a scalar passed from the host: a null base is refused even in a dry run,
    # where device arrays need no address
    from theano_amd.hip.ops import HipElemwise
    from theano_amd import scalar as scal
    x, y = T.fmatrix(), T.fscalar()
    node = HipElemwise(scal.add).make_node(x, y.dimshuffle("x", "x"))
    handle, _, _ = node.op._handle(node)
    a = runtime.HipArray.empty((4, 5), "float32")
    o = runtime.HipArray.empty((4, 5), "float32")
    ins = (runtime.thx_array * 2)()
    a.as_thx(ins[0])
    two = np.full((1, 1), 2.0, "float32")
    runtime.host_scalar_thx(two, 2, ins[1])
    outs = (runtime.thx_array * 1)()
    o.as_thx(outs[0])
    flags = runtime.THX_BROADCAST | runtime.THX_DRY_RUN
    assert runtime.lib.thx_elemwise_call(handle, ins, outs, flags) == 0
    ins[0].base = None
    outs[0].base = None
    assert runtime.lib.thx_elemwise_call(handle, ins, outs, flags) == 0
    ins[1].base = None
    assert runtime.lib.thx_elemwise_call(handle, ins, outs, flags) == 7
    assert b"no base address" in runtime.lib.thx_last_error()


def test_zero_length_max_raises(dry_run):
    x = T.fmatrix()
    f = th.function([x], x.max(axis=1))
    with pytest.raises(ValueError, match="zero-size"):
        f(np.zeros((3, 0), "float32"))
    g = th.function([x], x.sum(axis=1))
    assert g(np.zeros((3, 0), "float32")).shape == (3,)


def _plans(f, *args):
    f(*args)
    return hip.last_plan()


def test_every_kernel_family_compiles_for_gfx950(dry_run):
    x = T.fmatrix("x")
    r = T.frow("r")
    t4 = T.ftensor4("t")
    f32 = lambda *s: np.zeros(s, "float32")
    assert "|ew|nd1|" in _plans(th.function([x], T.exp(x) + 1), f32(64, 64))
    assert "|ew|nd2|" in _plans(th.function([x, r], x * r), f32(64, 64), f32(1, 64))
    assert "|rr|" in _plans(th.function([x], x.sum(axis=1)), f32(300, 500))
    assert "|rc|" in _plans(th.function([x], x.sum(axis=0)), f32(300, 512))
    p = _plans(th.function([x], x.sum()), f32(4096, 4096))
    assert "|rf|" in p or "|s" in p
    assert "|rr|" in _plans(th.function([t4], t4.sum(axis=(0, 2, 3))), f32(8, 16, 7, 7))
    assert "|rc|" in _plans(th.function([t4], t4.sum(axis=(0, 2))), f32(8, 16, 7, 8))
    t6 = T.TensorType("float32", (False,) * 6)("t6")
    assert "|rg|" in _plans(th.function([t6], t6.sum(axis=(0, 2, 4))), f32(3, 4, 5, 6, 7, 8))
    # every storage dtype goes through the elementwise and the reduction templates
    for dt in ("bool", "int8", "uint8", "int16", "uint16", "int32", "uint32", "int64", "uint64", "float16",
               "float32", "float64", "complex64", "complex128"):
        v = T.TensorType(dt, (False, False))("v")
        if dt.startswith("complex"):
            out = [v * v + 1, v.sum(axis=0), abs(v).max(axis=1)]
        elif dt == "bool":
            out = [v & v, T.any(v, axis=0), T.all(v, axis=1)]
        elif dt.startswith("float"):
            out = [v * v + 1, v.sum(axis=0), v.max(axis=1)]
        else:
            out = [(v % v) ^ v, v.sum(axis=0), v.min(axis=1)]
        th.function([v], out)(np.zeros((33, 40), dt))
    stats = hip.cache_stats()
    assert stats["compiled"] + stats["disk_hits"] > 0


def test_header_constants_match_the_binding():
    """Flag and dtype values written in include/thx_hip.h are the ones the ctypes
    binding uses."""
    header = open(os.path.join(ROOT, "include", "thx_hip.h")).read()
    defines = dict((k, int(v, 0)) for k, v in re.findall(r"#define\s+(THX_[A-Z_]+)\s+(0x[0-9a-fA-F]+|\d+)", header))
    for name in ("THX_BROADCAST", "THX_DRY_RUN", "THX_HOST_SCALAR", "THX_INDEX", "THX_REUSED"):
        assert defines[name] == getattr(runtime, name), name
    enum = re.search(r"THX_BOOL = 0.*?THX_NDTYPES = 14", header, re.S).group(0)
    codes = dict((k, int(v)) for k, v in re.findall(r"(THX_[A-Z0-9]+) = (\d+)", enum))
    from theano_amd import scalar as scal
    names = {"bool": "BOOL", "int8": "I8", "uint8": "U8", "int16": "I16", "uint16": "U16", "int32": "I32",
             "uint32": "U32", "int64": "I64", "uint64": "U64", "float16": "F16", "float32": "F32", "float64": "F64",
             "complex64": "C64", "complex128": "C128"}
    assert set(names) == set(scal.all_dtypes)
    for dt, short in names.items():
        assert scal.dtype_code(dt) == codes["THX_" + short], dt


def test_generated_sources_can_be_dumped(dry_run, tmp_path, monkeypatch):
    monkeypatch.setenv("THX_DUMP_DIR", str(tmp_path))
    x = T.fmatrix("x")
    th.function([x], T.tanh(x) * 3.5 + 0.25)(np.zeros((5, 77), "float32"))
    files = [f for f in os.listdir(str(tmp_path)) if f.endswith(".hip")]
    assert files and any("tanh" in open(os.path.join(str(tmp_path), f)).read() for f in files)


def test_product_never_touches_the_oracle_or_a_host_fallback():
    """Nothing under theano_amd/ imports, loads or names the oracle, NumPy
    never computes an op's result there (perform of every host op raises), and
    the binding refuses to import without the HIP library."""
    pkg = os.path.join(ROOT, "theano_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".h", ".hip")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("noracle", ""), os.path.join(dirpath, f)
    x = T.fmatrix("x")
    for var in (T.exp(x), T.sum(x, axis=0), T.max_and_argmax(x, axis=1)[1], x[1:3], x.reshape((-1,)),
                T.join(0, x, x), T.alloc(x, 2, 3, 4)):
        node = var.owner
        with pytest.raises(NotImplementedError):
            node.op.perform(node, [np.zeros((3, 4), "float32")] * len(node.inputs), [[None] for _ in node.outputs])
    src = open(os.path.join(pkg, "hip", "runtime.py")).read()
    assert "ctypes.CDLL" in src and "raise" in src[src.index("_LIB_PATH"):src.index("ctypes.CDLL")]


def _build_c_client(tmp_path):
    import subprocess
    exe = str(tmp_path / "abi_client")
    libdir = os.path.join(ROOT, "theano_amd", "csrc")
    cmd = ["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", os.path.join(ROOT, "tests", "abi_client.c"),
           "-I", os.path.join(ROOT, "include"), "-L", libdir, "-lthx_hip", "-lm", "-Wl,-rpath," + libdir, "-o", exe]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    return exe


def test_a_plain_c_host_binds_the_library(tmp_path):
    """include/thx_hip.h is valid C99 and a host written in C (tests/abi_client.c) can create an
    operation from functor text and have it planned and compiled; no Python, no C++ types."""
    import subprocess
    exe = _build_c_client(tmp_path)
    res = subprocess.run([exe, "dry"], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0 and res.stdout.strip().endswith("ok"), res.stdout + res.stderr
    assert "AxPlusB|e" in res.stdout


@pytest.mark.gpu
def test_the_c_host_runs_on_the_device(tmp_path):
    import subprocess
    exe = _build_c_client(tmp_path)
    res = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0 and res.stdout.strip().endswith("ok"), res.stdout + res.stderr


@pytest.mark.gpu
def test_device_operands_without_an_address_are_refused_before_any_launch():
    # every family of entry points: a null base behind a non-empty array comes back as THX_ERR_ARG, nothing runs
    from theano_amd.hip.ops import HipElemwise
    from theano_amd import scalar as scal
    runtime.init()
    a = runtime.HipArray.from_numpy(np.ones((4, 5), "float32"))
    b = runtime.HipArray.from_numpy(np.ones((4, 5), "float32"))
    o = runtime.HipArray.empty((4, 5), "float32")
    x, y = T.fmatrix(), T.fmatrix()
    node = HipElemwise(scal.add).make_node(x, y)
    handle, _, _ = node.op._handle(node)
    for which in ("in", "out"):
        ins = (runtime.thx_array * 2)()
        a.as_thx(ins[0]); b.as_thx(ins[1])
        outs = (runtime.thx_array * 1)()
        o.as_thx(outs[0])
        if which == "in":
            ins[1].base = None
        else:
            outs[0].base = None
        assert runtime.lib.thx_elemwise_call(handle, ins, outs, runtime.THX_BROADCAST) == 7
        assert b"no base address" in runtime.lib.thx_last_error()
    # the same operands with their addresses run
    ins = (runtime.thx_array * 2)()
    a.as_thx(ins[0]); b.as_thx(ins[1])
    outs = (runtime.thx_array * 1)()
    o.as_thx(outs[0])
    assert runtime.lib.thx_elemwise_call(handle, ins, outs, runtime.THX_BROADCAST) == 0
    np.testing.assert_array_equal(o.to_numpy(), np.full((4, 5), 2, "float32"))

    from theano_amd.hip import codegen
    src, name, acc_bytes = codegen.reduce_functor((scal.add,), ("float64",), ("float32",), ("float32",), None)
    codes = (ctypes.c_int32 * 2)(scal.dtype_code("float32"), scal.dtype_code("float32"))
    rhandle = ctypes.c_void_p()
    runtime.check(runtime.lib.thx_reduce_new(src.encode(), name.encode(), 1, 1, 0, codes, acc_bytes, ctypes.byref(rhandle)))
    mask = (ctypes.c_uint8 * 2)(0, 1)
    r = runtime.HipArray.empty((4,), "float32")
    for which in ("in", "out"):
        ins = (runtime.thx_array * 1)()
        a.as_thx(ins[0])
        outs = (runtime.thx_array * 1)()
        r.as_thx(outs[0])
        if which == "in":
            ins[0].base = None
        else:
            outs[0].base = None
        assert runtime.lib.thx_reduce_call(rhandle, ins, mask, outs, 0) == 7
        assert b"no base address" in runtime.lib.thx_last_error()
    runtime.lib.thx_reduce_free(rhandle)


def _damaged_cache_round_trip(tmp_path, dry):
    import subprocess
    import sys
    prog = ("import numpy as np, theano_amd as th, theano_amd.tensor as T\n"
            "from theano_amd import hip\n"
            "from theano_amd.hip import runtime\n"
            "hip.set_dry_run(%r)\n"
            "x = T.fvector()\n"
            "print(th.function([x], x * 3 + 1)(np.arange(5, dtype='float32')).tolist(), runtime.cache_stats())\n" % dry)
    env = dict(os.environ, THX_CACHE_DIR=str(tmp_path), PYTHONPATH=os.path.dirname(os.path.dirname(__file__)))

    def run():
        res = subprocess.run([sys.executable, "-c", prog], capture_output=True, text=True, timeout=300, env=env)
        assert res.returncode == 0, res.stdout + res.stderr
        assert dry or res.stdout.startswith("[1.0, 4.0, 7.0, 10.0, 13.0]"), res.stdout
        stats = eval(res.stdout[res.stdout.index("]") + 1:])
        return stats["compiled"], stats["disk_hits"]

    compiled, disk = run()
    files = sorted(tmp_path.glob("*.hsaco"))
    assert compiled >= 1 and disk == 0 and len(files) == compiled
    assert run() == (0, compiled)                           # served from the disk
    for k, f in enumerate(files):
        blob = f.read_bytes()
        f.write_bytes(blob[:len(blob) // 2] if k % 2 == 0 else b"not a code object")
    assert run() == (compiled, 0)                           # every one built again
    assert run() == (0, compiled)                           # and the files on the disk are good again
    blob = files[0].read_bytes()
    files[0].write_bytes(blob[:-1])                         # one byte short: the section table ends outside the file
    assert run()[0] == 1


def test_a_damaged_cached_code_object_is_rebuilt(tmp_path):
    """A file in the kernel cache that is not a whole code object (cut in half, one byte short, something else
    altogether) is never handed to the module loader: it is dropped and the kernel is compiled again."""
    _damaged_cache_round_trip(tmp_path, True)


@pytest.mark.gpu
def test_a_damaged_cached_code_object_is_rebuilt_and_runs(tmp_path):
    _damaged_cache_round_trip(tmp_path, False)
