"""Build libthx_hip.so in place with hipcc for gfx950.

Run as ``python -m theano_amd.csrc.build`` or through ``__graft_entry__.build()``.
The device headers under ``kernels/`` are embedded into the library as text
(they are compiled at run time by hipRTC), so the shared object is the only
file the Python side has to find.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
KERNEL_HEADERS = ["thx_common.h", "thx_special.h", "thx_reduce.h", "thx_elemwise.h", "thx_rowchain.h"]
SOURCES = ["thx_runtime.cpp", "thx_elemwise.cpp", "thx_reduce.cpp", "thx_rowchain.cpp", "thx_prelude.cpp"]
LIB = os.path.join(HERE, "libthx_hip.so")
# Packed FP32 instructions stay off in every translation unit of the library.
HIP_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def write_prelude():
    parts = []
    for name in KERNEL_HEADERS:
        path = os.path.join(HERE, "kernels", name)
        if not os.path.exists(path):
            continue
        with open(path) as f:
            text = f.read()
        parts.append("\n".join(l for l in text.splitlines() if l.strip() != "#pragma once"))
    body = "\n".join(parts) + "\n"
    assert ')THXSRC"' not in body
    out = os.path.join(HERE, "thx_prelude.inc")
    with open(out, "w") as f:
        f.write('R"THXSRC(' + body + ')THXSRC"\n')
    return out


def build(verbose=False):
    write_prelude()
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = [os.path.join(HERE, s) for s in SOURCES if os.path.exists(os.path.join(HERE, s))]
    cmd = [hipcc, "-x", "hip", "-O2", "-std=c++17", "-fPIC", "-shared"] + HIP_FLAGS + srcs + [
        "-o", LIB, "-L/opt/rocm/lib", "-lhiprtc", "-Wl,-rpath,/opt/rocm/lib"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
