"""TEST INFRASTRUCTURE - not part of the product.

Builds ``oracle/_build/liboracle.so`` from the C restatements in this folder
with the reference's own compiler flags, ``-O3 -fno-math-errno -march=native
-fopenmp`` and no ``-ffast-math`` (``theano/gof/cc.py:942-958``,
``theano/gof/cmodule.py:1930-2239``).  ``oracle/_build/`` is not tracked.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["careduce.c", "cpu_backend.c", "libm_ref.c"]
LIB = os.path.join(HERE, "_build", "liboracle.so")


def build(verbose=False):
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    srcs = [os.path.join(HERE, s) for s in SOURCES if os.path.exists(os.path.join(HERE, s))]
    cmd = ["gcc", "-O3", "-fno-math-errno", "-march=native", "-fopenmp", "-fPIC", "-shared", "-std=gnu11",
           "-Wno-unknown-pragmas"] + srcs + ["-o", LIB, "-lm"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("gcc failed:\n" + res.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
