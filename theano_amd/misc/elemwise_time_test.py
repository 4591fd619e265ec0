"""Call time of a cheap and a costly elementwise function over a float vector, the measurement of
``theano/misc/elemwise_time_test.py:21-52``: ``2 * x + x * x`` and ``tanh(x)`` over N elements
(default 200 000, the reference's ``openmp_elemwise_minsize``), minimum over 1000 calls.

Two figures per function, both wall-clock time of one call as the caller sees it:
  host    a NumPy argument, a NumPy result (upload, one kernel, download: what the reference's
          script times on its CPU backend)
  device  a device-resident argument, the result left on the device, the call followed by a
          synchronisation (one kernel launch and its completion)

    python -m theano_amd.misc.elemwise_time_test [-N 200000] [--loops 1000] [--script]

``--script`` prints the four times on one line (cheap host, costly host, cheap device, costly
device), as the reference's ``--script`` prints its two."""
import argparse
import sys
import time

import numpy as np


def eval_time(call, loops=1000):
    """Minimum wall-clock time of ``call()`` over ``loops`` calls."""
    best = 1e10
    for _ in range(loops):
        t0 = time.perf_counter()
        call()
        dt = time.perf_counter() - t0
        best = dt if dt < best else best
    return best


def elemwise_op_time(N=200000, loops=1000, dtype="float32"):
    """((cheap host, costly host), (cheap device, costly device)) in seconds per call."""
    import theano_amd as th
    from theano_amd import hip, tensor as T
    from theano_amd.compile import Out
    from theano_amd.hip.runtime import HipArray

    x = T.TensorType(dtype, (False,))("x")
    v = np.random.default_rng(1235).random(N).astype(dtype)
    cheap, costly = 2 * x + x * x, T.tanh(x)
    host, device = [], []
    for expr in (cheap, costly):
        f = th.function([x], expr)
        f(v)                                   # compiles and loads the kernel
        host.append(eval_time(lambda: f(v), loops))
        g = th.function([x], Out(expr, device=True))
        d = HipArray.from_numpy(v)
        g(d)
        hip.sync()

        def on_device():
            g(d)
            hip.sync()
        device.append(eval_time(on_device, loops))
    return tuple(host), tuple(device)


def main(argv=None):
    p = argparse.ArgumentParser(description="Compute time for fast and slow elemwise operations")
    p.add_argument("-N", "--N", type=int, default=200000, help="Number of vector elements")
    p.add_argument("--loops", type=int, default=1000, help="Calls per measurement (the minimum is reported)")
    p.add_argument("--script", action="store_true", help="Print the times alone, on one line")
    o = p.parse_args(argv)
    host, device = elemwise_op_time(o.N, o.loops)
    if o.script:
        sys.stdout.write("%2.9f %2.9f %2.9f %2.9f\n" % (host + device))
    else:
        for name, h, d in zip(("Fast op", "Slow op"), host, device):
            print("%s  run time in %d loops was %2.9f sec (host argument and result), %2.9f sec (device-resident)"
                  % (name, o.loops, h, d))
    sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
