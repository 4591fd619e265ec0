"""What PyTorch's own ROCm kernels reach on the benchmark's shapes: an independent yardstick for the
streaming rates this library's kernels are measured against (not used by the library or its tests).

Times single library kernels only - copy, negation, addition, row / column sums, row maxima over a
float32 8192 x 8192 matrix and a row softmax over 32768 x 1024 - over rotating operands, with HIP events
around back-to-back launches, and prints microseconds per launch and algorithmic GB/s.

    python -m theano_amd.misc.torch_yardstick"""
import sys


def main():
    import torch
    dev = torch.device("cuda:0")
    n = 8192 * 8192
    xs = [torch.randn(n, device=dev) for _ in range(3)]
    ys = [torch.empty(n, device=dev) for _ in range(3)]
    ms = [x.view(8192, 8192) for x in xs]
    rs = [torch.empty(8192, device=dev) for _ in range(3)]
    sm = [torch.randn(32768, 1024, device=dev) for _ in range(3)]
    so = [torch.empty(32768, 1024, device=dev) for _ in range(3)]

    def timeit(fn, iters=60):
        for k in range(6):
            fn(k)
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for k in range(iters):
            fn(k)
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / iters * 1e3

    cases = [
        ("copy", lambda k: ys[k % 3].copy_(xs[k % 3]), 2 * n * 4),
        ("out = -x", lambda k: torch.neg(xs[k % 3], out=ys[k % 3]), 2 * n * 4),
        ("out = x + y", lambda k: torch.add(xs[k % 3], xs[(k + 1) % 3], out=ys[k % 3]), 3 * n * 4),
        ("sum(axis=1)", lambda k: torch.sum(ms[k % 3], dim=1, out=rs[k % 3]), n * 4),
        ("sum(axis=0)", lambda k: torch.sum(ms[k % 3], dim=0, out=rs[k % 3]), n * 4),
        ("max(axis=1)", lambda k: torch.amax(ms[k % 3], dim=1, out=rs[k % 3]), n * 4),
        ("softmax 32768 x 1024", lambda k: torch.softmax(sm[k % 3], dim=1, out=so[k % 3]), 2 * 32768 * 1024 * 4),
    ]
    for name, fn, nbytes in cases:
        t = timeit(fn)
        print("%-22s %7.1f us  %6.0f GB/s" % (name, t, nbytes / t / 1e3), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
