"""Process-wide settings, the counterpart of the few ``theano.config`` flags the
Elemwise / CAReduce path reads (``theano/configdefaults.py:40-87``).

``floatX`` defaults to float32 here (the reference defaults to float64): Python
float literals take this dtype, so float32 graphs stay float32.
"""
import contextlib
import os


class _Config(object):
    floatX = os.environ.get("THEANO_AMD_FLOATX", "float32")
    cast_policy = "custom"          # theano/configdefaults.py:65-76
    int_division = "int"            # x / y on two integer tensors; 'int', 'floatX' or 'raise'
    device = int(os.environ.get("THEANO_AMD_DEVICE", "0"))
    # Largest number of inputs a fused Elemwise may take: the kernel argument
    # block is 4096 bytes (same budget as theano/gpuarray/elemwise.py:44-83).
    max_fused_inputs = 32
    # sum(sqr(x - mean(x))) over float16 / float32 data becomes one pass of shifted sums
    # accumulated in float64, merged with the pass that computes the mean
    single_pass_variance = True
    # An elementwise result that several kernels read is recomputed inside each of them, instead of
    # written once and read back, when it costs a few ALU instructions and at most this many calls of
    # exp / log / sqrt / tanh / sigmoid
    duplicate_transcendentals = int(os.environ.get("THEANO_AMD_DUP_TRANSCENDENTALS", "1"))

    # sum(g * (x - m)) with m a result of a reduction over the same elements becomes sum(g * x) - m * sum(g)
    # (float64 accumulators only), and the two reductions then share one pass over memory
    merge_dependent_reductions = True

    # Islands of elementwise nodes and reductions over axes other than the last (the per-channel statistics
    # of batch normalisation) run as one kernel that keeps each kept index's reduce domain on chip
    held_chains = os.environ.get("THEANO_AMD_HELD_CHAINS", "1") != "0"

    # function(..., mode="check"): how far a result of the optimised function may be from the same graph run
    # one kernel per node, (rtol, atol) by result dtype.  A fused kernel keeps in float32 registers what the
    # separate kernels round to the storage type in between, hence the width of the float16 entry.
    check_mode_tolerance = {"float16": (1e-2, 1e-2), "float32": (1e-4, 1e-5), "float64": (1e-9, 1e-10),
                            "complex64": (1e-4, 1e-5), "complex128": (1e-9, 1e-10)}

    @contextlib.contextmanager
    def change_flags(self, **kw):
        old = {k: getattr(self, k) for k in kw}
        try:
            for k, v in kw.items():
                setattr(self, k, v)
            yield self
        finally:
            for k, v in old.items():
                setattr(self, k, v)


config = _Config()
