"""Tensor-level API: types, elementwise functions and reductions."""
from .type import (TensorType, TensorVariable, TensorConstant, as_tensor_variable, constant, tensor, scalar, vector,
                   matrix, row, col, tensor3, tensor4, bscalar, bvector, bmatrix, wscalar, wvector, wmatrix, iscalar,
                   ivector, imatrix, itensor3, itensor4, lscalar, lvector, lmatrix, ltensor3, ltensor4, hscalar,
                   hvector, hmatrix, htensor3, htensor4, fscalar, fvector, fmatrix, frow, fcol, ftensor3, ftensor4,
                   dscalar, dvector, dmatrix, drow, dcol, dtensor3, dtensor4)
from . import type as _type
for _n in dir(_type):  # bscalar ... dtensor4 and friends
    if _n[0] in "bwilhfdcz" and _n[1:] in ("scalar", "vector", "matrix", "row", "col", "tensor3", "tensor4", "tensor5",
                                           "tensor6", "tensor7"):
        globals()[_n] = getattr(_type, _n)
    if _n.lstrip("fdil") in _type._PLURAL.values() or _n in ("tensor5", "tensor6", "tensor7"):
        globals()[_n] = getattr(_type, _n)
from .elemwise import DimShuffle, Elemwise, CAReduce, CAReduceDtype, Sum, Prod, All, Any
from .basic import *  # noqa: F401,F403
from .basic import Max, MaxAndArgmax, Min, ShapeFloat, makeKeepDims, cast, round  # noqa: F401
from . import nnet  # noqa: F401,E402
from .views import (Alloc, IncSubtensor, Join, Rebroadcast, Reshape, Subtensor, addbroadcast, alloc,  # noqa: F401,E402
                    concatenate, flatten, horizontal_stack, inc_subtensor, join, patternbroadcast, reshape,
                    set_subtensor, split, stack, subtensor, unbroadcast, vertical_stack)
