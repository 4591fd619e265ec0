"""Writes ``reference_vectors.json``: the literal inputs and expected outputs
that the reference's own tests hold for the Elemwise / CAReduce / MaxAndArgmax
path, transcribed by hand from the cited lines (data only; the reference is not
imported).  ``tests/test_golden.py`` checks the oracle (CPU) and the HIP path
(GPU) against every entry.

    python tests/golden/make_vectors.py
"""
import json
import os

VECTORS = [
    {"name": "prod_axis1_with_zeros", "cite": "theano/tensor/tests/test_elemwise.py:640-654",
     "graph": "prod_axis1", "dtype": "float32",
     "input": [[1.0, 2.0, 3.0], [0.0, 5.0, 6.0], [0.0, 0.0, 9.0]], "expected": [6.0, 0.0, 0.0]},
    {"name": "prod_axis1_no_zeros", "cite": "theano/tensor/tests/test_elemwise.py:674-680",
     "graph": "prod_axis1", "dtype": "float32",
     "input": [[1, 2, 3], [4, 5, 6], [7, 8, 9]], "expected": [6, 120, 504]},
    {"name": "prod_without_zeros_axis1", "cite": "theano/tensor/tests/test_elemwise.py:704-709",
     "graph": "prod_without_zeros_axis1", "dtype": "float64",
     "input": [[1, 2, 3], [0, 5, 6], [0, 0, 9]], "expected": [6, 30, 9]},
    {"name": "prod_without_zeros_axis0", "cite": "theano/tensor/tests/test_elemwise.py:704-713",
     "graph": "prod_without_zeros_axis0", "dtype": "float64",
     "input": [[1, 2, 3], [0, 5, 6], [0, 0, 9]], "expected": [1, 10, 162]},
    {"name": "prod_grad_axis1_zeros_a", "cite": "theano/tensor/tests/test_elemwise.py:723-736",
     "graph": "prod_grad_axis1", "dtype": "float64",
     "input": [[1, 2, 3], [0, 5, 6], [0, 0, 9]], "expected": [[6.0, 3.0, 2.0], [30.0, 0.0, 0.0], [0.0, 0.0, 0.0]]},
    {"name": "prod_grad_axis1_zeros_b", "cite": "theano/tensor/tests/test_elemwise.py:723-740",
     "graph": "prod_grad_axis1", "dtype": "float64",
     "input": [[1, 2, 0], [0, 5, 6], [7, 8, 9], [9, 10, 0]],
     "expected": [[0.0, 0.0, 2.0], [30.0, 0.0, 0.0], [72.0, 63.0, 56.0], [0.0, 0.0, 90.0]]},
    {"name": "prod_grad_axis0_zeros", "cite": "theano/tensor/tests/test_elemwise.py:742-748",
     "graph": "prod_grad_axis0", "dtype": "float64",
     "input": [[1, 2, 0], [0, 5, 6], [7, 8, 9], [9, 10, 0]],
     "expected": [[0.0, 400.0, 0.0], [63.0, 160.0, 0.0], [0.0, 100.0, 0.0], [0.0, 80.0, 0.0]]},
    {"name": "prod_all_no_zeros_grad", "cite": "theano/tensor/tests/test_elemwise.py:682-689",
     "graph": "prod_all_no_zeros_grad", "dtype": "float64", "input": [[1, 2, 3], [4, 5, 6], [7, 8, 9]],
     "expected": [[362880.0, 181440.0, 120960.0], [90720.0, 72576.0, 60480.0], [51840.0, 45360.0, 40320.0]]},
    {"name": "prod_all_no_zeros_second_grad", "cite": "theano/tensor/tests/test_elemwise.py:682-694",
     "graph": "prod_all_no_zeros_second_grad", "dtype": "float64", "input": [[1, 2, 3], [4, 5, 6], [7, 8, 9]],
     "expected": [[663696.0, 422568.0, 301872.0], [233964.0, 190800.0, 161016.0], [139248.0, 122652.0, 109584.0]]},
    {"name": "sum_needs_float64_accumulator", "cite": "theano/tensor/tests/test_elemwise.py:953-966",
     "graph": "sum_all", "dtype": "float32", "input": [1e8, 1, -1e8], "expected": 1.0},
    {"name": "max_and_argmax_vector", "cite": "theano/tensor/tests/test_basic.py:3114-3119",
     "graph": "max_and_argmax_all", "dtype": "int64", "input": [1, 2, 3, 2, -6], "expected": [3, 2]},
    {"name": "max_and_argmax_two_axes", "cite": "theano/tensor/tests/test_basic.py:3304-3309",
     "graph": "max_and_argmax_axes_1_2", "dtype": "int64",
     "input": [[[0, 1, 2, 3], [4, 5, 6, 7]], [[8, 9, 10, 11], [12, 13, 14, 15]], [[16, 17, 18, 19], [20, 21, 22, 23]]],
     "expected": [[7, 15, 23], [7, 7, 7]]},
    {"name": "fused_composite_times_six", "cite": "theano/tensor/tests/test_opt.py:1355-1362",
     "graph": "x_times_2_times_3", "dtype": "float32", "input": [1, 2, 3], "expected": [6, 12, 18]},
    {"name": "fusion_table_add3", "cite": "theano/tensor/tests/test_opt.py:948-966 (fx, fy, fz filled with 2, 3, 4)",
     "graph": "add3", "dtype": "float32", "input": [2.0, 3.0, 4.0], "expected": 9.0},
    {"name": "fusion_table_true_div_int", "cite": "theano/tensor/tests/test_opt.py:948-961, 1017 (ix = 60, iy = 70, fx = 2)",
     "graph": "true_div_int_times_float", "dtype": "float32", "input": [60, 70, 2.0], "expected": 1.7142857},
    {"name": "int8_mod_and_intdiv_follow_python", "cite": "theano/tensor/tests/test_basic.py:878-896",
     "graph": "mod_intdiv_int8", "dtype": "int8", "input": [[-128, -7, -1, 0, 1, 7, 127], [3, -3, 5, -5, 127, -128, -1]],
     "expected": [[1, -1, 4, 0, 1, -121, 0], [-43, 2, -1, 0, 0, -1, -127]]},
]

if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")
    with open(path, "w") as f:
        json.dump(VECTORS, f, indent=1)
    print(path, len(VECTORS), "vectors")
