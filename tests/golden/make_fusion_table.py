"""Writes ``fusion_table.json``: the 72 rows of the reference's elementwise-fusion test
(``theano/tensor/tests/test_opt.py:937-1112``) as data.  Each row names the symbolic
expression (in the operator API, over the variables below), the inputs it is compiled
with, the number of Elemwise nodes the reference expects after fusion, the NumPy
expression of the expected value and the expected dtype (for cast_policy 'custom').
The inputs are constant-filled arrays, as in the reference: fw = 1, fx = 2, fy = 3,
fz = 4 (float32), dw = 5 (float64), ix = 60, iy = 70, iz = 70 (int32); fv is a random
float32 vector of shape[0] entries and fs a random float32 scalar (seeded by the test).

    python tests/golden/make_fusion_table.py
"""
import json
import os

F4 = "fw, fx, fy, fz"
ROWS = [
    # expression, inputs, Elemwise nodes in the reference's fused graph, NumPy answer, dtype
    ("fx + fy + fz", "fx, fy, fz", 1, "fxv + fyv + fzv", "float32"),
    ("fx * fy * fz", "fx, fy, fz", 1, "fxv * fyv * fzv", "float32"),
    ("fx + fy * fz", "fx, fy, fz", 1, "fxv + fyv * fzv", "float32"),
    ("fx * fy + fz", "fx, fy, fz", 1, "fxv * fyv + fzv", "float32"),
    ("fw + fx + fy + fz", F4, 1, "fwv + fxv + fyv + fzv", "float32"),
    ("(fw + fx) + (fy + fz)", F4, 1, "fwv + fxv + fyv + fzv", "float32"),
    ("((fw + fx) + fy) + fz", F4, 1, "fwv + fxv + fyv + fzv", "float32"),
    ("(fw + (fx + fy)) + fz", F4, 1, "fwv + fxv + fyv + fzv", "float32"),
    ("(fw + (fx + fy) + fz)", F4, 1, "fwv + fxv + fyv + fzv", "float32"),
    ("fw + (fx + (fy + fz))", F4, 1, "fwv + fxv + fyv + fzv", "float32"),
    ("(fw + fx) + (fy + fz)", F4, 1, "fwv + fxv + fyv + fzv", "float32"),
    ("fw * fx * fy * fz", F4, 1, "fwv * fxv * fyv * fzv", "float32"),
    ("fw + fx * fy * fz", F4, 1, "fwv + fxv * fyv * fzv", "float32"),
    ("fx + fy * fz * fx", "fx, fy, fz", 1, "fxv + fyv * fzv * fxv", "float32"),
    ("fx * fy + fz + fy", "fx, fy, fz", 1, "fxv * fyv + fzv + fyv", "float32"),
    ("fx * fy * fz * fw + fx + fy + fz + fw", F4, 1, "fxv * fyv * fzv * fwv + fxv + fyv + fzv + fwv", "float32"),
    # with a constant
    ("(fw + fx) + (fy + fz) + 2.", F4, 1, "fwv + fxv + fyv + fzv + 2", "float32"),
    ("((fw + fx) + 2. + fy) + fz", F4, 1, "fwv + fxv + fyv + fzv + 2", "float32"),
    ("(fw + (fx + 2. + fy)) + fz", F4, 1, "fwv + fxv + fyv + fzv + 2", "float32"),
    ("(fw + (fx + fy) + 2 + fz)", F4, 1, "fwv + fxv + fyv + fzv + 2", "float32"),
    ("fw + (fx + (fy + fz) + 2.)", F4, 1, "fwv + fxv + fyv + fzv + 2", "float32"),
    ("2 + (fw + fx) + (fy + fz)", F4, 1, "fwv + fxv + fyv + fzv + 2", "float32"),
    # float32 mixed with float64
    ("2 + (dw + fx) + (fy + fz)", "dw, fx, fy, fz", 1, "dwv + fxv + fyv + fzv + 2", "float64"),
    ("2 + (fw + dw) + (fy + fz)", "fw, dw, fy, fz", 1, "fwv + dwv + fyv + fzv + 2", "float64"),
    ("2 + (fw + fx) + (dw + fz)", "fw, fx, dw, fz", 1, "fwv + fxv + dwv + fzv + 2", "float64"),
    ("2 + (fw + fx) + (fy + dw)", "fw, fx, fy, dw", 1, "fwv + fxv + fyv + dwv + 2", "float64"),
    # with an op that is not elementwise in between
    ("(fw + fx).sum() + (fw + fx) + (fy + fz)", F4, 2, "(fwv + fxv).sum() + fwv + fxv + fyv + fzv", "float32"),
    # other elementwise ops
    ("fx + fy + T.cos(fz)", "fx, fy, fz", 1, "fxv + fyv + np.cos(fzv)", "float32"),
    ("fx + fy + T.cosh(fz)", "fx, fy, fz", 1, "fxv + fyv + np.cosh(fzv)", "float32"),
    ("fx + fy + abs(fz)", "fx, fy, fz", 1, "fxv + fyv + np.absolute(fzv)", "float32"),
    ("ix + iy + abs(iz)", "ix, iy, iz", 1, "ixv + iyv + np.absolute(izv)", "int32"),
    ("fx + fy + T.log(fz)", "fx, fy, fz", 1, "fxv + fyv + np.log(fzv)", "float32"),
    ("fx + fy + T.log2(fz)", "fx, fy, fz", 1, "fxv + fyv + np.log2(fzv)", "float32"),
    ("fx + fy + T.log10(fz)", "fx, fy, fz", 1, "fxv + fyv + np.log10(fzv)", "float32"),
    ("fx + fy ** fz", "fx, fy, fz", 1, "fxv + fyv ** fzv", "float32"),
    ("fx + fy + T.exp(fz)", "fx, fy, fz", 1, "fxv + fyv + np.exp(fzv)", "float32"),
    ("fx - fy - fz", "fx, fy, fz", 1, "fxv - fyv - fzv", "float32"),
    ("fx - (fy / fz)", "fx, fy, fz", 1, "fxv - (fyv / fzv)", "float32"),
    ("fx - T.true_div(fy, 2)", "fx, fy", 1, "fxv - (fyv / 2)", "float32"),
    ("fx - T.true_div(fy, fz)", "fx, fy, fz", 1, "fxv - (fyv / fzv)", "float32"),
    ("fx - T.int_div(ix * 100, iy * 1000)", "fx, ix, iy", 1, "fxv - ((ixv * 100) // (iyv * 1000))", "float64"),
    ("fx - (fy / 2)", "fx, fy", 1, "fxv - (fyv / 2)", "float32"),
    ("fx - (fy % fz)", "fx, fy, fz", 1, "fxv - (fyv % fzv)", "float32"),
    ("fx - (fy > fz)", "fx, fy, fz", 1, "fxv - (fyv > fzv)", "float32"),
    ("fx - (fy >= fz)", "fx, fy, fz", 1, "fxv - (fyv >= fzv)", "float32"),
    ("fx - (fy < fz)", "fx, fy, fz", 1, "fxv - (fyv < fzv)", "float32"),
    ("fx - (fy <= fz)", "fx, fy, fz", 1, "fxv - (fyv <= fzv)", "float32"),
    ("fx - T.eq(fy, fz)", "fx, fy, fz", 1, "fxv - (fyv == fzv)", "float32"),
    ("fx - T.neq(fy, fz)", "fx, fy, fz", 1, "fxv - (fyv != fzv)", "float32"),
    ("fx - fy + T.tan(fz)", "fx, fy, fz", 1, "fxv - fyv + np.tan(fzv)", "float32"),
    ("fx - fy + T.tanh(fz)", "fx, fy, fz", 1, "fxv - fyv + np.tanh(fzv)", "float32"),
    ("fx - fy + T.sin(fz)", "fx, fy, fz", 1, "fxv - fyv + np.sin(fzv)", "float32"),
    ("fx - fy + T.sinh(fz)", "fx, fy, fz", 1, "fxv - fyv + np.sinh(fzv)", "float32"),
    ("fx - fy + T.sqr(fz)", "fx, fy, fz", 1, "fxv - fyv + (fzv * fzv)", "float32"),
    ("fx - fy + T.sqrt(fz)", "fx, fy, fz", 1, "fxv - fyv + np.sqrt(fzv)", "float32"),
    ("fx - fy + T.inv(fz)", "fx, fy, fz", 1, "fxv - fyv + (1 / fzv)", "float32"),
    ("fx - fy + T.neg(fz)", "fx, fy, fz", 1, "fxv - fyv + (-fzv)", "float32"),
    ("fx - fy + T.round(fz)", "fx, fy, fz", 1, "fxv - fyv + np.round(fzv)", "float32"),
    ("ix - iy + T.iround(fz)", "ix, iy, fz", 1, "ixv - iyv + np.round(fzv)", "int64"),
    # bit ops
    ("fx - T.or_(iy, iz)", "fx, iy, iz", 1, "fxv - (iyv | izv)", "float64"),
    ("fx - T.xor(iy, iz)", "fx, iy, iz", 1, "fxv - (iyv ^ izv)", "float64"),
    ("fx - T.and_(iy, iz)", "fx, iy, iz", 1, "fxv - (iyv & izv)", "float64"),
    ("fx - T.invert(iy)", "fx, iy", 1, "fxv - (~iyv)", "float64"),
    ("fx - T.cast(fy, dtype='float64')", "fx, fy", 1, "fxv - np.asarray(fyv, 'float64')", "float64"),
    ("T.pow(fx * fy + fz, fx * fy)", "fx, fy, fz", 1, "np.power(fxv * fyv + fzv, fxv * fyv)", "float32"),
    # fused with a dimshuffle
    ("fv + fy ** fz", "fv, fy, fz", 1, "fvv + fyv ** fzv", "float32"),
    ("fv - fy + T.tanh(fz)", "fv, fy, fz", 1, "fvv - fyv + np.tanh(fzv)", "float32"),
    # the same input many times
    ("T.mul(fx, fx, fx, fx)", "fx", 1, "fxv * fxv * fxv * fxv", "float32"),
    ("T.mul(fx, T.tan(fx), T.tan(fx))", "fx", 1, "fxv * np.tan(fxv) * np.tan(fxv)", "float32"),
    ("T.mul(fx, T.tan(fx), T.tan(fx), fx)", "fx", 1, "fxv * np.tan(fxv) * np.tan(fxv) * fxv", "float32"),
    ("T.mul(T.tan(fx), T.tan(fx), fx + fy)", "fx, fy", 1, "np.tan(fxv) * np.tan(fxv) * (fxv + fyv)", "float32"),
    # different broadcast pattern: not merged, that would duplicate computation
    ("fx * T.sin(fs)", "fx, fs", 2, "fxv * np.sin(fsv)", "float32"),
]

if __name__ == "__main__":
    rows = [{"row": k, "cite": "theano/tensor/tests/test_opt.py:964-1112, case %d" % k, "expr": e,
             "inputs": [n.strip() for n in i.split(",")], "elemwise_nodes": n, "numpy": a, "dtype": d}
            for k, (e, i, n, a, d) in enumerate(ROWS)]
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fusion_table.json")
    with open(path, "w") as f:
        json.dump(rows, f, indent=1)
    print(path, len(rows), "rows")
