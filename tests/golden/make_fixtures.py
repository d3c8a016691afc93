"""Writes tests/golden/fixtures.json: small known-answer vectors for the
pointwise-apply / reduction path. cutorch ships no such vectors (its tests
compare against a live torch7 TH), so these come from closed forms evaluated
with numpy's IEEE binary32 arithmetic and hand-checked index answers -- not
from the oracle and not from the engine. Run: python tests/golden/make_fixtures.py
"""
import json
import os

import numpy as np

F32 = np.float32
rng = np.random.default_rng(20240607)


def bits(a):
    return np.ascontiguousarray(a, dtype=F32).view(np.uint32).tolist()


def view(st, off, size, stride):
    return np.lib.stride_tricks.as_strided(st[off:], shape=size, strides=tuple(4 * s for s in stride))


def operand(st, off, size, stride):
    return {"storage_bits": bits(st), "offset": off, "size": list(size), "stride": list(stride)}


pointwise = []


def add_case(name, op, value, geoms, fn):
    """geoms: [(storage_len, offset, size, stride)] for out, in0, in1, ..."""
    sts = [rng.standard_normal(g[0]).astype(F32) for g in geoms]
    sts[0][:] = np.nan
    vs = [view(s, g[1], g[2], g[3]) for s, g in zip(sts, geoms)]
    ops = [operand(s, g[1], g[2], g[3]) for s, g in zip(sts, geoms)]
    expect = sts[0].copy()
    view(expect, geoms[0][1], geoms[0][2], geoms[0][3])[...] = fn(*vs[1:], F32(value)).astype(F32)
    pointwise.append({"name": name, "op": op, "value": float(value), "operands": ops,
                      "expect_storage_bits": bits(expect)})


# c = a + b, contiguous
add_case("add_contig", "add", 1, [(12, 0, (3, 4), (4, 1))] * 3, lambda a, b, v: a + b)
# out = a:t() * b + d  (the strided-apply benchmark configuration in miniature)
add_case("addcmul_transposed", "addcmul", 1,
         [(20, 0, (4, 5), (5, 1)), (20, 0, (4, 5), (5, 1)), (20, 0, (4, 5), (1, 4)), (20, 0, (4, 5), (5, 1))],
         lambda d, a, b, v: d + (v * (a * b).astype(F32)).astype(F32))
# holes + offset: narrowed views inside bigger storages
add_case("cdiv_holes", "div", 0,
         [(40, 3, (3, 4), (12, 2)), (30, 1, (3, 4), (8, 1)), (24, 0, (3, 4), (1, 3))],
         lambda a, b, v: a / b)
# cadd with value != 1 : a + rn(v*b)
add_case("cadd_scaled", "cadd", 0.3,
         [(24, 0, (2, 3, 4), (12, 4, 1)), (24, 0, (2, 3, 4), (1, 2, 6)), (24, 0, (2, 3, 4), (12, 4, 1))],
         lambda a, b, v: a + (v * b).astype(F32))
# permute(3,2,1) in miniature
add_case("add_permuted_3d", "add", 1,
         [(60, 0, (5, 4, 3), (12, 3, 1)), (60, 0, (5, 4, 3), (1, 5, 20)), (60, 0, (5, 4, 3), (12, 3, 1))],
         lambda a, b, v: a + b)
# scalar divide is a true division
add_case("div_scalar", "divc", 3, [(7, 0, (7,), (1,)), (7, 0, (7,), (1,))], lambda a, v: a / v)

argmax = [
    {"name": "ties_8_and_16", "which": "max", "dim": 1, "shape": [1, 24],
     "x_bits": bits(np.where(np.isin(np.arange(24), (8, 16)), 5.0, 1.0)), "indices": [9],
     "values_bits": bits([5.0])},
    {"name": "all_equal", "which": "min", "dim": 1, "shape": [2, 6], "x_bits": bits(np.full(12, 2.5)),
     "indices": [1, 1], "values_bits": bits([2.5, 2.5])},
    {"name": "max_last", "which": "max", "dim": 0, "shape": [4, 2],
     "x_bits": bits([0, 9, 1, 9, 2, 3, 2, 9]), "indices": [3, 1], "values_bits": bits([2, 9])},
    {"name": "neg_inf_row", "which": "max", "dim": 1, "shape": [1, 3],
     "x_bits": bits([-np.inf] * 3), "indices": [1], "values_bits": bits([-np.inf])},
    {"name": "signed_zero_tie", "which": "max", "dim": 1, "shape": [1, 3],
     "x_bits": bits([-0.0, 0.0, -1.0]), "indices": [1], "values_bits": bits([-0.0])},
]

sums = [
    {"name": "sum_rows", "kind": "sum", "dim": 1, "shape": [2, 4], "x": [1, 2, 3, 4, 10, 20, 30, 40],
     "expect": [10.0, 100.0]},
    {"name": "sum_cols", "kind": "sum", "dim": 0, "shape": [2, 4], "x": [1, 2, 3, 4, 10, 20, 30, 40],
     "expect": [11.0, 22.0, 33.0, 44.0]},
    {"name": "norm2_345", "kind": "norm", "p": 2, "dim": 1, "shape": [2, 2], "x": [3, 4, 5, 12],
     "expect": [5.0, 13.0]},
    {"name": "norm1", "kind": "norm", "p": 1, "dim": 0, "shape": [3, 1], "x": [-1, 2, -3], "expect": [6.0]},
    {"name": "norm0", "kind": "norm", "p": 0, "dim": 0, "shape": [4, 1], "x": [0, 2, 0, -3], "expect": [2.0]},
    {"name": "mean", "kind": "mean", "dim": 1, "shape": [1, 4], "x": [1, 2, 3, 6], "expect": [3.0]},
    {"name": "prod", "kind": "prod", "dim": 1, "shape": [1, 4], "x": [1, -2, 3, 4], "expect": [-24.0]},
    {"name": "big_cancel", "kind": "sum", "dim": 1, "shape": [1, 3], "x": [16777216, 1, -16777216],
     "expect": [1.0]},   # exact only with an accumulator wider than binary32
]

half = []
for f in [1.0, 65504.0, 65520.0, 65519.0, 5.9604645e-08, 2.9802322e-08, 2.9802326e-08, 6.1035156e-05,
          6.0975552e-05, 0.1, -0.33333334, 1.0009766, 1.0004883, 1.0014648, 1e-10, 70000.0]:
    half.append({"f32_bits": int(np.float32(f).view(np.uint32)),
                 "f16_bits": int(np.float32(f).astype(np.float16).view(np.uint16))})

out = {"pointwise": pointwise, "argmax": argmax, "sum": sums, "half": half}
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fixtures.json")
with open(path, "w") as f:
    json.dump(out, f)
print("wrote", path, os.path.getsize(path), "bytes")
