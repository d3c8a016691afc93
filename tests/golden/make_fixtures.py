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

# Hand-checked known answers for the integer types, double, comparisons, conversions and scans
# (C semantics on the element type: wrap-around, truncating division, fmod = sign of the dividend,
# remainder = sign of the divisor; conversions truncate toward zero).
typed = [
    {"kind": "byte", "op": "add", "a": [250, 1, 255], "b": [10, 2, 1], "expect": [4, 3, 0]},
    {"kind": "byte", "op": "sub", "a": [3, 0], "b": [5, 1], "expect": [254, 255]},
    {"kind": "byte", "op": "mul", "a": [16, 200], "b": [16, 2], "expect": [0, 144]},
    {"kind": "char", "op": "add", "a": [127, -128], "b": [1, -1], "expect": [-128, 127]},
    {"kind": "short", "op": "mul", "a": [300, -300], "b": [300, 300], "expect": [24464, -24464]},
    {"kind": "int", "op": "div", "a": [7, -7, 7, -7], "b": [2, 2, -2, -2], "expect": [3, -3, -3, 3]},
    {"kind": "int", "op": "fn:cfmod", "a": [7, -7, 7, -7], "b": [3, 3, -3, -3], "expect": [1, -1, 1, -1]},
    {"kind": "int", "op": "fn:cremainder", "a": [7, -7, 7, -7], "b": [3, 3, -3, -3], "expect": [1, 2, -2, -1]},
    {"kind": "int", "op": "add", "a": [2147483647], "b": [1], "expect": [-2147483648]},
    {"kind": "long", "op": "mul", "a": [4294967296, 3037000500], "b": [4294967296, 3037000500],
     "expect": [0, -9223372036709301616]},
    {"kind": "long", "op": "fn:cpow", "a": [3, -2, 2], "b": [4, 3, 62], "expect": [81, -8, 4611686018427387904]},
    {"kind": "short", "op": "fn:cbitand", "a": [0x0ff0, -1], "b": [0x00ff, 0x1234], "expect": [0x00f0, 0x1234]},
    {"kind": "byte", "op": "fn:clshift", "a": [1, 0x81], "b": [7, 1], "expect": [128, 2]},
    {"kind": "char", "op": "fn:crshift", "a": [-128, 64], "b": [2, 3], "expect": [-32, 8]},
    {"kind": "double", "op": "add", "a": [0.1, 1e308], "b": [0.2, 1e308], "expect": [0.30000000000000004, float("inf")]},
    {"kind": "double", "op": "div", "a": [1.0, -1.0], "b": [3.0, 0.0], "expect": [0.3333333333333333, float("-inf")]},
]
compare = [
    {"kind": "float", "cmp": "lt", "a": [1.0, 2.0, float("nan"), -0.0], "b": [2.0, 2.0, 1.0, 0.0], "expect": [1, 0, 0, 0]},
    {"kind": "float", "cmp": "ne", "a": [1.0, float("nan"), -0.0], "b": [1.0, float("nan"), 0.0], "expect": [0, 1, 0]},
    {"kind": "byte", "cmp": "gt", "a": [200, 5], "b": [100, 5], "expect": [1, 0]},       # unsigned: 200 > 100
    {"kind": "char", "cmp": "gt", "a": [-56, 5], "b": [100, 5], "expect": [0, 0]},       # signed: -56 < 100
    {"kind": "long", "cmp": "ge", "a": [9007199254740993, -1], "b": [9007199254740992, 0], "expect": [1, 0]},
    {"kind": "half", "cmp": "eq", "a": [1.0, 0.5], "b": [1.0, 0.25], "expect": [1, 0]},
]
convert = [
    {"src": "float", "dst": "int", "x": [2.9, -2.9, 0.5, -0.5, 1e9], "expect": [2, -2, 0, 0, 1000000000]},
    {"src": "double", "dst": "byte", "x": [0.99, 255.0, 128.5], "expect": [0, 255, 128]},
    {"src": "int", "dst": "byte", "x": [256, 257, -1, 511], "expect": [0, 1, 255, 255]},
    {"src": "long", "dst": "int", "x": [4294967297, -4294967295], "expect": [1, 1]},
    {"src": "char", "dst": "byte", "x": [-1, -128, 127], "expect": [255, 128, 127]},
    {"src": "byte", "dst": "char", "x": [255, 128, 127], "expect": [-1, -128, 127]},
    {"src": "int", "dst": "float", "x": [16777217, -16777219], "expect": [16777216.0, -16777220.0]},
    {"src": "long", "dst": "double", "x": [9007199254740993], "expect": [9007199254740992.0]},
    {"src": "float", "dst": "half", "x": [65519.0, 65520.0, 1.0009766], "expect": [65504.0, float("inf"), 1.0009765625]},
    {"src": "double", "dst": "float", "x": [0.1, 1e40], "expect": [0.10000000149011612, float("inf")]},
    {"src": "half", "dst": "long", "x": [2.5, -3.5, 2048.0], "expect": [2, -3, 2048]},
]
typed_reduce = [
    {"kind": "byte", "op": "sum", "shape": [2, 3], "dim": 1, "x": [100, 100, 100, 255, 1, 0], "expect": [44, 0]},
    {"kind": "byte", "op": "sumall", "shape": [2, 3], "x": [100, 100, 100, 255, 1, 0], "expect": 556},
    {"kind": "char", "op": "prod", "shape": [1, 3], "dim": 1, "x": [16, 16, 2], "expect": [0]},
    {"kind": "int", "op": "mean", "shape": [1, 4], "dim": 1, "x": [-1, -2, -3, -1], "expect": [-1]},   # -7 / 4 truncates
    {"kind": "long", "op": "max", "shape": [1, 4], "dim": 1, "x": [-5, 7, 7, 1], "expect": [7], "index": [2]},
    {"kind": "short", "op": "min", "shape": [3, 1], "dim": 0, "x": [4, -9, -9], "expect": [-9], "index": [2]},
    {"kind": "int", "op": "cumsum", "shape": [1, 4], "dim": 1, "x": [2147483647, 1, 1, -3],
     "expect": [2147483647, -2147483648, -2147483647, 2147483646]},
    {"kind": "byte", "op": "cumprod", "shape": [1, 4], "dim": 1, "x": [3, 5, 20, 2], "expect": [3, 15, 44, 88]},
    {"kind": "double", "op": "sum", "shape": [1, 3], "dim": 1, "x": [1e16, 1.0, -1e16], "expect": [1.0]},  # needs > 53 bits
]

out = {"pointwise": pointwise, "argmax": argmax, "sum": sums, "half": half, "typed": typed, "compare": compare,
       "convert": convert, "typed_reduce": typed_reduce}
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fixtures.json")
with open(path, "w") as f:
    json.dump(out, f)
print("wrote", path, os.path.getsize(path), "bytes")
