"""Hand-checked known answers (tests/golden/fixtures.json, sections typed /
compare / convert / typed_reduce, plus the float sections on the GPU): the
oracle and the engine must both reproduce them."""
import json
import os

import numpy as np
import pytest

from tests.util import assert_bit_equal

with open(os.path.join(os.path.dirname(__file__), "golden", "fixtures.json")) as _f:
    FX = json.load(_f)
F32 = np.float32


def arr(oracle, kind, values):
    dt = oracle.NP_OF[kind]
    if kind in ("float", "double", "half"):
        return np.array(values, dtype=np.float64).astype(dt)
    return np.array([int(v) for v in values], dtype=object).astype(np.int64).astype(dt) if kind != "byte" else \
        np.array(values, dtype=np.int64).astype(dt)


def same(got, want, what):
    assert_bit_equal(np.ascontiguousarray(got).ravel(), np.ascontiguousarray(want).ravel(), what)


def test_oracle_reproduces_typed_fixtures(oracle):
    for c in FX["typed"]:
        a, b, want = (arr(oracle, c["kind"], c[k]) for k in ("a", "b", "expect"))
        out = oracle.typed_pointwise(c["op"], oracle.View(np.zeros_like(a)), oracle.View(a), oracle.View(b))
        same(out.storage, want, "%s %s" % (c["kind"], c["op"]))
    for c in FX["compare"]:
        a, b = arr(oracle, c["kind"], c["a"]), arr(oracle, c["kind"], c["b"])
        out = oracle.typed_compare(c["cmp"], oracle.View(np.zeros(len(a), np.uint8)), oracle.View(a), oracle.View(b))
        assert out.storage.tolist() == c["expect"], c
    for c in FX["convert"]:
        x, want = arr(oracle, c["src"], c["x"]), arr(oracle, c["dst"], c["expect"])
        out = oracle.typed_convert(oracle.View(np.zeros_like(want)), oracle.View(x))
        same(out.storage, want, "%s -> %s" % (c["src"], c["dst"]))
    for c in FX["typed_reduce"]:
        x = arr(oracle, c["kind"], c["x"]).reshape(c["shape"])
        v = oracle.View.of(x)
        if c["op"] == "sumall":
            assert oracle.typed_reduce_all("sum", v) == c["expect"]
        elif c["op"] in ("cumsum", "cumprod"):
            same(oracle.typed_scan_dim(v, c["dim"], c["op"] == "cumprod").numpy(), arr(oracle, c["kind"], c["expect"]), c["op"])
        elif c["op"] in ("max", "min"):
            vals, idx = oracle.typed_minmax_dim(c["op"], v, c["dim"])
            same(vals.numpy(), arr(oracle, c["kind"], c["expect"]), c["op"])
            assert idx.numpy().ravel().tolist() == c["index"]
        else:
            same(oracle.typed_reduce_dim(c["op"], v, c["dim"]).numpy(), arr(oracle, c["kind"], c["expect"]),
                 "%s %s" % (c["kind"], c["op"]))


GPU_OP = {"add": ("cadd", True), "sub": ("csub", True), "mul": ("cmul", False), "div": ("cdiv", False)}


@pytest.mark.gpu
def test_gpu_reproduces_typed_fixtures(thc, oracle):
    for c in FX["typed"]:
        a, b, want = (arr(oracle, c["kind"], c[k]) for k in ("a", "b", "expect"))
        da, db, out = thc.Tensor.from_numpy(a), thc.Tensor.from_numpy(b), thc.Tensor(c["kind"])
        if c["op"] in GPU_OP:
            name, scaled = GPU_OP[c["op"]]
            getattr(out, name)(da, 1, db) if scaled else getattr(out, name)(da, db)
        else:
            out.binary(c["op"].replace("fn:", ""), da, db)
        same(out.numpy(), want, "%s %s" % (c["kind"], c["op"]))
    for c in FX["compare"]:
        a, b = arr(oracle, c["kind"], c["a"]), arr(oracle, c["kind"], c["b"])
        out = thc.Tensor("byte").compare_tensor(c["cmp"], thc.Tensor.from_numpy(a), thc.Tensor.from_numpy(b))
        assert out.numpy().tolist() == c["expect"], c
    for c in FX["convert"]:
        x, want = arr(oracle, c["src"], c["x"]), arr(oracle, c["dst"], c["expect"])
        out = thc.Tensor(c["dst"]).resize((len(x),)).copy_from(thc.Tensor.from_numpy(x))
        same(out.numpy(), want, "%s -> %s" % (c["src"], c["dst"]))
    for c in FX["typed_reduce"]:
        x = arr(oracle, c["kind"], c["x"]).reshape(c["shape"])
        d = thc.Tensor.from_numpy(x)
        if c["op"] == "sumall":
            assert d.sumall() == c["expect"]
        elif c["op"] in ("cumsum", "cumprod"):
            same(getattr(thc.Tensor(c["kind"]), c["op"])(d, c["dim"]).numpy(), arr(oracle, c["kind"], c["expect"]), c["op"])
        elif c["op"] in ("max", "min"):
            vals, idx = thc.Tensor(c["kind"]), thc.Tensor("long")
            getattr(vals, c["op"])(idx, d, c["dim"])
            same(vals.numpy(), arr(oracle, c["kind"], c["expect"]), c["op"])
            assert idx.numpy().ravel().tolist() == c["index"]
        elif c["kind"] == "double":
            # a double accumulator cannot hold 1e16 + 1: within 1e-13 of the mass instead
            got = getattr(thc.Tensor("double"), c["op"])(d, c["dim"]).numpy().ravel()
            assert np.all(np.abs(got - np.array(c["expect"])) <= 1e-13 * np.abs(x).sum())
        else:
            same(getattr(thc.Tensor(c["kind"]), c["op"])(d, c["dim"]).numpy(), arr(oracle, c["kind"], c["expect"]),
                 "%s %s" % (c["kind"], c["op"]))


@pytest.mark.gpu
def test_gpu_reproduces_float_fixtures(thc):
    """The float sections of the fixtures through the C ABI: whole storages bit
    for bit for the pointwise cases, exact values and indices for the argmax
    cases, sums within 1e-5 of the mass."""
    for case in FX["pointwise"]:
        ts = []
        for t in case["operands"]:
            st = np.array(t["storage_bits"], dtype=np.uint32).view(F32)
            ts.append(thc.Tensor.from_storage(st, t["offset"], t["size"], t["stride"]))
        out, ins, v = ts[0], ts[1:], case["value"]
        op = case["op"]
        if op == "add":
            out.cadd(ins[0], 1.0, ins[1])
        elif op == "cadd":
            out.cadd(ins[0], v, ins[1])
        elif op == "addcmul":
            out.addcmul(ins[0], v, ins[1], ins[2])
        elif op == "div":
            out.cdiv(ins[0], ins[1])
        elif op == "divc":
            out.div(ins[0], v)
        else:
            raise AssertionError(op)
        same(out.storage_numpy(), np.array(case["expect_storage_bits"], dtype=np.uint32).view(F32), case["name"])
    for case in FX["argmax"]:
        x = np.array(case["x_bits"], dtype=np.uint32).view(F32).reshape(case["shape"])
        vals, idx = thc.Tensor("float"), thc.Tensor("long")
        getattr(vals, case["which"])(idx, thc.Tensor.from_numpy(x), case["dim"])
        assert idx.numpy().ravel().tolist() == case["indices"], case["name"]
        same(vals.numpy(), np.array(case["values_bits"], dtype=np.uint32).view(F32), case["name"])
    for case in FX["sum"]:
        x = np.array(case["x"], dtype=F32).reshape(case["shape"])
        d, out = thc.Tensor.from_numpy(x), thc.Tensor("float")
        if case["kind"] == "norm":
            out.norm(d, case["p"], case["dim"])
        else:
            getattr(out, case["kind"])(d, case["dim"])
        got = out.numpy().ravel().astype(np.float64)
        mass = np.abs(x).sum()
        assert np.all(np.abs(got - np.array(case["expect"])) <= 1e-5 * mass), case["name"]
    for case in FX["half"]:
        f = np.uint32(case["f32_bits"]).view(F32)
        assert thc.lib().THC_float2half(float(f)) == case["f16_bits"]
