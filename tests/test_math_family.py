"""The unary / binary math family on the apply engine (the "remaining apply
users" row: generic/THCTensorMathPointwise.cu:5-255,345-580,
generic/THCTensorMathPairwise.cu:116-258).

CPU part: the oracle's formulas are pinned against numpy (bit-exact where the
operation is exactly rounded in binary32, within 2 ulp of the float64 result
for libm functions). GPU part: the HIP path against the oracle on strided
operands -- bit-exact for the exactly rounded operations, 1e-5 relative (+1e-6
absolute) for the transcendental ones, whose device and host libm differ in
the last ulps (the reference's own tolerance is 1e-5, test/test.lua:13)."""
import numpy as np
import pytest

from tests.util import assert_bit_equal, contiguous_geometry, fill_storage, random_geometry

F32 = np.float32
EXACT1 = {
    "sqrt": (np.sqrt, (0.0, 9.0)), "ceil": (np.ceil, (-5, 5)), "floor": (np.floor, (-5, 5)),
    "trunc": (np.trunc, (-5, 5)), "neg": (np.negative, (-5, 5)), "abs": (np.abs, (-5, 5)),
    "sign": (np.sign, (-2, 2)), "cinv": (lambda x: F32(1) / x, (-4, 4)),
    "frac": (lambda x: x - np.trunc(x), (-9, 9)),
    "rsqrt": (lambda x: F32(1) / np.sqrt(x), (0.1, 9.0)),
    "round": (lambda x: np.where(x >= 0, np.floor(x + F32(0.5)), np.ceil(x - F32(0.5))).astype(F32), (-6, 6)),
}
LIBM1 = {
    "sigmoid": (lambda x: 1 / (1 + np.exp(-x)), (-8, 8)), "log": (np.log, (0.01, 50)),
    "log1p": (np.log1p, (-0.9, 50)), "exp": (np.exp, (-10, 10)), "cos": (np.cos, (-6, 6)),
    "acos": (np.arccos, (-1, 1)), "cosh": (np.cosh, (-5, 5)), "sin": (np.sin, (-6, 6)),
    "asin": (np.arcsin, (-1, 1)), "sinh": (np.sinh, (-5, 5)), "tan": (np.tan, (-1.4, 1.4)),
    "atan": (np.arctan, (-20, 20)), "tanh": (np.tanh, (-5, 5)),
}
SCALAR = {   # name -> (numpy formula of (x, v), v, exact?)
    "pow": [(lambda x, v: x, 1.0, True), (lambda x, v: x * x, 2.0, True),
            (lambda x, v: (x * x).astype(F32) * x, 3.0, True), (lambda x, v: F32(1) / x, -1.0, True),
            (lambda x, v: F32(1) / (x * x).astype(F32), -2.0, True),
            (lambda x, v: np.power(np.abs(x).astype(np.float64), v), 2.5, False)],
    "cmaxValue": [(lambda x, v: np.where(x > F32(v), x, F32(v)), 0.25, True)],
    "cminValue": [(lambda x, v: np.where(x < F32(v), x, F32(v)), 0.25, True)],
    "fmod": [(lambda x, v: np.fmod(x, F32(v)), 0.75, True)],
    "remainder": [(lambda x, v: x - F32(v) * np.floor(x / F32(v)), 0.75, True)],
    # shifts of floating types scale by 2^v (THCTensorMathPairwise.cu:436-462)
    "lshift": [(lambda x, v: x * F32(2.0 ** v), 3.0, True)],
    "rshift": [(lambda x, v: x / F32(2.0 ** v), 2.0, True)],
}
BINARY = {
    "cmax": (lambda a, b: np.where(a > b, a, b), True), "cmin": (lambda a, b: np.where(a < b, a, b), True),
    "cfmod": (np.fmod, True), "cremainder": (lambda a, b: a - b * np.floor(a / b), True),
    "atan2": (lambda a, b: np.arctan2(a.astype(np.float64), b.astype(np.float64)), False),
    "cpow": (lambda a, b: np.power(np.abs(a).astype(np.float64), b.astype(np.float64)), False),
    "clshift": (lambda a, b: a.astype(np.float64) * np.power(2.0, b.astype(np.float64)), False),
    "crshift": (lambda a, b: a.astype(np.float64) / np.power(2.0, b.astype(np.float64)), False),
}


def ulp_close(got, want64, ulps=2.0):
    want = want64.astype(F32)
    tol = ulps * np.spacing(np.abs(want)).astype(np.float64) + 1e-45
    return np.all(np.abs(got.astype(np.float64) - want64) <= tol + np.abs(want64) * 2.0 ** -24)


# ------------------------------------------------------------------ oracle --
@pytest.mark.parametrize("name", sorted(EXACT1))
def test_oracle_exact_unary(oracle, name):
    f, (lo, hi) = EXACT1[name]
    rng = np.random.default_rng(len(name))
    x = np.concatenate([rng.uniform(lo, hi, 4000), np.arange(lo, hi, 0.5)]).astype(F32)
    if name in ("cinv",):
        x = x[x != 0]
    out = oracle.View.empty(x.shape)
    oracle.pointwise("fn:" + name, out, oracle.View.of(x))
    with np.errstate(all="ignore"):
        assert_bit_equal(out.storage, f(x).astype(F32), name)


@pytest.mark.parametrize("name", sorted(LIBM1))
def test_oracle_libm_unary(oracle, name):
    f, (lo, hi) = LIBM1[name]
    x = np.random.default_rng(len(name)).uniform(lo, hi, 4000).astype(F32)
    out = oracle.View.empty(x.shape)
    oracle.pointwise("fn:" + name, out, oracle.View.of(x))
    assert ulp_close(out.storage, f(x.astype(np.float64))), name


def test_oracle_scalar_binary_lerp_clamp(oracle):
    rng = np.random.default_rng(3)
    x = rng.uniform(-4, 4, 3000).astype(F32)
    for name, cases in SCALAR.items():
        for f, v, exact in cases:
            xin = np.abs(x) + F32(0.1) if not exact else x
            out = oracle.View.empty(x.shape)
            oracle.pointwise("fn:" + name, out, oracle.View.of(xin), value=v)
            with np.errstate(all="ignore"):
                want = f(xin, v)
            if exact:
                assert_bit_equal(out.storage, want.astype(F32), "%s %g" % (name, v))
            else:
                assert ulp_close(out.storage, want, 4), name
    y = rng.uniform(0.2, 4, 3000).astype(F32) * np.where(rng.random(3000) < 0.5, -1, 1).astype(F32)
    for name, (f, exact) in BINARY.items():
        a = np.abs(x) + F32(0.1) if name == "cpow" else x
        out = oracle.View.empty(x.shape)
        oracle.pointwise("fn:" + name, out, oracle.View.of(a), oracle.View.of(y))
        with np.errstate(all="ignore"):
            want = f(a, y)
        if exact:
            assert_bit_equal(out.storage, want.astype(F32), name)
        else:
            assert ulp_close(out.storage, want, 4), name
    out = oracle.View.empty(x.shape)
    oracle.pointwise("lerp", out, oracle.View.of(x), oracle.View.of(y), value=0.3)
    assert_bit_equal(out.storage, x + (F32(0.3) * (y - x)).astype(F32), "lerp")
    oracle.pointwise("fn:clamp", out, oracle.View.of(x), value=-1.0, value2=2.0)
    assert_bit_equal(out.storage, np.clip(x, F32(-1), F32(2)), "clamp")
    oracle.pointwise("fn:tpow", out, oracle.View.of(x), value=2.0)
    assert ulp_close(out.storage, np.power(2.0, x.astype(np.float64)), 2)
    oracle.pointwise("fn:lgamma", out, oracle.View.of(np.abs(x) + F32(0.5)))
    from math import lgamma
    want = np.array([lgamma(float(t)) for t in (np.abs(x) + F32(0.5))])
    assert np.allclose(out.storage, want, rtol=2e-6, atol=2e-6)


# --------------------------------------------------------------------- GPU --
def _gpu_case(thc, oracle, rng, shape, lo, hi, kind="float"):
    dtype = np.float16 if kind == "half" else F32
    g_in = random_geometry(rng, shape)
    st = rng.uniform(lo, hi, g_in[0]).astype(dtype)
    return (thc.Tensor.from_storage(st, *g_in[1:], kind=kind), oracle.View(st.copy(), *g_in[1:]))


def _check(got, want, exact, what):
    if exact:
        assert_bit_equal(got, want, what)
    else:
        np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=1e-5,
                                   atol=1e-6, err_msg=what)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(EXACT1) + sorted(LIBM1) + ["lgamma"])
def test_gpu_unary(thc, oracle, name):
    exact = name in EXACT1
    lo, hi = (EXACT1.get(name) or LIBM1.get(name) or (None, (0.5, 6.0)))[1]
    rng = np.random.default_rng(len(name) * 7)
    for shape, inplace in (((5000,), False), ((40, 70), True), ((6, 7, 9), False)):
        dev, ref = _gpu_case(thc, oracle, rng, shape, lo, hi)
        if inplace:
            out, rout = dev, ref
        else:
            out, rout = thc.Tensor("float"), oracle.View.empty(shape)
        out.unary(name, dev)
        oracle.pointwise("fn:" + name, rout, ref)
        assert out.shape == tuple(shape)
        _check(out.numpy(), rout.numpy(), exact, name)


@pytest.mark.gpu
def test_gpu_scalar_binary_lerp_clamp_equal(thc, oracle):
    rng = np.random.default_rng(91)
    shape = (37, 65)
    for name, cases in SCALAR.items():
        for _, v, exact in cases:
            lo = 0.1 if not exact else -4
            dev, ref = _gpu_case(thc, oracle, rng, shape, lo, 4)
            out = thc.Tensor("float")
            out.pow(dev, v) if name == "pow" else out.scalar2(name, dev, v)
            rout = oracle.pointwise("fn:" + name, oracle.View.empty(shape), ref, value=v)
            _check(out.numpy(), rout.numpy(), exact, "%s %g" % (name, v))
    for name, (_, exact) in BINARY.items():
        a, ra = _gpu_case(thc, oracle, rng, shape, 0.1 if name == "cpow" else -4, 4)
        b, rb = _gpu_case(thc, oracle, rng, shape, 0.2, 4)
        out = thc.Tensor("float").binary(name, a, b)
        rout = oracle.pointwise("fn:" + name, oracle.View.empty(shape), ra, rb)
        _check(out.numpy(), rout.numpy(), exact, name)
        a.binary(name, a, b)                                   # in place
        _check(a.numpy(), rout.numpy(), exact, name + " in place")
    a, ra = _gpu_case(thc, oracle, rng, shape, -4, 4)
    b, rb = _gpu_case(thc, oracle, rng, shape, -4, 4)
    out = thc.Tensor("float").lerp(a, b, 0.3)
    assert_bit_equal(out.numpy(), oracle.pointwise("lerp", oracle.View.empty(shape), ra, rb, value=0.3).numpy())
    out = thc.Tensor("float").clamp(a, -1.0, 2.0)
    assert_bit_equal(out.numpy(), oracle.pointwise("fn:clamp", oracle.View.empty(shape), ra, value=-1.0,
                                                   value2=2.0).numpy())
    out = thc.Tensor("float").tpow(2.0, a)
    _check(out.numpy(), oracle.pointwise("fn:tpow", oracle.View.empty(shape), ra, value=2.0).numpy(), False, "tpow")
    # equal: same sizes and same elements
    c = a.clone()
    assert a.equal(c) and a.equal(a)
    c.add(c, 1.0)
    assert not a.equal(c)
    assert not a.equal(thc.Tensor.from_numpy(np.zeros((65, 37), F32)))
    assert a.t().equal(thc.Tensor.from_numpy(a.numpy().T.copy()))


@pytest.mark.gpu
def test_gpu_half_math(thc, oracle):
    rng = np.random.default_rng(92)
    for name, (lo, hi) in (("exp", (-3, 3)), ("abs", (-4, 4)), ("sqrt", (0, 9)), ("floor", (-5, 5))):
        dev, ref = _gpu_case(thc, oracle, rng, (33, 40), lo, hi, kind="half")
        out = thc.Tensor("half").unary(name, dev)
        want = oracle.pointwise("fn:" + name, oracle.View.empty((33, 40), np.float16), ref).numpy()
        got = out.numpy()
        if name == "exp":     # one half ulp of slack for the libm difference before rounding
            assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= np.spacing(np.abs(want)))
        else:
            assert_bit_equal(got, want, name)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half", "double", "byte", "char", "short", "int", "long"])
def test_gpu_equal_is_one_fused_reduction_on_dense_operands(thc, kind):
    """equal (generic/THCTensorMathPairwise.cu:235-258): same sizes and every element pair equal under
    the element type's ==, so NaN differs from NaN, -0 equals +0 and inf equals inf. Dense operands take
    the fused two-input whole-tensor reduction (no flags temporary); strided ones the two-pass form."""
    dt = {"float": np.float32, "half": np.float16, "double": np.float64, "byte": np.uint8, "char": np.int8,
          "short": np.int16, "int": np.int32, "long": np.int64}[kind]
    rng = np.random.default_rng(95)
    for n in (1, 5, 4099, (1 << 21) + 77):
        if kind in ("float", "half", "double"):
            x = rng.uniform(-4, 4, n).astype(dt)
        else:
            info = np.iinfo(dt)
            x = rng.integers(info.min, info.max, n, dtype=np.int64).astype(dt)
        a, b = thc.Tensor.from_numpy(x), thc.Tensor.from_numpy(x.copy())
        assert a.equal(b)
        assert thc.last_kernel() == "all"
        for pos in {0, n // 2, n - 1}:
            y = x.copy()
            y[pos] = dt(0) if x[pos] != 0 else dt(1)
            assert not a.equal(thc.Tensor.from_numpy(y)), (kind, n, pos)
    if kind in ("float", "half", "double"):
        z = np.array([0.0, 1.0, np.inf, -np.inf, 2.0], dt)
        assert thc.Tensor.from_numpy(z).equal(thc.Tensor.from_numpy(np.array([-0.0, 1.0, np.inf, -np.inf, 2.0], dt)))
        w = np.array([0.0, np.nan, 1.0], dt)
        assert not thc.Tensor.from_numpy(w).equal(thc.Tensor.from_numpy(w.copy()))
        assert not thc.Tensor.from_numpy(z).equal(thc.Tensor.from_numpy(np.array([0.0, 1.0, -np.inf, np.inf, 2.0], dt)))
    m = rng.integers(0, 100, (40, 30)).astype(dt)
    a = thc.Tensor.from_numpy(m)
    assert not a.equal(thc.Tensor.from_numpy(m.reshape(30, 40)))       # shape mismatch
    assert a.t().equal(thc.Tensor.from_numpy(np.ascontiguousarray(m.T)))   # strided operand: two passes
    assert not a.t().equal(thc.Tensor.from_numpy(np.ascontiguousarray(m.T) + dt(1)))
