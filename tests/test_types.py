"""The element types beyond float/half (byte, char, short, int, long, double):
pointwise arithmetic, comparisons of all eight types, and type-converting
copies (the per-type expansion of generic/THCTensorMathPairwise.cu,
generic/THCTensorMathPointwise.cu, generic/THCTensorMathCompare{,T}.cu and the
copyCuda<Type> entries of generic/THCTensorCopy.h:16-24).

CPU half: the oracle (oracle/th_oracle_types.c) is pinned against numpy's
fixed-width integer arithmetic, float64 ufuncs and astype casts.
GPU half: the engine against the oracle, bit for bit on whole storages
(transcendental double functions within 4 ulp)."""
import numpy as np
import pytest

from tests.util import assert_bit_equal, contiguous_geometry, random_geometry

INT_KINDS = ["byte", "char", "short", "int", "long"]
WIDE_KINDS = INT_KINDS + ["double"]
ALL_KINDS = WIDE_KINDS + ["float", "half"]


def np_of(oracle, kind):
    return oracle.NP_OF[kind]


def minus_one(dt):
    return np.array(-1, np.int64).astype(dt)


def rand_storage(rng, kind, n, oracle, small=False):
    dt = np_of(oracle, kind)
    if kind in ("double", "float", "half"):
        return rng.uniform(-4, 4, n).astype(dt)
    info = np.iinfo(dt)
    if small:
        return rng.integers(max(info.min, -9), min(info.max, 9) + 1, n).astype(dt)
    pick = rng.integers(0, 3, n)
    wide = rng.integers(info.min, info.max, n, dtype=np.int64 if dt != np.uint8 else np.int64).astype(dt)
    narrow = rng.integers(max(info.min, -100), min(info.max, 100) + 1, n).astype(dt)
    edge = rng.choice(np.array([info.min, info.max, 0, 1, info.max - 1], dtype=dt), n)
    return np.where(pick == 0, wide, np.where(pick == 1, narrow, edge)).astype(dt)


def trunc_div(a, b):
    """C integer division (toward zero) on numpy integer arrays, exact."""
    a64, b64 = a.astype(object), b.astype(object) if isinstance(b, np.ndarray) else int(b)
    q = np.frompyfunc(lambda x, y: 0 if y == 0 else (abs(x) // abs(y)) * (1 if (x < 0) == (y < 0) else -1), 2, 1)(a64, b64)
    return np.array(q, dtype=object)


def wrap(obj_arr, dt):
    bits = np.iinfo(dt).bits
    m = np.frompyfunc(lambda x: int(x) & ((1 << bits) - 1), 1, 1)(obj_arr)
    return np.array(m, dtype=np.uint64).astype({8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}[bits]).view(
        {8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}[bits]).astype(dt) if dt == np.uint8 else \
        np.array(m, dtype=np.uint64).astype({8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}[bits]).view(dt)


# --------------------------------------------------------------- oracle pins --
@pytest.mark.parametrize("kind", INT_KINDS)
def test_oracle_integer_arithmetic_matches_numpy(oracle, kind):
    rng = np.random.default_rng(7)
    dt = np_of(oracle, kind)
    n = 4000
    a, b, c = (rand_storage(rng, kind, n, oracle) for _ in range(3))
    bnz = np.where(b == 0, dt(3), b)
    V = oracle.View
    v = int(dt(7))

    def run(op, *ins, **kw):
        return oracle.typed_pointwise(op, V(np.zeros(n, dt)), *[V(x.copy()) for x in ins], **kw).storage

    with np.errstate(over="ignore"):
        assert_bit_equal(run("add", a, b), a + b)
        assert_bit_equal(run("sub", a, b), a - b)
        assert_bit_equal(run("mul", a, b), a * b)
        assert_bit_equal(run("addc", a, value=v), a + dt(v))
        assert_bit_equal(run("mulc", a, value=v), a * dt(v))
        assert_bit_equal(run("cadd", a, b, value=v), a + dt(v) * b)
        assert_bit_equal(run("addcmul", a, b, c, value=v), a + dt(v) * (b * c))
        assert_bit_equal(run("div", a, bnz), wrap(trunc_div(a, bnz), dt))
        assert_bit_equal(run("divc", a, value=v), wrap(trunc_div(a, v), dt))
        assert_bit_equal(run("addcdiv", a, b, bnz, value=v), a + dt(v) * wrap(trunc_div(b, bnz), dt))
        # numpy has the same two conventions: fmod = sign of dividend, remainder = sign of divisor
        safe = bnz if kind == "byte" else np.where(bnz == -1, dt(5), bnz)
        assert_bit_equal(run("fn:cfmod", a, safe), np.fmod(a, safe))
        assert_bit_equal(run("fn:cremainder", a, safe), np.remainder(a, safe))
        assert_bit_equal(run("fn:fmod", a, value=v), np.fmod(a, dt(v)))
        assert_bit_equal(run("fn:remainder", a, value=v), np.remainder(a, dt(v)))
        assert_bit_equal(run("fn:cmax", a, b), np.maximum(a, b))
        assert_bit_equal(run("fn:cmin", a, b), np.minimum(a, b))
        assert_bit_equal(run("fn:cmaxValue", a, value=v), np.maximum(a, dt(v)))
        assert_bit_equal(run("fn:clamp", a, value=2, value2=50), np.clip(a, dt(2), dt(50)))
        assert_bit_equal(run("fn:abs", a), np.abs(a))
        assert_bit_equal(run("fn:sign", a), np.sign(a).astype(dt))
        if kind != "byte":
            assert_bit_equal(run("fn:neg", a), -a)
        assert_bit_equal(run("fn:bitand", a, value=v), a & dt(v))
        assert_bit_equal(run("fn:bitor", a, value=v), a | dt(v))
        assert_bit_equal(run("fn:cbitxor", a, b), a ^ b)
        assert_bit_equal(run("fn:lshift", a, value=3), np.left_shift(a, 3))
        assert_bit_equal(run("fn:rshift", a, value=2), np.right_shift(a, 2))
        e = rng.integers(0, 6, n).astype(dt)
        assert_bit_equal(run("fn:cpow", a, e), np.power(a, e))
        assert_bit_equal(run("fill", value=v), np.full(n, v, dt))


def test_oracle_double_arithmetic_matches_numpy(oracle):
    rng = np.random.default_rng(8)
    n = 3000
    a, b, c = (rng.uniform(-3, 3, n) for _ in range(3))
    V = oracle.View

    def run(op, *ins, **kw):
        return oracle.typed_pointwise(op, V(np.zeros(n)), *[V(x.copy()) for x in ins], **kw).storage

    assert_bit_equal(run("add", a, b), a + b)
    assert_bit_equal(run("div", a, b), a / b)
    assert_bit_equal(run("cadd", a, b, value=0.3), a + 0.3 * b)
    assert_bit_equal(run("addcmul", a, b, c, value=0.7), a + 0.7 * (b * c))
    assert_bit_equal(run("lerp", a, b, value=0.25), a + 0.25 * (b - a))
    assert_bit_equal(run("fn:sqrt", np.abs(a)), np.sqrt(np.abs(a)))
    assert_bit_equal(run("fn:floor", a), np.floor(a))
    assert_bit_equal(run("fn:cfmod", a, b), np.fmod(a, b))
    assert_bit_equal(run("fn:cremainder", a, b), a - b * np.floor(a / b))
    assert_bit_equal(run("fn:clamp", a, value=-1.0, value2=0.5), np.clip(a, -1.0, 0.5))
    np.testing.assert_allclose(run("fn:exp", a), np.exp(a), rtol=4e-16)
    np.testing.assert_allclose(run("fn:tanh", a), np.tanh(a), rtol=1e-15, atol=1e-300)
    np.testing.assert_allclose(run("fn:atan2", a, b), np.arctan2(a, b), rtol=1e-15)
    np.testing.assert_allclose(run("fn:cpow", np.abs(a), b), np.power(np.abs(a), b), rtol=1e-14)


@pytest.mark.parametrize("kind", ALL_KINDS)
def test_oracle_compare_matches_numpy(oracle, kind):
    rng = np.random.default_rng(9)
    dt = np_of(oracle, kind)
    n = 2000
    a = rand_storage(rng, kind, n, oracle, small=True)
    b = rand_storage(rng, kind, n, oracle, small=True)
    ops = {"lt": np.less, "gt": np.greater, "le": np.less_equal, "ge": np.greater_equal, "eq": np.equal,
           "ne": np.not_equal}
    v = dt(2)
    for name, f in ops.items():
        got = oracle.typed_compare(name, oracle.View(np.zeros(n, np.uint8)), oracle.View(a), oracle.View(b))
        assert_bit_equal(got.storage, f(a, b).astype(np.uint8), name)
        got = oracle.typed_compare(name, oracle.View(np.zeros(n, dt)), oracle.View(a), value=v)
        assert_bit_equal(got.storage, f(a, v).astype(dt), name + " value")


def conv_source(rng, oracle, src, dst, n):
    """Values of kind `src` that convert to `dst` without undefined behaviour."""
    sdt, ddt = np_of(oracle, src), np_of(oracle, dst)
    if src in ("float", "double", "half"):
        if dst in ("float", "double", "half"):
            return rng.uniform(-1000, 1000, n).astype(sdt)
        lo, hi = (0, 200) if dst == "byte" else (-100, 100)
        return rng.uniform(lo, hi, n).astype(sdt)
    return rand_storage(rng, src, n, oracle, small=(dst == "half"))


@pytest.mark.parametrize("src", ALL_KINDS)
def test_oracle_convert_matches_numpy_astype(oracle, src):
    rng = np.random.default_rng(10)
    n = 1500
    for dst in ALL_KINDS:
        x = conv_source(rng, oracle, src, dst, n)
        got = oracle.typed_convert(oracle.View(np.zeros(n, np_of(oracle, dst))), oracle.View(x.copy())).storage
        if dst == "half" and src == "double":
            want = x.astype(np.float32).astype(np.float16)      # through float, as the reference does
        elif dst == "half" and src in INT_KINDS:
            want = x.astype(np.float32).astype(np.float16)
        else:
            want = x.astype(np_of(oracle, dst))
        assert_bit_equal(got, want, "%s -> %s" % (src, dst))


# ------------------------------------------------------------------ GPU parity --
def dev_ref(thc, oracle, rng, kind, geom, small=False):
    st = rand_storage(rng, kind, geom[0], oracle, small)
    return thc.Tensor.from_storage(st, *geom[1:], kind=kind), oracle.View(st.copy(), *geom[1:])


def whole(dev, ref, what, ulp=0):
    got, want = dev.storage_numpy(), ref.storage
    if ulp == 0:
        assert_bit_equal(got, want, what)
    else:
        ok = np.isclose(got, want, rtol=ulp * 2.3e-16, atol=0, equal_nan=True)
        assert ok.all(), (what, got[~ok][:3], want[~ok][:3])


BIN_OPS = ["add", "sub", "mul", "div", "fn:cmax", "fn:cmin", "fn:cfmod", "fn:cremainder", "fn:cpow",
           "fn:clshift", "fn:crshift"]
BIT_OPS = ["fn:cbitand", "fn:cbitor", "fn:cbitxor"]
GPU_NAME = {"add": "cadd", "sub": "csub", "mul": "cmul", "div": "cdiv"}


@pytest.mark.gpu
@pytest.mark.parametrize("kind", WIDE_KINDS)
def test_gpu_binary_ops_random_geometry(thc, oracle, kind):
    rng = np.random.default_rng(100)
    ops = BIN_OPS + (BIT_OPS if kind != "double" else [])
    for trial in range(6):
        nd = int(rng.integers(1, 4))
        shape = tuple(int(x) for x in rng.integers(1, 40, nd))
        for op in ops:
            small = op in ("fn:cpow", "fn:clshift", "fn:crshift")
            ga, gb, go = (random_geometry(rng, shape, permute=trial % 2 == 1) for _ in range(3))
            da, ra = dev_ref(thc, oracle, rng, kind, ga, small)
            db, rb = dev_ref(thc, oracle, rng, kind, gb, small)
            do, ro = dev_ref(thc, oracle, rng, kind, go)
            if small and kind != "double":       # exponents / shift counts 0..5
                stb = rng.integers(0, 6, gb[0]).astype(np_of(oracle, kind))
                db, rb = thc.Tensor.from_storage(stb, *gb[1:], kind=kind), oracle.View(stb.copy(), *gb[1:])
            if kind == "double" and op == "fn:cpow":
                sta = np.abs(ra.storage) + 0.1
                da, ra = thc.Tensor.from_storage(sta, *ga[1:], kind=kind), oracle.View(sta.copy(), *ga[1:])
            if op in ("div", "fn:cfmod", "fn:cremainder") and kind != "double":   # keep away from x/0, x%-1
                stb = rb.storage.copy()
                stb[(stb == 0) | (stb == minus_one(np_of(oracle, kind)))] = 3
                db, rb = thc.Tensor.from_storage(stb, *gb[1:], kind=kind), oracle.View(stb.copy(), *gb[1:])
            name = GPU_NAME.get(op, op.replace("fn:", ""))
            if name in ("cadd", "csub"):
                getattr(do, name)(da, 1, db)
            else:
                do.binary(name, da, db)
            oracle.typed_pointwise(op, ro, ra, rb)
            whole(do, ro, "%s %s %s" % (kind, op, shape), ulp=4 if (kind == "double" and small) else 0)     # pow() on the device vs libm


@pytest.mark.gpu
@pytest.mark.parametrize("kind", WIDE_KINDS)
def test_gpu_scalar_unary_ternary_ops(thc, oracle, kind):
    rng = np.random.default_rng(101)
    dt = np_of(oracle, kind)
    v = 3 if kind != "double" else 1.75
    for trial in range(4):
        shape = tuple(int(x) for x in rng.integers(1, 50, int(rng.integers(1, 4))))
        geoms = [random_geometry(rng, shape, permute=trial % 2 == 1) for _ in range(4)]
        for op, call in (("addc", lambda o, a: o.add(a, v)), ("subc", lambda o, a: o.sub(a, v)),
                         ("mulc", lambda o, a: o.mul(a, v)), ("divc", lambda o, a: o.div(a, v)),
                         ("fn:fmod", lambda o, a: o.scalar2("fmod", a, v)),
                         ("fn:remainder", lambda o, a: o.scalar2("remainder", a, v)),
                         ("fn:cmaxValue", lambda o, a: o.scalar2("cmaxValue", a, v)),
                         ("fn:cminValue", lambda o, a: o.scalar2("cminValue", a, v)),
                         ("fn:lshift", lambda o, a: o.scalar2("lshift", a, v if kind != "double" else 3)),
                         ("fn:rshift", lambda o, a: o.scalar2("rshift", a, v if kind != "double" else 3))):
            da, ra = dev_ref(thc, oracle, rng, kind, geoms[0])
            do, ro = dev_ref(thc, oracle, rng, kind, geoms[1])
            call(do, da)
            vv = 3 if (kind == "double" and "shift" in op) else v
            oracle.typed_pointwise(op, ro, ra, value=vv)
            whole(do, ro, "%s %s" % (kind, op))
        for fn in ("abs", "sign") + (("neg",) if kind != "byte" else ()):
            da, ra = dev_ref(thc, oracle, rng, kind, geoms[0])
            do, ro = dev_ref(thc, oracle, rng, kind, geoms[1])
            do.unary(fn, da)
            oracle.typed_pointwise("fn:" + fn, ro, ra)
            whole(do, ro, "%s %s" % (kind, fn))
        da, ra = dev_ref(thc, oracle, rng, kind, geoms[0])
        do, ro = dev_ref(thc, oracle, rng, kind, geoms[1])
        do.clamp(da, 2, 60)
        oracle.typed_pointwise("fn:clamp", ro, ra, value=2, value2=60)
        whole(do, ro, kind + " clamp")
        if kind != "double":
            for name in ("bitand", "bitor", "bitxor"):
                do.scalar2(name, da, 0x35)
                oracle.typed_pointwise("fn:" + name, ro, ra, value=0x35)
                whole(do, ro, kind + " " + name)
        # cadd / csub with a value, addcmul / addcdiv (out of place and in place on t)
        db, rb = dev_ref(thc, oracle, rng, kind, geoms[2])
        dc, rc = dev_ref(thc, oracle, rng, kind, geoms[3])
        if kind != "double":
            stc = rc.storage.copy()
            stc[(stc == 0) | (stc == minus_one(dt))] = 5
            dc, rc = thc.Tensor.from_storage(stc, *geoms[3][1:], kind=kind), oracle.View(stc.copy(), *geoms[3][1:])
        do.cadd(da, v, db)
        oracle.typed_pointwise("cadd", ro, ra, rb, value=v)
        whole(do, ro, kind + " cadd v")
        do.csub(da, v, db)
        oracle.typed_pointwise("cadd", ro, ra, rb, value=-v)
        whole(do, ro, kind + " csub v")
        do.addcmul(da, v, db, dc)
        oracle.typed_pointwise("addcmul", ro, ra, rb, rc, value=v)
        whole(do, ro, kind + " addcmul")
        da.addcdiv(da, v, db, dc)
        oracle.typed_pointwise("addcdiv", ra, ra, rb, rc, value=v)
        whole(da, ra, kind + " addcdiv in place")
        do.fill(v)
        oracle.typed_pointwise("fill", ro, value=v)
        whole(do, ro, kind + " fill")
        do.zero()
        oracle.typed_pointwise("fill", ro, value=0)
        whole(do, ro, kind + " zero")


@pytest.mark.gpu
def test_gpu_double_math_family(thc, oracle):
    rng = np.random.default_rng(102)
    geom = random_geometry(rng, (37, 29))
    pos = ("log", "sqrt", "rsqrt", "lgamma", "log1p")
    unit = ("acos", "asin")
    exact = ("sqrt", "ceil", "floor", "round", "trunc", "frac", "cinv", "neg", "abs", "sign", "rsqrt")
    for fn in oracle.FNS[:oracle.FNS.index("clamp")]:
        st = rng.uniform(-3, 3, geom[0])
        if fn in pos:
            st = np.abs(st) + 0.05
        if fn in unit:
            st = rng.uniform(-1, 1, geom[0])
        da = thc.Tensor.from_storage(st, *geom[1:], kind="double")
        ra = oracle.View(st.copy(), *geom[1:])
        do, ro = dev_ref(thc, oracle, rng, "double", contiguous_geometry((37, 29)))
        do.unary(fn, da)
        oracle.typed_pointwise("fn:" + fn, ro, ra)
        whole(do, ro, "double " + fn, ulp=0 if fn in exact else 8)
    da, ra = dev_ref(thc, oracle, rng, "double", geom)
    db, rb = dev_ref(thc, oracle, rng, "double", geom)
    do, ro = dev_ref(thc, oracle, rng, "double", geom)
    do.binary("atan2", da, db)
    oracle.typed_pointwise("fn:atan2", ro, ra, rb)
    whole(do, ro, "atan2", ulp=8)
    do.lerp(da, db, 0.3)
    oracle.typed_pointwise("lerp", ro, ra, rb, value=0.3)
    whole(do, ro, "lerp")
    do.pow(da, 2.0)
    oracle.typed_pointwise("mul", ro, ra, ra)
    whole(do, ro, "pow 2")
    do.tpow(1.7, da)
    oracle.typed_pointwise("fn:tpow", ro, ra, value=1.7)
    whole(do, ro, "tpow", ulp=8)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ALL_KINDS)
def test_gpu_compare_ops(thc, oracle, kind):
    rng = np.random.default_rng(103)
    dt = np_of(oracle, kind)
    for trial in range(3):
        shape = tuple(int(x) for x in rng.integers(1, 60, int(rng.integers(1, 4))))
        ga, gb = (random_geometry(rng, shape, permute=trial == 1) for _ in range(2))
        da, ra = dev_ref(thc, oracle, rng, kind, ga, small=True)
        db, rb = dev_ref(thc, oracle, rng, kind, gb, small=True)
        if kind in ("double", "float", "half"):          # make ties likely
            sta = np.round(ra.storage * 2) / 2
            stb = np.round(rb.storage * 2) / 2
            da, ra = thc.Tensor.from_storage(sta, *ga[1:], kind=kind), oracle.View(sta.astype(dt), *ga[1:])
            db, rb = thc.Tensor.from_storage(stb, *gb[1:], kind=kind), oracle.View(stb.astype(dt), *gb[1:])
        for cmp in ("lt", "gt", "le", "ge", "eq", "ne"):
            out = thc.Tensor("byte").compare_tensor(cmp, da, db)
            assert out.shape == shape
            want = oracle.typed_compare(cmp, oracle.View.empty(shape, np.uint8), ra, rb)
            assert_bit_equal(out.numpy(), want.numpy(), "%s %sTensor" % (kind, cmp))
            out = thc.Tensor(kind).compare_tensor(cmp, da, db, same_type=True)
            want = oracle.typed_compare(cmp, oracle.View.empty(shape, dt), ra, rb)
            assert_bit_equal(out.numpy(), want.numpy(), "%s %sTensorT" % (kind, cmp))
            out = thc.Tensor("byte").compare_value(cmp, da, 1)
            want = oracle.typed_compare(cmp, oracle.View.empty(shape, np.uint8), ra, value=1)
            assert_bit_equal(out.numpy(), want.numpy(), "%s %sValue" % (kind, cmp))
            out = thc.Tensor(kind).compare_value(cmp, da, 1, same_type=True)
            want = oracle.typed_compare(cmp, oracle.View.empty(shape, dt), ra, value=1)
            assert_bit_equal(out.numpy(), want.numpy(), "%s %sValueT" % (kind, cmp))
    with pytest.raises(thc.THCError, match="sizes do not match"):
        thc.Tensor("byte").compare_tensor("lt", thc.Tensor.from_numpy(np.zeros(4, dt)),
                                          thc.Tensor.from_numpy(np.zeros(5, dt)))


@pytest.mark.gpu
@pytest.mark.parametrize("src", ALL_KINDS)
def test_gpu_converting_copies(thc, oracle, src):
    rng = np.random.default_rng(104)
    for dst in ALL_KINDS:
        for shape, strided in (((1000,), False), ((13, 21), True), ((4099,), False)):
            gs = random_geometry(rng, shape) if strided else contiguous_geometry(shape)
            gd = random_geometry(rng, shape) if strided else contiguous_geometry(shape)
            st = conv_source(rng, oracle, src, dst, gs[0])
            dsrc = thc.Tensor.from_storage(st, *gs[1:], kind=src)
            rsrc = oracle.View(st.copy(), *gs[1:])
            std = rand_storage(rng, dst, gd[0], oracle)
            ddst = thc.Tensor.from_storage(std, *gd[1:], kind=dst)
            rdst = oracle.View(std.copy(), *gd[1:])
            ddst.copy_from(dsrc)
            oracle.typed_convert(rdst, rsrc)
            assert_bit_equal(ddst.storage_numpy(), rdst.storage, "%s -> %s %s" % (src, dst, shape))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["byte", "short", "int", "double"])
def test_gpu_same_type_copy_of_transposed_tensors(thc, oracle, kind):
    rng = np.random.default_rng(105)
    dt = np_of(oracle, kind)
    x = rand_storage(rng, kind, 300 * 260, oracle).reshape(300, 260)
    d = thc.Tensor.from_numpy(x)
    out = thc.Tensor(kind).resize((260, 300))
    out.copy(d.t())
    assert_bit_equal(out.numpy(), np.ascontiguousarray(x.T))
    assert thc.last_kernel().startswith("tiled")


# ------------------------------------------------------------------ reductions --
@pytest.mark.parametrize("kind", WIDE_KINDS)
def test_oracle_typed_reductions_match_numpy(oracle, kind):
    rng = np.random.default_rng(11)
    dt = np_of(oracle, kind)
    for shape, dim in (((5, 40), 1), ((30, 6), 0), ((3, 17, 4), 1)):
        geom = random_geometry(rng, shape)
        st = rand_storage(rng, kind, geom[0], oracle)
        v = oracle.View(st, *geom[1:])
        x = v.numpy()
        if kind == "double":
            np.testing.assert_allclose(oracle.typed_reduce_dim("sum", v, dim).numpy(), x.sum(axis=dim, keepdims=True),
                                       rtol=1e-13, atol=1e-13)
            np.testing.assert_allclose(oracle.typed_reduce_dim("mean", v, dim).numpy(), x.mean(axis=dim, keepdims=True),
                                       rtol=1e-13, atol=1e-13)
            import math
            assert abs(oracle.typed_reduce_all("sum", v) - math.fsum(x.ravel())) <= 1e-13 * np.abs(x).sum()
        else:
            with np.errstate(over="ignore"):
                want = x.astype(np.int64).sum(axis=dim, keepdims=True)           # wraps in 64 bits
                assert_bit_equal(oracle.typed_reduce_dim("sum", v, dim).numpy(), want.astype(dt), "sum")
                wantp = np.multiply.reduce(x.astype(np.int64), axis=dim, keepdims=True)
                assert_bit_equal(oracle.typed_reduce_dim("prod", v, dim).numpy(), wantp.astype(dt), "prod")
                assert oracle.typed_reduce_all("sum", v) == int(x.astype(np.int64).sum())
                s_t = want.astype(dt).astype(np.int64)
                n_t = int(np.array(shape[dim]).astype(dt))
                q = np.sign(s_t) * (np.abs(s_t) // n_t)                            # C division truncates
                assert_bit_equal(oracle.typed_reduce_dim("mean", v, dim).numpy(), q.astype(dt), "mean")
        assert_bit_equal(oracle.typed_reduce_dim("max", v, dim).numpy(), x.max(axis=dim, keepdims=True))
        assert_bit_equal(oracle.typed_reduce_dim("min", v, dim).numpy(), x.min(axis=dim, keepdims=True))
        xs = v.numpy()
        small = oracle.View.of((xs % 5).astype(dt) if kind != "double" else np.round(xs))   # many ties
        for which, f in (("max", np.argmax), ("min", np.argmin)):
            vals, idx = oracle.typed_minmax_dim(which, small, dim)
            assert np.array_equal(idx.numpy(), np.expand_dims(f(small.numpy(), axis=dim), dim) + 1)
            assert_bit_equal(vals.numpy(), getattr(small.numpy(), which)(axis=dim, keepdims=True))
        assert oracle.typed_reduce_all("max", v) == x.max() and oracle.typed_reduce_all("min", v) == x.min()


@pytest.mark.gpu
@pytest.mark.parametrize("kind", WIDE_KINDS)
def test_gpu_typed_reductions(thc, oracle, kind):
    rng = np.random.default_rng(106)
    dt = np_of(oracle, kind)
    shapes = [((7, 1024), 1), ((300, 64), 1), ((64, 512), 0), ((6, 300, 40), 1), ((3, 1 << 17), 1),
              ((2, 8192, 96), 1), ((5, 3), 0), ((1000, 17), 1), ((4097,), 0)]
    for trial, (shape, dim) in enumerate(shapes):
        geom = contiguous_geometry(shape) if trial < 6 else random_geometry(rng, shape)
        dev, ref = dev_ref(thc, oracle, rng, kind, geom)
        for op in ("sum", "prod", "mean"):
            if op == "mean" and kind != "double" and int(np.array(shape[dim]).astype(dt)) == 0:
                continue
            if op == "prod" and kind == "double":
                st = rng.uniform(0.9, 1.1, geom[0])
                dev2, ref2 = thc.Tensor.from_storage(st, *geom[1:], kind=kind), oracle.View(st.copy(), *geom[1:])
            else:
                dev2, ref2 = dev, ref
            got = getattr(thc.Tensor(kind), op)(dev2, dim).numpy()
            want = oracle.typed_reduce_dim(op, ref2, dim).numpy()
            if kind == "double":
                mass = np.abs(ref2.numpy()).sum(axis=dim, keepdims=True) if op != "prod" else np.abs(want)
                if op == "mean":
                    mass = mass / shape[dim]
                assert np.all(np.abs(got - want) <= 1e-13 * np.maximum(mass, 1e-300)), (kind, op, shape)
            else:
                assert_bit_equal(got, want, "%s %s %s" % (kind, op, shape))
        for which in ("max", "min"):
            small = (ref.numpy() % 7).astype(dt) if kind != "double" else np.round(ref.numpy())
            ds, rs = thc.Tensor.from_numpy(small), oracle.View.of(small)
            vals, idx = thc.Tensor(kind), thc.Tensor("long")
            getattr(vals, which)(idx, ds, dim)
            wv, wi = oracle.typed_minmax_dim(which, rs, dim)
            assert_bit_equal(vals.numpy(), wv.numpy(), "%s %s values %s" % (kind, which, shape))
            assert np.array_equal(idx.numpy(), wi.numpy()), (kind, which, shape)
            vals, idx = thc.Tensor(kind), thc.Tensor("long")
            getattr(vals, which)(idx, dev, dim)                  # full-range values
            wv, wi = oracle.typed_minmax_dim(which, ref, dim)
            assert_bit_equal(vals.numpy(), wv.numpy())
            assert np.array_equal(idx.numpy(), wi.numpy())
        if kind == "double":
            assert abs(dev.sumall() - oracle.typed_reduce_all("sum", ref)) <= 1e-13 * np.abs(ref.numpy()).sum()
            assert abs(dev.meanall() - oracle.typed_reduce_all("mean", ref)) <= 1e-13 * np.abs(ref.numpy()).mean()
        else:
            assert dev.sumall() == oracle.typed_reduce_all("sum", ref)
            assert dev.prodall() == oracle.typed_reduce_all("prod", ref)
            assert dev.meanall() == oracle.typed_reduce_all("mean", ref)
        assert dev.maxall() == oracle.typed_reduce_all("max", ref)
        assert dev.minall() == oracle.typed_reduce_all("min", ref)
        assert dev.equal(dev.clone())
        other = dev.clone()
        other.add(other, 1)
        assert not dev.equal(other)


@pytest.mark.gpu
def test_gpu_logicalall_any(thc):
    rng = np.random.default_rng(107)
    for n in (1, 1000, 1 << 20):
        x = np.ones(n, np.uint8) * 3
        t = thc.Tensor.from_numpy(x)
        assert t.logicalall() == 1 and t.logicalany() == 1
        x[int(rng.integers(0, n))] = 0
        t = thc.Tensor.from_numpy(x)
        assert t.logicalall() == 0 and t.logicalany() == (1 if n > 1 else 0)
        z = thc.Tensor.from_numpy(np.zeros(n, np.uint8))
        assert z.logicalall() == 0 and z.logicalany() == 0
    # the usual use: any(a > b)
    a = thc.Tensor.from_numpy(rng.standard_normal((50, 70)).astype(np.float32))
    m = thc.Tensor("byte").compare_value("gt", a, 10.0)
    assert m.logicalany() == 0
    m = thc.Tensor("byte").compare_value("lt", a, 10.0)
    assert m.logicalall() == 1


@pytest.mark.gpu
def test_gpu_double_norm_var_std_dist(thc, oracle):
    rng = np.random.default_rng(108)
    x = rng.uniform(-2, 2, (40, 300, 24))
    y = rng.uniform(-2, 2, (40, 300, 24))
    d, e = thc.Tensor.from_numpy(x), thc.Tensor.from_numpy(y)
    for dim in (0, 1, 2):
        np.testing.assert_allclose(thc.Tensor("double").norm(d, 2.0, dim).numpy(),
                                   np.sqrt((x * x).sum(axis=dim, keepdims=True)), rtol=1e-13)
        np.testing.assert_allclose(thc.Tensor("double").norm(d, 3.0, dim).numpy(),
                                   (np.abs(x) ** 3).sum(axis=dim, keepdims=True) ** (1 / 3.0), rtol=1e-12)
        np.testing.assert_allclose(thc.Tensor("double").var(d, dim).numpy(), x.var(axis=dim, ddof=1, keepdims=True),
                                   rtol=1e-12)
        np.testing.assert_allclose(thc.Tensor("double").std(d, dim, biased=1).numpy(),
                                   x.std(axis=dim, keepdims=True), rtol=1e-12)
    assert abs(d.normall(2.0) - np.sqrt((x * x).sum())) <= 1e-12 * np.sqrt((x * x).sum())
    assert abs(d.varall() - x.var(ddof=1)) <= 1e-12
    assert abs(d.stdall(1) - x.std()) <= 1e-12
    assert abs(d.dist(e, 2.0) - np.sqrt(((x - y) ** 2).sum())) <= 1e-11


# ------------------------------------------------------------ scans and renorm --
@pytest.mark.parametrize("kind", WIDE_KINDS)
def test_oracle_typed_scan_matches_numpy(oracle, kind):
    rng = np.random.default_rng(12)
    dt = np_of(oracle, kind)
    for shape, dim in (((4, 50), 1), ((30, 5), 0), ((3, 9, 4), 1)):
        geom = random_geometry(rng, shape)
        v = oracle.View(rand_storage(rng, kind, geom[0], oracle, small=True), *geom[1:])
        x = v.numpy()
        if kind == "double":
            np.testing.assert_allclose(oracle.typed_scan_dim(v, dim).numpy(), np.cumsum(x, axis=dim), rtol=1e-14, atol=1e-14)
            np.testing.assert_allclose(oracle.typed_scan_dim(v, dim, True).numpy(), np.cumprod(x, axis=dim), rtol=1e-13)
        else:
            with np.errstate(over="ignore"):
                assert_bit_equal(oracle.typed_scan_dim(v, dim).numpy(), np.cumsum(x.astype(np.int64), axis=dim).astype(dt))
                assert_bit_equal(oracle.typed_scan_dim(v, dim, True).numpy(),
                                 np.cumprod(x.astype(np.int64), axis=dim).astype(dt))


@pytest.mark.parametrize("kind", ["float", "double", "half"])
def test_oracle_renorm_matches_numpy(oracle, kind):
    rng = np.random.default_rng(13)
    dt = np_of(oracle, kind)
    x = rng.uniform(-2, 2, (6, 7, 5)).astype(dt)
    for dim, p in ((0, 2.0), (1, 1.0), (2, 3.0)):
        xd = x.astype(np.float64)
        other = tuple(d for d in range(3) if d != dim)
        norm = (np.abs(xd) ** p).sum(axis=other, keepdims=True) ** (1 / p)
        srt = np.sort(norm.ravel())
        maxnorm = float(srt[len(srt) // 2 - 1] + srt[len(srt) // 2]) / 2     # strictly between two norms
        got = oracle.renorm(oracle.View.of(x), p, dim, maxnorm).numpy().astype(np.float64)
        want = xd * np.where(norm > maxnorm, maxnorm / (norm + 1e-7), 1.0)
        assert (norm > maxnorm).any() and (norm <= maxnorm).any()
        np.testing.assert_allclose(got, want, rtol={"float": 1e-6, "double": 1e-14, "half": 1e-3}[kind])


@pytest.mark.gpu
@pytest.mark.parametrize("kind", WIDE_KINDS)
def test_gpu_typed_scans(thc, oracle, kind):
    rng = np.random.default_rng(109)
    for shape, dim in (((7, 1000), 1), ((300, 5), 1), ((50, 64), 0), ((4, 33, 20), 1), ((9000,), 0),
                       ((2, 1000, 24), 1), ((3, 300, 7), 1), ((5, 2049), 1)):
        geom = random_geometry(rng, shape) if len(shape) == 3 else contiguous_geometry(shape)
        dev, ref = dev_ref(thc, oracle, rng, kind, geom, small=(kind != "double"))
        got = thc.Tensor(kind).cumsum(dev, dim).numpy()
        want = oracle.typed_scan_dim(ref, dim).numpy()
        if kind == "double":
            mass = np.cumsum(np.abs(ref.numpy()), axis=dim)
            assert np.all(np.abs(got - want) <= 1e-13 * mass), (shape, dim)
            st = rng.uniform(0.95, 1.05, geom[0])
            dp, rp = thc.Tensor.from_storage(st, *geom[1:], kind=kind), oracle.View(st.copy(), *geom[1:])
            np.testing.assert_allclose(thc.Tensor(kind).cumprod(dp, dim).numpy(),
                                       oracle.typed_scan_dim(rp, dim, True).numpy(), rtol=1e-12)
        else:
            assert_bit_equal(got, want, "%s cumsum %s" % (kind, shape))
            assert_bit_equal(thc.Tensor(kind).cumprod(dev, dim).numpy(), oracle.typed_scan_dim(ref, dim, True).numpy(),
                             "%s cumprod %s" % (kind, shape))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "double", "half"])
def test_gpu_renorm(thc, oracle, kind):
    rng = np.random.default_rng(110)
    dt = np_of(oracle, kind)
    tol = {"float": 1e-5, "double": 1e-12, "half": 2e-3}[kind]
    for shape in ((6, 70, 5), (40, 33), (3, 4, 5, 6)):
        geom = random_geometry(rng, shape)
        st = rng.uniform(-2, 2, geom[0]).astype(dt)
        dev = thc.Tensor.from_storage(st, *geom[1:], kind=kind)
        ref = oracle.View(st.copy(), *geom[1:])
        for dim in range(len(shape)):
            for p in (1.0, 2.0, 3.0):
                x = ref.numpy().astype(np.float64)
                other = tuple(d for d in range(len(shape)) if d != dim)
                norms = np.sort((np.abs(x) ** p).sum(axis=other) ** (1 / p))
                k = len(norms) // 2                            # about half of the slices are scaled;
                maxnorm = float(norms[k - 1] + norms[k]) / 2   # never a tie with a slice's own norm
                got = thc.Tensor(kind).renorm(dev, p, dim, maxnorm)
                assert got.shape == tuple(shape)
                want = oracle.renorm(ref, p, dim, maxnorm).numpy().astype(np.float64)
                np.testing.assert_allclose(got.numpy().astype(np.float64), want, rtol=tol, atol=tol * 1e-3)
    t = thc.Tensor.from_numpy(np.ones((4, 4), dt))
    t.renorm(t, 2.0, 0, 1.0)                                  # in place
    np.testing.assert_allclose(t.numpy().astype(np.float64), np.full((4, 4), 0.5), rtol=2e-3)
    with pytest.raises(thc.THCError, match="at least 2 dimensions"):
        thc.Tensor(kind).renorm(thc.Tensor.from_numpy(np.ones(4, dt)), 2.0, 0, 1.0)
    with pytest.raises(thc.THCError, match="invalid dimension"):
        thc.Tensor(kind).renorm(thc.Tensor.from_numpy(np.ones((4, 4), dt)), 2.0, 2, 1.0)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "double", "half"])
def test_gpu_renorm_of_dense_rows_is_one_pass(thc, oracle, kind):
    """renorm over dim 0 of a contiguous tensor (the rows of an embedding
    table): norm, factor and scaling in one kernel that stages runs of rows in
    LDS. Short and long rows, a misaligned storage offset, in place, and a row
    too long for the staging buffer (which takes the general route)."""
    rng = np.random.default_rng(113)
    dt = np_of(oracle, kind)
    tol = {"float": 1e-5, "double": 1e-12, "half": 2e-3}[kind]
    for shape, fused in (((1000, 33), True), ((300, 128), True), ((50, 1000), True), ((7, 4096), True),
                         ((5, 3, 11), True), ((3, 1), True), ((2, 20000), False)):
        n = int(np.prod(shape))
        for off in (0, 1):
            st = rng.uniform(-2, 2, n + off).astype(dt)
            strides = [1] * len(shape)
            for d in range(len(shape) - 2, -1, -1):
                strides[d] = strides[d + 1] * shape[d + 1]
            dev = thc.Tensor.from_storage(st, off, shape, tuple(strides), kind=kind)
            ref = oracle.View(st.copy(), off, shape, tuple(strides))
            x = ref.numpy().astype(np.float64).reshape(shape[0], -1)
            for p in (1.0, 2.0, 3.0):
                norms = np.sort((np.abs(x) ** p).sum(axis=1) ** (1 / p))
                k = len(norms) // 2
                maxnorm = float(norms[k - 1] + norms[k]) / 2
                got = thc.Tensor(kind).renorm(dev, p, 0, maxnorm)
                assert (thc.last_kernel() == "renorm-rows") == fused, (shape, thc.last_kernel())
                want = oracle.renorm(ref, p, 0, maxnorm).numpy().astype(np.float64)
                np.testing.assert_allclose(got.numpy().astype(np.float64), want, rtol=tol, atol=tol * 1e-3)
            before = dev.storage_numpy().copy()
            dev.renorm(dev, 2.0, 0, 1e9)                         # nothing exceeds: bit-identical
            assert thc.last_kernel() == ("renorm-rows" if fused else thc.last_kernel())
            assert_bit_equal(dev.storage_numpy(), before)
            dev.renorm(dev, 2.0, 0, 0.5)                          # in place
            got = dev.numpy().astype(np.float64).reshape(shape[0], -1)
            np.testing.assert_allclose(np.minimum(np.sqrt((got ** 2).sum(axis=1)), 0.5),
                                       np.minimum(np.sqrt((x ** 2).sum(axis=1)), 0.5), rtol=max(tol, 1e-6) * 4)
            assert_bit_equal(dev.storage_numpy()[:off], before[:off])
    thc.set_tuning("renorm.rows", 0)
    try:
        thc.Tensor(kind).renorm(thc.Tensor.from_numpy(np.ones((8, 8), dt)), 2.0, 0, 1.0)
        assert thc.last_kernel() != "renorm-rows"
    finally:
        thc.set_tuning("renorm.rows", 1)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["int", "byte", "double"])
def test_gpu_transposed_input_of_wider_types_runs_on_lds_tiles(thc, oracle, kind):
    """add / sub / mul / cadd of int, long and double run on plain functors with
    every kernel of the engine, the specialised LDS-tiled ones included; everything
    else of the wider types (and all comparisons) meets a transposed input in the
    general LDS-tile kernel: one pass, nothing is densified."""
    rng = np.random.default_rng(111)
    dt = np_of(oracle, kind)
    a = rand_storage(rng, kind, 200 * 136, oracle).reshape(200, 136)
    b = rand_storage(rng, kind, 200 * 136, oracle).reshape(136, 200)
    da, db = thc.Tensor.from_numpy(a), thc.Tensor.from_numpy(b)
    out = thc.Tensor(kind).cadd(da.t(), 1, db)
    assert thc.last_kernel() == ("lds-tile-shift" if kind == "byte" else "tiled")   # 200 x 136 bytes: not whole 16-element packs
    ra = oracle.View(a.reshape(-1).copy(), 0, (136, 200), (1, 136))
    want = oracle.typed_pointwise("add", oracle.View.empty((136, 200), dt), ra, oracle.View.of(b))
    assert_bit_equal(out.numpy(), want.numpy())
    for name, op, value in (("cmul", "mul", 0), ("csub", "cadd", 3), ("cadd", "cadd", -7)):
        out = thc.Tensor(kind)
        if name == "cmul":
            out.cmul(da.t(), db)
        else:
            getattr(out, name)(da.t(), value, db)
        assert thc.last_kernel() == ("lds-tile-shift" if kind == "byte" else "tiled"), (name, thc.last_kernel())
        v = -value if name == "csub" else value
        want = oracle.typed_pointwise(op, oracle.View.empty((136, 200), dt), ra, oracle.View.of(b), value=v)
        assert_bit_equal(out.numpy(), want.numpy(), name)
    out = thc.Tensor(kind).cdiv(da.t(), thc.Tensor.from_numpy(np.where(b == 0, 1, b).astype(dt)))
    assert thc.last_kernel() == {"double": "tiled", "int": "lds-tile", "byte": "lds-tile-shift"}[kind]   # integer division is code-dispatched
    m = thc.Tensor("byte").compare_tensor("lt", da.t(), db)
    assert thc.last_kernel() == ("lds-tile-shift" if kind == "byte" else "lds-tile")
    wm = oracle.typed_compare("lt", oracle.View.empty((136, 200), np.uint8), ra, oracle.View.of(b))
    assert_bit_equal(m.numpy(), wm.numpy())
    f = thc.Tensor.from_numpy(rng.standard_normal((200, 136)).astype(np.float32))
    g = thc.Tensor.from_numpy(rng.standard_normal((136, 200)).astype(np.float32))
    # float into Byte owns the pack variant of the tiled kernel (4-byte output packs) ...
    m = thc.Tensor("byte").compare_tensor("ge", f.t(), g)
    assert thc.last_kernel() == "tiled"
    assert_bit_equal(m.numpy(), (f.numpy().T >= g.numpy()).astype(np.uint8))
    m = thc.Tensor("byte").compare_value("lt", f.t(), 0.25)
    assert thc.last_kernel() == "tiled"
    assert_bit_equal(m.numpy(), (f.numpy().T < np.float32(0.25)).astype(np.uint8))
    thc.force_64bit_index(True)
    try:
        m = thc.Tensor("byte").compare_tensor("ne", g, f.t())
        assert thc.last_kernel() == "tiled"
    finally:
        thc.force_64bit_index(False)
    assert_bit_equal(m.numpy(), (g.numpy() != f.numpy().T).astype(np.uint8))
    # ... and only that one: shapes whose rows are not whole aligned packs take the general LDS-tile
    # kernel, as does a comparison whose output has the input's type
    f2 = thc.Tensor.from_numpy(rng.standard_normal((201, 137)).astype(np.float32))
    g2 = thc.Tensor.from_numpy(rng.standard_normal((137, 201)).astype(np.float32))
    m = thc.Tensor("byte").compare_tensor("le", f2.t(), g2)
    assert thc.last_kernel() == "lds-tile-shift"
    assert_bit_equal(m.numpy(), (f2.numpy().T <= g2.numpy()).astype(np.uint8))
    mt = thc.Tensor("float").compare_tensor("gt", f.t(), g, same_type=True)
    assert thc.last_kernel() == "lds-tile"
    assert_bit_equal(mt.numpy(), (f.numpy().T > g.numpy()).astype(np.float32))
    # a transposed Byte OUTPUT of a float comparison (its memory order decides): 4-byte output packs along its rows
    mb = thc.Tensor.from_numpy(np.zeros((200, 136), np.uint8))
    mb.t().compare_tensor("lt", g, f.t())
    assert_bit_equal(mb.numpy().T, (g.numpy() < f.numpy().T).astype(np.uint8))


@pytest.mark.gpu
def test_gpu_transposed_output_and_math_family_run_on_lds_tiles(thc, oracle):
    """The same when it is the output that is transposed (its memory order
    decides), for a wider type and for the code-dispatched float math; 3-D
    permutations included. With the general kernel switched off the densify
    route (same-type copy into the output's order, then the op) still serves."""
    rng = np.random.default_rng(112)
    a = rng.integers(-1000, 1000, (136, 200)).astype(np.int32)
    b = rng.integers(-1000, 1000, (136, 200)).astype(np.int32)
    da, db = thc.Tensor.from_numpy(a), thc.Tensor.from_numpy(b)
    base = thc.Tensor.from_numpy(np.zeros((200, 136), np.int32))
    base.t().cadd(da, 3, db)
    assert thc.last_kernel().startswith("tiled")     # plain int arithmetic owns tiled kernels
    assert_bit_equal(base.numpy(), (a + 3 * b).T)
    base.t().cdiv(da, thc.Tensor.from_numpy(np.where(b == 0, 1, b).astype(np.int32)))
    assert thc.last_kernel() == "lds-tile"           # the code-dispatched family: the general LDS-tile kernel
    want_div = (a.astype(np.int64) / np.where(b == 0, 1, b)).astype(np.int64).astype(np.int32).T
    assert_bit_equal(base.numpy(), want_div)
    thc.set_tuning("apply.ldstile.enable", 0)
    try:
        base.fill(0)
        base.t().cdiv(da, thc.Tensor.from_numpy(np.where(b == 0, 1, b).astype(np.int32)))
        assert thc.last_kernel() == "contig"         # densified: copy into the output's order, then a flat op
    finally:
        thc.set_tuning("apply.ldstile.enable", 1)
    assert_bit_equal(base.numpy(), want_div)

    x = rng.standard_normal((136, 200)).astype(np.float32)
    y = rng.standard_normal((200, 136)).astype(np.float32)
    dx, dy = thc.Tensor.from_numpy(x), thc.Tensor.from_numpy(y)
    fbase = thc.Tensor.from_numpy(np.zeros((200, 136), np.float32))
    fbase.t().unary("exp", dx)          # one-input float math owns tiled kernels
    assert thc.last_kernel().startswith("tiled")
    want = oracle.pointwise("fn:exp", oracle.View.empty((136, 200)), oracle.View.of(x))
    np.testing.assert_allclose(fbase.numpy().T, want.numpy(), rtol=2e-6)
    out = thc.Tensor("float").binary("cmax", dx, dy.t())
    assert thc.last_kernel() == "lds-tile"
    assert_bit_equal(out.numpy(), np.maximum(x, y.T))
    fbase.t().binary("cmin", dx, dy.t())   # y is already in the output's order
    assert thc.last_kernel() == "lds-tile"
    assert_bit_equal(fbase.numpy().T, np.minimum(x, y.T))
    hx = x.astype(np.float16)
    hbase = thc.Tensor.from_numpy(np.zeros((200, 136), np.float16))
    hbase.t().unary("abs", thc.Tensor.from_numpy(hx))
    assert thc.last_kernel() == "lds-tile"
    assert_bit_equal(hbase.numpy().T, np.abs(hx))
    out = thc.Tensor("half").unary("neg", thc.Tensor.from_numpy(hx).t())
    assert thc.last_kernel() == "lds-tile"
    assert_bit_equal(out.numpy(), -hx.T)

    z = rng.standard_normal((24, 40, 56)).astype(np.float32)
    dz = thc.Tensor.from_numpy(z)
    out = thc.Tensor("float").unary("neg", dz.t(0, 2))
    assert_bit_equal(out.numpy(), -z.transpose(2, 1, 0))
    zbase = thc.Tensor.from_numpy(np.zeros((56, 40, 24), np.float32))
    zbase.t(0, 2).unary("neg", dz)
    assert_bit_equal(zbase.numpy(), -z.transpose(2, 1, 0))


@pytest.mark.gpu
def test_gpu_error_paths_of_the_wider_types(thc):
    a = thc.Tensor.from_numpy(np.arange(6, dtype=np.int32).reshape(2, 3))
    b = thc.Tensor.from_numpy(np.arange(8, dtype=np.int32).reshape(2, 4))
    with pytest.raises(thc.THCError, match="sizes do not match"):
        thc.Tensor("int").cadd(a, 1, b)
    with pytest.raises(thc.THCError, match="sizes do not match"):
        thc.Tensor("int").binary("cmax", a, b)
    with pytest.raises(thc.THCError, match="sizes do not match"):
        thc.Tensor("int").addcmul(a, 1, a, b)
    with pytest.raises(thc.THCError, match="divide by zero"):
        thc.Tensor("int").div(a, 0)
    with pytest.raises(thc.THCError, match="dimension out of range"):
        thc.Tensor("int").sum(a, 2)
    with pytest.raises(thc.THCError, match="out of range"):
        thc.Tensor("int").cumsum(a, -1)
    with pytest.raises(thc.THCError, match="sizes do not match"):
        thc.Tensor("long").resize((5,)).copy_from(a)
    with pytest.raises(thc.THCError, match="empty Tensor"):
        thc.Tensor("double").meanall()
    e = thc.Tensor("short")
    assert e.sumall() == 0 and e.prodall() == 1 and e.maxall() == -32768 and e.minall() == 32767
    assert thc.Tensor("byte").logicalall() == 1 and thc.Tensor("byte").logicalany() == 0
    out = thc.Tensor("int").cadd(thc.Tensor("int"), 1, thc.Tensor("int"))       # empty operands: no-op
    assert out.shape == ()
    # in place on a view with holes: untouched storage stays untouched
    st = np.arange(40, dtype=np.int16)
    t = thc.Tensor.from_storage(st, 2, (3, 4), (12, 2), kind="short")
    t.mul(t, 3)
    want = st.copy()
    v = np.lib.stride_tricks.as_strided(want[2:], (3, 4), (24, 4))
    v *= 3
    assert_bit_equal(t.storage_numpy(), want)
