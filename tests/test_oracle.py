"""Pins the CPU oracle (oracle/th_oracle.c) without the reference at hand.

cutorch's own tests hold no golden vectors for this path: every check is a live
comparison with torch7's TH (test/test.lua:247-323), which is not in the tree.
So each oracle function is pinned against something the mathematics fixes:
numpy's IEEE binary32 arithmetic on views that numpy builds with its own
stride machinery, math.fsum (exactly rounded sums), numpy.argmax/argmin
(first occurrence), exhaustive float16 conversion, and integer known answers.
A dropped term, a swapped operand, a wrong stride or an off-by-one index
fails at least one of them.
"""
import json
import math
import os

import numpy as np
import pytest

from tests.util import assert_bit_equal, fill_storage, random_geometry

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def np_view(storage, offset, size, stride):
    item = storage.itemsize
    return np.lib.stride_tricks.as_strided(storage[offset:], shape=size,
                                           strides=tuple(s * item for s in stride))


F32 = np.float32
NP_POINT = {
    "add": lambda a, b, c, v: a + b,
    "sub": lambda a, b, c, v: a - b,
    "mul": lambda a, b, c, v: a * b,
    "div": lambda a, b, c, v: a / b,
    "cadd": lambda a, b, c, v: a + (F32(v) * b).astype(F32),
    "addcmul": lambda a, b, c, v: a + (F32(v) * (b * c).astype(F32)).astype(F32),
    "addcdiv": lambda a, b, c, v: a + (F32(v) * (b / c).astype(F32)).astype(F32),
    "addc": lambda a, b, c, v: a + F32(v),
    "subc": lambda a, b, c, v: a - F32(v),
    "mulc": lambda a, b, c, v: a * F32(v),
    "divc": lambda a, b, c, v: a / F32(v),
    "copy": lambda a, b, c, v: a,
}
NIN = {"add": 2, "sub": 2, "mul": 2, "div": 2, "cadd": 2, "addcmul": 3, "addcdiv": 3,
       "addc": 1, "subc": 1, "mulc": 1, "divc": 1, "copy": 1}


@pytest.mark.parametrize("op", sorted(NP_POINT))
@pytest.mark.parametrize("seed", range(6))
def test_pointwise_matches_numpy_ieee_on_strided_views(oracle, op, seed):
    rng = np.random.default_rng(1000 * seed + len(op))
    nd = int(rng.integers(1, 5))
    shape = tuple(int(x) for x in rng.integers(1, 7, nd))
    v = float(F32(rng.uniform(-3, 3)))
    views, npviews, npstores = [], [], []
    for k in range(NIN[op] + 1):
        n, off, size, stride = random_geometry(rng, shape)
        st = fill_storage(rng, n)
        if k == 0:
            st[:] = np.nan  # holes of the output must stay NaN
        views.append(oracle.View(st, off, size, stride))
        npstores.append(st.copy())
        npviews.append(np_view(npstores[-1], off, size, stride))
    ins = views[1:] + [None] * (3 - NIN[op])
    oracle.pointwise(op, views[0], *ins, value=v)
    a, b, c = (npviews[1:] + [None, None])[:3]
    with np.errstate(all="ignore"):
        want_vals = NP_POINT[op](a, b, c, v).astype(F32)
    npviews[0][...] = want_vals
    assert_bit_equal(views[0].storage, npstores[0], op)


def test_pointwise_pairs_by_linear_index_when_shapes_differ(oracle):
    rng = np.random.default_rng(7)
    a = fill_storage(rng, 24)
    b = fill_storage(rng, 24)
    out = oracle.View.empty((4, 6))
    va = oracle.View(a, 0, (2, 12))
    vb = oracle.View(b, 0, (6, 4), (1, 6))           # transposed, other shape
    oracle.pointwise("add", out, va, vb)
    want = a.reshape(-1) + np_view(b, 0, (6, 4), (1, 6)).reshape(-1)
    assert_bit_equal(out.storage, want)


def test_pointwise_special_values_are_ieee(oracle):
    a = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, 3e38, 1.0, -1e-40], dtype=F32)
    b = np.array([-0.0, 0.0, -np.inf, 2.0, 1.0, 1e-45, 3e38, 3.0, 1e-40], dtype=F32)
    for op in ("add", "mul", "div", "sub"):
        out = oracle.View.empty(a.shape)
        oracle.pointwise(op, out, oracle.View.of(a), oracle.View.of(b))
        with np.errstate(all="ignore"):
            assert_bit_equal(out.storage, NP_POINT[op](a, b, None, 0), op)


def test_addcmul_is_two_roundings_not_fma(oracle):
    # (1+2^-12)^2 = 1 + 2^-11 + 2^-24: the product rounds to 1 + 2^-11 (tie to
    # even), so unfused a + b*c with a = -(1+2^-11) is exactly 0, fused is 2^-24.
    b = np.array([1 + 2.0 ** -12], dtype=F32)
    a = np.array([-(1 + 2.0 ** -11)], dtype=F32)
    out = oracle.View.empty((1,))
    oracle.pointwise("addcmul", out, oracle.View.of(a), oracle.View.of(b), oracle.View.of(b), value=1.0)
    assert out.storage[0] == 0.0
    out2 = oracle.View.empty((1,))
    oracle.pointwise("cadd", out2, oracle.View.of(a), oracle.View.of(b * b), value=1.0)
    assert out2.storage[0] == 0.0


def test_sum_and_norm_against_fsum(oracle):
    rng = np.random.default_rng(3)
    for shape, dim in (((5, 7, 3), 1), ((4, 9), 1), ((6, 5), 0), ((11,), 0), ((3, 1, 4), 1)):
        n, off, size, stride = random_geometry(rng, shape)
        st = fill_storage(rng, n, dist="uniform")
        src = oracle.View(st, off, size, stride)
        x = np_view(st, off, size, stride).astype(np.float64)
        moved = np.moveaxis(x, dim, -1)
        flat = moved.reshape(-1, shape[dim])
        for kind, p, f in (("sum", 0, lambda r: math.fsum(r)),
                           ("norm", 2, lambda r: math.sqrt(math.fsum(v * v for v in r))),
                           ("norm", 1, lambda r: math.fsum(abs(v) for v in r)),
                           ("norm", 0, lambda r: float(sum(v != 0 for v in r))),
                           ("norm", 3, lambda r: math.fsum(abs(v) ** 3 for v in r) ** (1 / 3.0)),
                           ("mean", 0, lambda r: float(F32(F32(math.fsum(r)) / F32(len(r))))),
                           ("prod", 0, lambda r: float(np.prod(np.array(r))))):
            got = oracle.reduce_dim(kind, src, dim, p=p).numpy()
            want = np.array([f(list(r)) for r in flat]).reshape(moved.shape[:-1])
            want = np.expand_dims(want, dim)
            assert got.shape == want.shape
            # double accumulation vs exactly rounded: at most 1 fp32 ulp apart
            np.testing.assert_allclose(got, want.astype(F32), rtol=2.0 ** -23, atol=1e-45)


def test_sum_exact_on_integer_valued_input(oracle):
    rng = np.random.default_rng(5)
    x = rng.integers(-100, 100, (37, 513)).astype(F32)
    got = oracle.reduce_dim("sum", oracle.View.of(x), 1).numpy()
    assert_bit_equal(got, x.astype(np.int64).sum(1, keepdims=True).astype(F32))
    got0 = oracle.reduce_dim("sum", oracle.View.of(x), 0).numpy()
    assert_bit_equal(got0, x.astype(np.int64).sum(0, keepdims=True).astype(F32))
    assert oracle.reduce_all("sum", oracle.View.of(x)) == float(x.astype(np.int64).sum())
    # 3-4-5 rows: exact L2 norms
    t = np.array([[3, 4, 0], [5, 12, 0], [8, 15, 0]], dtype=F32)
    assert_bit_equal(oracle.reduce_dim("norm", oracle.View.of(t), 1, p=2).numpy(),
                     np.array([[5], [13], [17]], dtype=F32))
    assert oracle.reduce_all("norm", oracle.View.of(np.array([3, 4], dtype=F32)), p=2) == 5.0


@pytest.mark.parametrize("seed", range(8))
def test_minmax_first_occurrence_matches_numpy(oracle, seed):
    rng = np.random.default_rng(seed)
    nd = int(rng.integers(1, 4))
    shape = tuple(int(x) for x in rng.integers(1, 9, nd))
    dim = int(rng.integers(0, nd))
    n, off, size, stride = random_geometry(rng, shape)
    st = rng.integers(-3, 4, n).astype(F32)       # few distinct values: many ties
    src = oracle.View(st, off, size, stride)
    x = np_view(st, off, size, stride)
    for which, arg, red in (("max", np.argmax, np.max), ("min", np.argmin, np.min)):
        v, i = oracle.minmax_dim(which, src, dim)
        assert_bit_equal(v.numpy(), red(x, axis=dim, keepdims=True))
        assert np.array_equal(i.numpy(), np.expand_dims(arg(x, axis=dim), dim) + 1)


def test_minmax_nan_and_inf_rows(oracle):
    x = np.array([[1, np.nan, 5, np.nan], [-np.inf, -np.inf, -np.inf, -np.inf],
                  [2, 7, 7, 1], [np.inf, 1, np.inf, 0]], dtype=F32)
    v, i = oracle.minmax_dim("max", oracle.View.of(x), 1)
    assert np.array_equal(i.numpy().ravel(), [2, 1, 2, 1])
    assert np.isnan(v.numpy()[0, 0]) and v.numpy()[1, 0] == -np.inf and v.numpy()[2, 0] == 7
    v, i = oracle.minmax_dim("min", oracle.View.of(x), 1)
    assert np.array_equal(i.numpy().ravel(), [2, 1, 4, 4])
    # numpy agrees on the NaN row (argmax returns the first NaN)
    assert int(np.argmax(x[0])) + 1 == 2


def test_reduce_all_matches_fsum_and_numpy(oracle):
    rng = np.random.default_rng(11)
    n, off, size, stride = random_geometry(rng, (7, 5, 3))
    st = fill_storage(rng, n)
    src = oracle.View(st, off, size, stride)
    x = np_view(st, off, size, stride).astype(np.float64).ravel()
    assert abs(oracle.reduce_all("sum", src) - math.fsum(x)) <= 1e-12 * math.fsum(abs(x))
    assert oracle.reduce_all("max", src) == x.max() and oracle.reduce_all("min", src) == x.min()
    assert abs(oracle.reduce_all("norm", src, p=2) - math.sqrt(math.fsum(x * x))) < 1e-12
    assert abs(oracle.reduce_all("mean", src) - math.fsum(x) / x.size) < 1e-13
    assert oracle.reduce_all("sum", oracle.View.empty(())) == 0.0


def test_half_conversion_exhaustive_against_numpy(oracle):
    allbits = np.arange(65536, dtype=np.uint16)
    want = allbits.view(np.float16).astype(F32)
    got = np.empty(65536, dtype=F32)
    oracle.lib().th_half2float_array(got.ctypes.data, allbits.ctypes.data, 65536)
    assert_bit_equal(got, want, "half->float")
    back = np.empty(65536, dtype=np.uint16)
    oracle.lib().th_float2half_array(back.ctypes.data, got.ctypes.data, 65536)
    nan = np.isnan(want)
    assert np.array_equal(back[~nan], allbits[~nan])
    assert np.all((back[nan] & 0x7c00) == 0x7c00) and np.all((back[nan] & 0x3ff) != 0)
    # rounding: midpoints and neighbours of every adjacent half pair, plus random floats
    rng = np.random.default_rng(0)
    fin = want[np.isfinite(want)].astype(np.float64)
    fin.sort()
    mids = ((fin[:-1] + fin[1:]) / 2).astype(F32)
    probes = np.concatenate([mids, np.nextafter(mids, F32(np.inf)), np.nextafter(mids, F32(-np.inf)),
                             rng.standard_normal(200000).astype(F32) * F32(100),
                             (rng.standard_normal(50000) * 1e-6).astype(F32),
                             np.array([65504, 65519.99, 65520, 65536, 1e10, 5.96e-8, 2.98e-8,
                                       2.9802322e-8, 2.9802326e-8, 0, -0.0], dtype=F32)])
    got16 = np.empty(probes.size, dtype=np.uint16)
    oracle.lib().th_float2half_array(got16.ctypes.data, np.ascontiguousarray(probes).ctypes.data,
                                     probes.size)
    with np.errstate(over="ignore"):
        assert np.array_equal(got16, probes.astype(np.float16).view(np.uint16))


def test_half_ops_round_once_from_fp32(oracle):
    rng = np.random.default_rng(2)
    a = rng.uniform(-2, 2, (6, 10)).astype(np.float16)
    b = rng.uniform(-2, 2, (6, 10)).astype(np.float16)
    out = oracle.View.empty(a.shape, np.float16)
    oracle.pointwise("mul", out, oracle.View.of(a), oracle.View.of(b))
    assert_bit_equal(out.numpy(), (a.astype(F32) * b.astype(F32)).astype(np.float16))
    s = oracle.reduce_dim("sum", oracle.View.of(a), 1).numpy()
    want = np.array([math.fsum(r) for r in a.astype(np.float64)]).astype(F32).astype(np.float16)
    assert_bit_equal(s.ravel(), want)


def test_golden_fixtures(oracle):
    """Small committed vectors (tests/golden/make_fixtures.py wrote them from
    numpy/closed forms); the oracle must reproduce them bit for bit."""
    with open(os.path.join(GOLDEN, "fixtures.json")) as f:
        fx = json.load(f)
    for case in fx["pointwise"]:
        views = []
        for t in case["operands"]:
            st = np.array(t["storage_bits"], dtype=np.uint32).view(F32)
            views.append(oracle.View(st.copy(), t["offset"], t["size"], t["stride"]))
        ins = views[1:] + [None] * (4 - len(views))
        oracle.pointwise(case["op"], views[0], *ins, value=case["value"])
        want = np.array(case["expect_storage_bits"], dtype=np.uint32).view(F32)
        assert_bit_equal(views[0].storage, want, case["name"])
    for case in fx["argmax"]:
        x = np.array(case["x_bits"], dtype=np.uint32).view(F32).reshape(case["shape"])
        v, i = oracle.minmax_dim(case["which"], oracle.View.of(x), case["dim"])
        assert i.numpy().ravel().tolist() == case["indices"], case["name"]
        assert_bit_equal(v.numpy().ravel(), np.array(case["values_bits"], dtype=np.uint32).view(F32))
    for case in fx["sum"]:
        x = np.array(case["x"], dtype=F32).reshape(case["shape"])
        got = oracle.reduce_dim(case["kind"], oracle.View.of(x), case["dim"], p=case.get("p", 0)).numpy()
        assert got.ravel().tolist() == case["expect"], case["name"]
    for case in fx["half"]:
        assert oracle.lib().th_float2half(np.uint32(case["f32_bits"]).view(F32)) == case["f16_bits"]
