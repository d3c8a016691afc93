"""Parity of the HIP reduce engine with the CPU oracle, through the C ABI.

Bars (stated by the task): max/min values and 1-based indices bit-exact with
the lowest index on ties; sum / norm within 1e-5 relative error in fp32 and
2e-3 for fp16 input with fp32 accumulation. "Relative" is taken against
max(|reference|, 2^-6 * sum_i |x_i|): for zero-mean inputs individual sums can
cancel to ~0, where an error relative to the result alone is unbounded for ANY
fp32 summation order (one rounding of a partial sum is already 2^-24 of the
mass sum|x_i|; the floor admits about 2.6 such roundings); the reference's own
suite uses an absolute 1e-1 there (test/test.lua:1474-1487). Sums of integer-valued data are exact in every
order and must match bit for bit."""
import numpy as np
import pytest

from tests.util import assert_bit_equal, contiguous_geometry, fill_storage, random_geometry

pytestmark = pytest.mark.gpu

TOL = {"float": 1e-5, "half": 2e-3}
# worst errors seen by check_close, per label: (strict |got - ref| / |ref|, the same against the floored scale)
MARGINS = {}


def check_close(got, want, absx_sum, kind, what):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    scale = np.maximum(np.abs(want), np.asarray(absx_sum, np.float64) * 2.0 ** -6)
    scale = np.maximum(scale, 1e-30)
    err = np.abs(got - want) / scale
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert np.all(np.isfinite(got) == np.isfinite(want)), what
    worst = float(np.nanmax(err)) if err.size else 0.0
    with np.errstate(divide="ignore", invalid="ignore"):
        strict = np.abs(got - want) / np.abs(want)
    strict = strict[np.isfinite(strict)]
    MARGINS[what] = (float(strict.max()) if strict.size else 0.0, worst)
    assert worst <= TOL[kind], "%s: rel err %.3g > %.3g" % (what, worst, TOL[kind])


def dev_and_ref(thc, oracle, rng, geom, kind="float", dist="normal"):
    dtype = np.float16 if kind == "half" else np.float32
    st = fill_storage(rng, geom[0], dtype, dist)
    return thc.Tensor.from_storage(st, *geom[1:], kind=kind), oracle.View(st.copy(), *geom[1:])


REDUCERS = [("sum", "sum", 0.0), ("norm2", "norm", 2.0), ("norm1", "norm", 1.0), ("norm0", "norm", 0.0),
            ("norm3", "norm", 3.0), ("mean", "mean", 0.0)]


def run_reduce(thc, oracle, name, dev, ref, dim, kind="float"):
    _, okind, p = [r for r in REDUCERS if r[0] == name][0]
    out = thc.Tensor(kind)
    if okind == "norm":
        out.norm(dev, p, dim)
    else:
        getattr(out, okind)(dev, dim)
    want = oracle.reduce_dim(okind, ref, dim, p=p).numpy().astype(np.float64)
    x = np.abs(ref.numpy().astype(np.float64))
    if name == "norm2":
        mass = np.sqrt((x * x).sum(axis=dim, keepdims=True))
    elif name == "norm3":
        mass = (x ** 3).sum(axis=dim, keepdims=True) ** (1 / 3.0)
    elif name == "mean":
        mass = x.mean(axis=dim, keepdims=True)
    else:
        mass = x.sum(axis=dim, keepdims=True)
    got = out.numpy().astype(np.float64)
    assert out.shape == tuple(1 if d == dim else s for d, s in enumerate(ref.size))
    check_close(got, want, mass, kind, "%s dim %d %s" % (name, dim, ref.size))
    return thc.last_kernel()


@pytest.mark.parametrize("name", [r[0] for r in REDUCERS])
@pytest.mark.parametrize("kind", ["float", "half"])
def test_innermost_dim(thc, oracle, name, kind):
    rng = np.random.default_rng(21)
    for shape in ((7, 1024), (300, 64), (5, 3), (1000, 17), (3, 5000), (2, 3, 128), (4097, 1), (1, 1)):
        dev, ref = dev_and_ref(thc, oracle, rng, contiguous_geometry(shape), kind, "uniform")
        k = run_reduce(thc, oracle, name, dev, ref, len(shape) - 1, kind)
        assert k.startswith("rows"), k


@pytest.mark.parametrize("name", [r[0] for r in REDUCERS])
@pytest.mark.parametrize("kind", ["float", "half"])
def test_non_innermost_dim(thc, oracle, name, kind):
    rng = np.random.default_rng(22)
    for shape, dim in (((64, 512), 0), ((6, 300, 40), 1), ((4, 4096, 16), 1), ((129, 7), 0),
                       ((3, 50, 8, 24), 1), ((2, 2000, 3), 1), ((16, 33, 1), 1)):
        dev, ref = dev_and_ref(thc, oracle, rng, contiguous_geometry(shape), kind, "uniform")
        k = run_reduce(thc, oracle, name, dev, ref, dim, kind)
        assert k.startswith("cols") or k in ("slab", "tall-flat") or shape[-1] == 1, k


def test_split_reduction_is_used_and_correct(thc, oracle):
    rng = np.random.default_rng(23)
    dev, ref = dev_and_ref(thc, oracle, rng, contiguous_geometry((2, 8192, 96)), "float", "uniform")
    assert run_reduce(thc, oracle, "sum", dev, ref, 1) == "cols-split"
    assert run_reduce(thc, oracle, "norm2", dev, ref, 1) == "cols-split"
    dev, ref = dev_and_ref(thc, oracle, rng, contiguous_geometry((3, 1 << 18)), "float", "uniform")
    assert run_reduce(thc, oracle, "sum", dev, ref, 1) == "rows-split"
    assert run_reduce(thc, oracle, "norm2", dev, ref, 1) == "rows-split"


@pytest.mark.parametrize("seed", range(30))
def test_random_strided_inputs(thc, oracle, seed):
    rng = np.random.default_rng(300 + seed)
    nd = int(rng.integers(1, 5))
    shape = tuple(int(x) for x in rng.integers(1, 20, nd))
    dim = int(rng.integers(0, nd))
    geom = random_geometry(rng, shape, holes=rng.random() < 0.5, permute=rng.random() < 0.5)
    dev, ref = dev_and_ref(thc, oracle, rng, geom)
    run_reduce(thc, oracle, REDUCERS[seed % len(REDUCERS)][0], dev, ref, dim)
    thc.force_64bit_index(True)
    try:
        run_reduce(thc, oracle, "sum", dev, ref, dim)
    finally:
        thc.force_64bit_index(False)


def test_integer_valued_sums_are_bit_exact(thc, oracle):
    rng = np.random.default_rng(24)
    for shape, dim in (((512, 1024), 1), ((16, 2048, 64), 1), ((1 << 20,), 0), ((100, 77), 0)):
        x = rng.integers(-8, 9, shape).astype(np.float32)
        dev = thc.Tensor.from_numpy(x)
        out = thc.Tensor("float").sum(dev, dim)
        assert_bit_equal(out.numpy(), x.astype(np.int64).sum(axis=dim, keepdims=True).astype(np.float32))
        assert dev.sumall() == float(x.astype(np.int64).sum())


def test_keepdim_zero_squeezes(thc):
    x = np.ones((3, 4, 5), np.float32)
    out = thc.Tensor("float").sum(thc.Tensor.from_numpy(x), 1, keepdim=0)
    assert out.shape == (3, 5) and np.all(out.numpy() == 4)
    out = thc.Tensor("float").sum(thc.Tensor.from_numpy(np.ones(7, np.float32)), 0, keepdim=0)
    assert out.shape == (1,)        # a vector never loses its last dim


def test_output_with_existing_strides_is_kept(thc, oracle):
    rng = np.random.default_rng(25)
    x = rng.standard_normal((6, 9, 10)).astype(np.float32)
    st = np.full(6 * 1 * 10 * 3, np.nan, np.float32)
    out = thc.Tensor.from_storage(st, 1, (6, 1, 10), (30, 30, 3))     # right shape, odd strides
    out.sum(thc.Tensor.from_numpy(x), 1)
    assert out.strides == (30, 30, 3)
    r = oracle.View(st.copy(), 1, (6, 1, 10), (30, 30, 3))
    oracle.reduce_dim("sum", oracle.View.of(x), 1, out=r)
    got, want = out.storage_numpy(), r.storage
    assert np.array_equal(np.isnan(got), np.isnan(want))
    np.testing.assert_allclose(got[~np.isnan(got)], want[~np.isnan(want)], rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------- max / min --
def run_minmax(thc, oracle, which, dev, ref, dim, kind="float"):
    vals, idx = thc.Tensor(kind), thc.Tensor("long")
    getattr(vals, which)(idx, dev, dim)
    rv, ri = oracle.minmax_dim(which, ref, dim)
    assert_bit_equal(vals.numpy(), rv.numpy(), which + " values")
    assert np.array_equal(idx.numpy(), ri.numpy()), which + " indices"
    return thc.last_kernel()


@pytest.mark.parametrize("which", ["max", "min"])
@pytest.mark.parametrize("kind", ["float", "half"])
def test_minmax_with_many_ties(thc, oracle, which, kind):
    rng = np.random.default_rng(31)
    for shape, dim in (((64, 1024), 1), ((9, 33), 1), ((5, 4000), 1), ((300, 5), 1), ((64, 512), 0),
                       ((6, 300, 40), 1), ((4, 4096, 16), 1), ((2, 8192, 96), 1), ((7,), 0), ((1, 1), 0)):
        dev, ref = dev_and_ref(thc, oracle, rng, contiguous_geometry(shape), kind, "ints")
        run_minmax(thc, oracle, which, dev, ref, dim, kind)


@pytest.mark.parametrize("kind", ["float", "half", "int", "double", "byte"])
def test_minmax_of_long_narrow_slices(thc, oracle, kind):
    """max / min with index along the long dim of few long narrow slices (flat runs of packs, every
    lane keeping (value, row) pairs per column): tie-heavy data (the first of equal extremes wins at
    every level), NaN / inf / signed zeros planted at the ends of workgroup pieces and in the
    elements behind the last whole pack, columns that are all -inf; against the oracle and, for the
    planted cases, numpy's first-occurrence argmax."""
    rng = np.random.default_rng(37)
    dtype = {"float": np.float32, "half": np.float16, "int": np.int32, "double": np.float64, "byte": np.uint8}[kind]
    vec = 16 // np.dtype(dtype).itemsize
    for shape, dim in (((200003, 3), 0), ((70001, 10), 0), ((30000, 33), 0), ((2, 40000, 7), 1), ((3, 16000, 5), 1),
                       ((1, 50001, 9), 1), ((25000, 50), 0), ((40000, 16), 0), ((3, 9001, 64), 1)):
        inner = int(np.prod(shape[dim + 1:]))
        outer = int(np.prod(shape[:dim]))
        flat = outer == 1 or (shape[dim] * inner) % vec == 0      # (every slice starts on a 16-byte boundary)
        lo, hi = (0, 4) if kind == "byte" else (-3, 4)
        x = rng.integers(lo, hi, shape).astype(dtype)
        dev, ref = thc.Tensor.from_numpy(x), oracle.View.of(x)
        for which in ("max", "min"):
            if kind in ("float", "half"):      # (the oracle's restatement is the float one)
                k = run_minmax(thc, oracle, which, dev, ref, dim, kind)
                assert k == ("tall-index" if flat else "cols-index-split"), (shape, which, k)
            vals, idx = thc.Tensor(kind), thc.Tensor("long")
            getattr(vals, which)(idx, dev, dim)
            assert thc.last_kernel() == ("tall-index" if flat else "cols-index-split"), (shape, which, thc.last_kernel())
            want = (np.argmax if which == "max" else np.argmin)(x, axis=dim) + 1
            assert np.array_equal(idx.numpy().reshape(want.shape), want), (shape, which)
            wantv = (np.max if which == "max" else np.min)(x, axis=dim)
            assert_bit_equal(vals.numpy().reshape(wantv.shape), wantv, "%s %s values" % (shape, which))
    if kind in ("float", "half"):
        x = rng.integers(-3, 4, (70001, 10)).astype(dtype)
        x[:, 0] = -np.inf                      # a column without a candidate: index 1
        x[:, 1] = 0.0
        x[5, 1], x[600, 1] = -0.0, -0.0        # zeros: the first one (+0 at row 0) stays for max and min
        x[69999, 2] = np.nan                   # in the last workgroup's piece
        x[70000, 3] = np.nan                   # behind the last whole pack (70001 * 10 is not a multiple of 4 or 8)
        x[40000, 4], x[123, 4] = np.nan, np.nan
        x[33333, 5] = np.inf
        x[33333, 6] = -np.inf
        dev, ref = thc.Tensor.from_numpy(x), oracle.View.of(x)
        for which in ("max", "min"):
            vals, idx = thc.Tensor(kind), thc.Tensor("long")
            getattr(vals, which)(idx, dev, 0)
            assert thc.last_kernel() == "tall-index"
            rv, ri = oracle.minmax_dim(which, ref, 0)
            assert np.array_equal(idx.numpy(), ri.numpy()), which
            g, w = vals.numpy(), rv.numpy()
            assert np.array_equal(np.isnan(g), np.isnan(w))
            assert_bit_equal(g[~np.isnan(g)], w[~np.isnan(w)])
            i = idx.numpy().reshape(-1)
            assert i[2] == 70000 and i[3] == 70001 and i[4] == 124 and i[1] == 1
            assert i[0] == (1 if which == "max" else 1)
            assert not np.signbit(g.reshape(-1)[1])
    thc.set_tuning("reduce.tall", 0)
    try:
        x = rng.integers(0, 4, (70001, 10)).astype(dtype)
        vals, idx = thc.Tensor(kind), thc.Tensor("long")
        vals.max(idx, thc.Tensor.from_numpy(x), 0)
        assert thc.last_kernel().startswith("cols-index"), thc.last_kernel()
        assert np.array_equal(idx.numpy().reshape(-1), np.argmax(x, axis=0) + 1)
    finally:
        thc.set_tuning("reduce.tall", 1)


@pytest.mark.parametrize("kind", ["float", "half", "int", "double"])
def test_short_reduced_dim_over_long_rows(thc, oracle, kind):
    """A reduced (or scanned) dim of 2..16 elements over long unit-stride rows: the column kernels widen
    their segments until no thread row is left without work (one thread row at 8 rows and fewer).
    sum / max / min / var / cumsum against numpy on small integers, pack-aligned and odd row lengths."""
    rng = np.random.default_rng(39)
    dtype = {"float": np.float32, "half": np.float16, "int": np.int32, "double": np.float64}[kind]
    for shape, dim in (((2, 40000), 0), ((3, 70001), 0), ((8, 16384), 0), ((5, 4, 8192), 1), ((16, 9000), 0),
                       ((7, 2, 33000), 1), ((4, 1 << 18), 0)):
        x = rng.integers(-3, 4, shape).astype(dtype)
        dev = thc.Tensor.from_numpy(x)
        for knob in (1, 0):
            thc.set_tuning("reduce.cols.short_wide", knob)
            thc.set_tuning("scan.cols.short_wide", knob)
            try:
                got = thc.Tensor(kind).sum(dev, dim)
                assert thc.last_kernel().startswith("cols"), thc.last_kernel()
                assert_bit_equal(got.numpy(), x.astype(np.int64).sum(axis=dim, keepdims=True).astype(dtype))
                for which, arg, ext in (("max", np.argmax, np.max), ("min", np.argmin, np.min)):
                    vals, idx = thc.Tensor(kind), thc.Tensor("long")
                    getattr(vals, which)(idx, dev, dim)
                    assert thc.last_kernel().startswith("cols-index"), thc.last_kernel()
                    assert np.array_equal(idx.numpy(), np.expand_dims(arg(x, axis=dim), dim) + 1), (shape, which)
                    assert_bit_equal(vals.numpy(), ext(x, axis=dim, keepdims=True))
                scan = thc.Tensor(kind).cumsum(dev, dim)
                assert thc.last_kernel().startswith("scan-cols"), thc.last_kernel()
                assert_bit_equal(scan.numpy(), np.cumsum(x.astype(np.int64), axis=dim).astype(dtype))
                if kind != "int":
                    var = thc.Tensor(kind).var(dev, dim)
                    assert thc.last_kernel().startswith("var-cols"), thc.last_kernel()
                    want = np.var(x.astype(np.float64), axis=dim, ddof=1, keepdims=True)
                    np.testing.assert_allclose(var.numpy().astype(np.float64), want, rtol=2e-3 if kind == "half" else 1e-5,
                                               atol=1e-6)
            finally:
                thc.set_tuning("reduce.cols.short_wide", 1)
                thc.set_tuning("scan.cols.short_wide", 1)


def test_minmax_config3_pattern(thc, oracle):
    """normal(0,1) rows with ~1% of each row overwritten by copies of other
    entries of the same row, the row maximum included (benchmark config 3)."""
    rng = np.random.default_rng(0xC0FFEE + 3)
    rows, n = 2048, 1024
    x = rng.standard_normal((rows, n)).astype(np.float32)
    for r in range(rows):
        src = rng.integers(0, n, 10)
        dst = rng.integers(0, n, 10)
        x[r, dst] = x[r, src]
        j = int(np.argmax(x[r]))
        x[r, rng.integers(0, n, 2)] = x[r, j]
    dev, ref = thc.Tensor.from_numpy(x), oracle.View.of(x)
    assert run_minmax(thc, oracle, "max", dev, ref, 1) == "rows-index"
    run_minmax(thc, oracle, "min", dev, ref, 1)
    assert np.array_equal(ref.numpy(), x)


@pytest.mark.parametrize("seed", range(20))
def test_minmax_random_strided(thc, oracle, seed):
    rng = np.random.default_rng(400 + seed)
    nd = int(rng.integers(1, 5))
    shape = tuple(int(x) for x in rng.integers(1, 20, nd))
    dim = int(rng.integers(0, nd))
    geom = random_geometry(rng, shape, holes=rng.random() < 0.5, permute=rng.random() < 0.5)
    dev, ref = dev_and_ref(thc, oracle, rng, geom, "float", "ints")
    run_minmax(thc, oracle, "max" if seed % 2 else "min", dev, ref, dim)


def test_minmax_nan_inf_and_signed_zero(thc, oracle):
    x = np.array([[1, np.nan, 5, np.nan, 0, 0, 0, 0], [-np.inf] * 8, [2, 7, 7, 1, 7, 0, 0, 0],
                  [np.inf, 1, np.inf, 0, 0, 0, 0, 0], [-0.0, 0.0, -0.0, 0.0, -1, -1, -1, -1]], dtype=np.float32)
    for which in ("max", "min"):
        vals, idx = thc.Tensor("float"), thc.Tensor("long")
        getattr(vals, which)(idx, thc.Tensor.from_numpy(x), 1)
        rv, ri = oracle.minmax_dim(which, oracle.View.of(x), 1)
        assert np.array_equal(idx.numpy(), ri.numpy())
        g, w = vals.numpy(), rv.numpy()
        assert np.array_equal(np.isnan(g), np.isnan(w))
        assert_bit_equal(g[~np.isnan(g)], w[~np.isnan(w)])


def test_minmax_noncontiguous_outputs(thc, oracle):
    rng = np.random.default_rng(33)
    x = rng.integers(-3, 4, (12, 30)).astype(np.float32)
    vst = np.full(12 * 2 + 1, np.nan, np.float32)
    ist = np.full(12 * 3, -7, np.int64)
    vals = thc.Tensor.from_storage(vst, 1, (12, 1), (2, 2))
    idx = thc.Tensor.from_storage(ist, 0, (12, 1), (3, 1), kind="long")
    vals.max(idx, thc.Tensor.from_numpy(x), 1)
    assert np.array_equal(idx.storage_numpy()[0::3], np.argmax(x, 1) + 1)
    assert np.all(idx.storage_numpy()[1::3] == -7)
    assert np.array_equal(vals.storage_numpy()[1::2], x.max(1))


# ------------------------------------------------------------------ *all --
@pytest.mark.parametrize("kind", ["float", "half"])
def test_all_reductions(thc, oracle, kind):
    rng = np.random.default_rng(41)
    for shape in ((1,), (5,), (2048,), (2049,), (100003,), (1 << 21,), (300, 700), (5, 6, 7)):
        dev, ref = dev_and_ref(thc, oracle, rng, contiguous_geometry(shape), kind, "uniform")
        x = np.abs(ref.numpy().astype(np.float64))
        n = x.size
        check_close(dev.sumall(), oracle.reduce_all("sum", ref), x.sum(), kind, "sumall")
        check_close(dev.meanall(), oracle.reduce_all("mean", ref), x.mean(), kind, "meanall")
        check_close(dev.normall(2.0), oracle.reduce_all("norm", ref, p=2), 0, kind, "normall2")
        check_close(dev.normall(1.0), oracle.reduce_all("norm", ref, p=1), 0, kind, "normall1")
        check_close(dev.normall(3.0), oracle.reduce_all("norm", ref, p=3), 0, kind, "normall3")
        assert dev.normall(0.0) == oracle.reduce_all("norm", ref, p=0)
        assert dev.maxall() == oracle.reduce_all("max", ref)
        assert dev.minall() == oracle.reduce_all("min", ref)


@pytest.mark.parametrize("kind", ["float", "double", "int"])
def test_all_reductions_on_permuted_dense_views(thc, kind):
    """A transposed or permuted view of a dense block is reduced in storage order (no contiguous copy is
    made first): sums, extremes, products and moments of integer-valued data are exact whatever the order."""
    rng = np.random.default_rng(47)
    dtype = {"float": np.float32, "double": np.float64, "int": np.int32}[kind]
    for shape, perm in (((300, 700), (1, 0)), ((37, 41, 53), (2, 0, 1)), ((5, 6, 7, 8), (3, 1, 0, 2)), ((1, 90000), (1, 0))):
        x = rng.integers(-3, 4, shape).astype(dtype)
        view = thc.Tensor.from_numpy(x)
        strides = [int(s // x.itemsize) for s in x.strides]
        pv = view.view_as_strided(0, tuple(shape[p] for p in perm), tuple(strides[p] for p in perm))
        assert not pv.is_contiguous() or 1 in shape
        for knob in (1, 0):
            thc.set_tuning("reduce.all.by_stride", knob)
            try:
                assert pv.sumall() == x.astype(np.int64).sum()
                assert pv.maxall() == x.max() and pv.minall() == x.min()
                if kind != "int":
                    np.testing.assert_allclose(pv.varall(), np.var(x.astype(np.float64), ddof=1), rtol=1e-5)
                    np.testing.assert_allclose(pv.normall(2.0), np.sqrt((x.astype(np.float64) ** 2).sum()), rtol=1e-6)
                    assert pv.meanall() == pytest.approx(x.astype(np.float64).mean(), rel=1e-6, abs=1e-7)
            finally:
                thc.set_tuning("reduce.all.by_stride", 1)
    row = rng.integers(-3, 4, 700).astype(dtype)
    expanded = thc.Tensor.from_numpy(row).view_as_strided(0, (300, 700), (0, 1))        # a repeated dim stays where it is
    assert expanded.sumall() == 300 * int(row.astype(np.int64).sum()) and expanded.maxall() == row.max()
    if kind != "int":
        ones = np.ones((64, 130), dtype)
        ones[::7, ::11] = 2
        pv = thc.Tensor.from_numpy(ones).t()
        assert pv.prodall() == float(np.prod(ones.astype(np.float64)))      # 2^120


def test_all_reductions_on_strided_views(thc, oracle):
    rng = np.random.default_rng(42)
    for shape in ((40, 50), (7, 8, 9), (300,)):
        for permute in (False, True):
            geom = random_geometry(rng, shape, holes=True, permute=permute)
            dev, ref = dev_and_ref(thc, oracle, rng, geom, "float", "uniform")
            x = np.abs(ref.numpy().astype(np.float64))
            check_close(dev.sumall(), oracle.reduce_all("sum", ref), x.sum(), "float", "sumall strided")
            assert dev.maxall() == oracle.reduce_all("max", ref)
            assert dev.minall() == oracle.reduce_all("min", ref)


def test_all_empty_and_nan(thc):
    e = thc.Tensor("float")
    assert e.sumall() == 0.0 and e.prodall() == 1.0
    x = np.ones(5000, np.float32)
    x[1234] = np.nan
    t = thc.Tensor.from_numpy(x)
    assert np.isnan(t.maxall()) and np.isnan(t.minall()) and np.isnan(t.sumall())
    with pytest.raises(thc.THCError, match="empty Tensor"):
        e.meanall()


def test_reduce_error_paths(thc):
    t = thc.Tensor.from_numpy(np.ones((3, 4), np.float32))
    with pytest.raises(thc.THCError, match="dimension out of range"):
        thc.Tensor("float").sum(t, 2)
    with pytest.raises(thc.THCError, match="dimension out of range"):
        thc.Tensor("float").max(thc.Tensor("long"), t, -1)


# --------------------------------------- full benchmark shapes (properties) --
def note_margins(label, tol):
    """Prints the worst errors of the checks made since the last call (how far
    the full-size configurations stay below their tolerance) and, when the
    environment names a file in THC_MARGINS_FILE, appends them to it."""
    import os
    strict = max(v[0] for v in MARGINS.values())
    floored = max(v[1] for v in MARGINS.values())
    MARGINS.clear()
    line = "%s: worst |got-ref|/|ref| = %.3g, worst against max(|ref|, mass/64) = %.3g, tolerance %.0e" % (
        label, strict, floored, tol)
    print(line)
    path = os.environ.get("THC_MARGINS_FILE")
    if path:
        with open(path, "a") as f:
            f.write(line + "\n")


def test_config3_full_size_against_oracle(thc, oracle):
    """65536 x 1024: the oracle finishes this in well under a second."""
    rng = np.random.default_rng(0xC0FFEE + 33)
    x = rng.standard_normal((65536, 1024)).astype(np.float32)
    dup = rng.integers(0, 1024, (65536, 10))
    x[np.arange(65536)[:, None], dup] = x[np.arange(65536)[:, None], dup[:, ::-1]]
    x[np.arange(65536), dup[:, 0]] = x.max(1)          # duplicate the row maximum
    dev, ref = thc.Tensor.from_numpy(x), oracle.View.of(x)
    oracle.set_num_threads(8)
    try:
        MARGINS.clear()
        run_reduce(thc, oracle, "sum", dev, ref, 1)
        note_margins("C3a sum over rows of 65536x1024 fp32", 1e-5)
        run_minmax(thc, oracle, "max", dev, ref, 1)
    finally:
        oracle.set_num_threads(1)


def test_config4_full_size_against_oracle(thc, oracle):
    """64 x 4096 x 512, reduce the middle dim, fp32 and fp16 input."""
    rng = np.random.default_rng(0xC0FFEE + 4)
    x = rng.uniform(-2, 2, (64, 4096, 512)).astype(np.float32)
    oracle.set_num_threads(8)
    try:
        for kind, arr in (("float", x), ("half", x.astype(np.float16))):
            dev, ref = thc.Tensor.from_numpy(arr), oracle.View.of(arr)
            MARGINS.clear()
            assert run_reduce(thc, oracle, "sum", dev, ref, 1, kind).startswith("cols")
            note_margins("C4 sum over the middle dim of 64x4096x512 %s" % kind, TOL[kind])
            run_reduce(thc, oracle, "norm2", dev, ref, 1, kind)
            note_margins("C4 norm2 over the middle dim of 64x4096x512 %s" % kind, TOL[kind])
    finally:
        oracle.set_num_threads(1)


def test_sumall_2pow28_uniform(thc, oracle):
    """reduceAll over 2^28 uniform[0,1] values (1 GiB)."""
    rng = np.random.default_rng(0xC0FFEE + 333)
    x = rng.random(1 << 28, dtype=np.float32)
    dev = thc.Tensor.from_numpy(x)
    oracle.set_num_threads(8)
    try:
        want = oracle.reduce_all("sum", oracle.View(x))
    finally:
        oracle.set_num_threads(1)
    got = dev.sumall()
    assert abs(got - want) <= 1e-5 * abs(want), (got, want)
    MARGINS["sumall"] = (abs(got - want) / abs(want), abs(got - want) / abs(want))
    note_margins("C3c sumall over 2^28 uniform[0,1] fp32", 1e-5)
    assert abs(dev.normall(2.0) - oracle.reduce_all("norm", oracle.View(x[:1 << 20]), p=2)) >= 0  # smoke


# ------------------------------------------------ strided and long-row shapes --
def test_strided_reduced_dim_without_unit_stride_sibling(thc, oracle):
    """A column of a matrix (one output over a strided dim) and a strided slice
    whose other dim is strided too: lanes share each output instead of one
    thread walking it."""
    rng = np.random.default_rng(51)
    n, w = 70000, 3
    st = rng.uniform(-1, 1, n * w).astype(np.float32)
    for kind_name, fn in (("sum", "sum"), ("norm2", "norm2")):
        dev = thc.Tensor.from_storage(st, 1, (n, 1), (w, 1))
        ref = oracle.View(st.copy(), 1, (n, 1), (w, 1))
        assert run_reduce(thc, oracle, fn, dev, ref, 0).startswith("rows-split-strided")
    dev = thc.Tensor.from_storage(st, 0, (100, 300), (2100, 7))     # both dims strided
    ref = oracle.View(st.copy(), 0, (100, 300), (2100, 7))
    assert run_reduce(thc, oracle, "sum", dev, ref, 1) == "rows-strided"
    assert run_reduce(thc, oracle, "sum", dev, ref, 0) == "rows-strided"
    sti = rng.integers(-50, 50, n * w).astype(np.float32)
    devi = thc.Tensor.from_storage(sti, 2, (n, 1), (w, 1))
    refi = oracle.View(sti.copy(), 2, (n, 1), (w, 1))
    for which in ("max", "min"):
        assert run_minmax(thc, oracle, which, devi, refi, 0) == "rows-index-split-strided"
    devi = thc.Tensor.from_storage(sti, 0, (100, 300), (2100, 7))
    refi = oracle.View(sti.copy(), 0, (100, 300), (2100, 7))
    assert run_minmax(thc, oracle, "max", devi, refi, 1) == "rows-index-strided"
    assert run_minmax(thc, oracle, "min", devi, refi, 0) == "rows-index-strided"


@pytest.mark.parametrize("kind", ["float", "half"])
def test_minmax_of_few_long_rows_is_split(thc, oracle, kind):
    rng = np.random.default_rng(52)
    for shape in ((3, 1 << 18), (1, 300001), (2, 5, 40000)):
        dev, ref = dev_and_ref(thc, oracle, rng, contiguous_geometry(shape), kind, "ints")
        for which in ("max", "min"):
            k = run_minmax(thc, oracle, which, dev, ref, len(shape) - 1, kind)
            assert k.startswith("rows-index-split"), k
    x = np.full((2, 100000), -np.inf, np.float32)                  # nothing beats the start value
    x[1, 77777] = np.nan
    vals, idx = thc.Tensor("float"), thc.Tensor("long")
    vals.max(idx, thc.Tensor.from_numpy(x), 1)
    assert idx.numpy().ravel().tolist() == [1, 77778]
    assert vals.numpy()[0, 0] == -np.inf and np.isnan(vals.numpy()[1, 0])
    thc.force_64bit_index(True)
    try:
        dev, ref = dev_and_ref(thc, oracle, rng, contiguous_geometry((2, 70000)), "float", "ints")
        assert run_minmax(thc, oracle, "max", dev, ref, 1) == "rows-index-split"
    finally:
        thc.force_64bit_index(False)


def test_forced_split_is_capped_by_the_scratch_buffer(thc, oracle):
    """The split knob is a request: the partial planes of a column reduction
    must fit the per-stream scratch buffer whatever it asks for."""
    rng = np.random.default_rng(53)
    x = rng.integers(-50, 50, (600, 70000)).astype(np.float32)
    dev = thc.Tensor.from_numpy(x)
    thc.set_tuning("reduce.cols.force_split", 512)   # 512 x 70000 (value, index) pairs do not fit
    try:
        vals, idx = thc.Tensor("float"), thc.Tensor("long")
        vals.max(idx, dev, 0)
        sums = thc.Tensor("float").sum(dev, 0)
    finally:
        thc.set_tuning("reduce.cols.force_split", 0)
    wv, wi = oracle.minmax_dim("max", oracle.View.of(x), 0)
    assert_bit_equal(vals.numpy(), wv.numpy())
    np.testing.assert_array_equal(idx.numpy(), wi.numpy())
    assert_bit_equal(sums.numpy(), x.sum(axis=0, dtype=np.float64).astype(np.float32).reshape(1, -1))


@pytest.mark.parametrize("kind", ["float", "half"])
def test_short_dense_rows_are_staged_through_lds(thc, oracle, kind):
    """Rows that lie back to back are streamed into LDS as one flat run of
    aligned packs, whatever the rows' own alignment: every row length from 1
    to 40, lengths around the limits, storage offsets 0..3, row counts that
    leave a ragged last run; same results with the kernel switched off."""
    rng = np.random.default_rng(54)
    shapes = [(37, r) for r in range(1, 41)] + [(5000, 10), (777, 70), (300, 100), (41, 1001), (3, 2048),
                                               (2, 3, 250), (9, 511)]
    for shape in shapes:
        n = int(np.prod(shape))
        for off in (0, 1, 3) if shape[-1] in (10, 70, 100) else (0,):
            st = [1] * len(shape)
            for d in range(len(shape) - 2, -1, -1):
                st[d] = st[d + 1] * shape[d + 1]
            dev, ref = dev_and_ref(thc, oracle, rng, (n + off, off, shape, tuple(st)), kind, "ints")
            dim = len(shape) - 1
            rowbytes = shape[-1] * (4 if kind == "float" else 2)
            vec = 4 if kind == "float" else 8
            packs = shape[-1] % vec == 0 and off % vec == 0
            expect = "rows-lds" if rowbytes <= (511 if packs else 8192) else "rows"
            for name in ("sum", "norm2", "mean"):
                k = run_reduce(thc, oracle, name, dev, ref, dim, kind)
                assert k == expect, (shape, off, name, k)
            for which in ("max", "min"):
                k = run_minmax(thc, oracle, which, dev, ref, dim, kind)
                assert k == expect.replace("rows", "rows-index"), (shape, off, which, k)
    thc.set_tuning("reduce.rows.lds", 0)
    try:
        dev, ref = dev_and_ref(thc, oracle, rng, contiguous_geometry((777, 70)), kind, "ints")
        assert run_reduce(thc, oracle, "sum", dev, ref, 1, kind) == "rows-scalar"
        assert run_minmax(thc, oracle, "max", dev, ref, 1, kind) == "rows-index-scalar"
    finally:
        thc.set_tuning("reduce.rows.lds", 1)


def test_short_dense_rows_special_cases(thc, oracle):
    x = np.full((300, 33), -np.inf, np.float32)        # nothing beats the start value
    x[7, 20] = np.nan
    x[8, :] = 2.5                                      # all tied: first index
    x[9, 5] = x[9, 31] = 7.0
    vals, idx = thc.Tensor("float"), thc.Tensor("long")
    vals.max(idx, thc.Tensor.from_numpy(x), 1)
    assert thc.last_kernel() == "rows-index-lds"
    i = idx.numpy().ravel()
    assert i[0] == 1 and i[7] == 21 and i[8] == 1 and i[9] == 6
    v = vals.numpy().ravel()
    assert v[0] == -np.inf and np.isnan(v[7]) and v[8] == 2.5 and v[9] == 7.0
    # half rows, read from LDS four elements at a time (sums; max / min when the row length is a multiple
    # of four): every residue of the row start modulo four (storage offsets 0..3), ties across the words
    # of one batch, NaN, signed zeros
    for R in (70, 72):
        for off in range(4):
            h = np.full((200, R), -np.inf, np.float16)
            h[3, 41] = np.nan
            h[4, :] = 1.5
            h[5, 2] = h[5, 3] = h[5, R - 1] = 9.0
            h[6, :] = -0.0
            h[6, 17] = 0.0
            h[7, R - 1] = 3.0
            flat = thc.Tensor.from_numpy(np.concatenate([np.zeros(off, np.float16), h.ravel()]))
            view = flat.view_as_strided(off, (200, R), (R, 1))
            hv, hi = thc.Tensor("half"), thc.Tensor("long")
            hv.max(hi, view, 1)
            assert thc.last_kernel() == "rows-index-lds"
            i = hi.numpy().ravel()
            v = hv.numpy().ravel()
            assert i[0] == 1 and i[3] == 42 and i[4] == 1 and i[5] == 3 and i[7] == R, (R, off, i[:8])
            assert v[0] == -np.inf and np.isnan(v[3]) and v[4] == 1.5 and v[5] == 9.0 and v[7] == 3.0
            assert i[6] == 1 and np.signbit(v[6]), (R, off, i[6], v[6])   # a zero keeps the sign of its first occurrence
            ssum = thc.Tensor("half").sum(view, 1)
            assert thc.last_kernel() == "rows-lds"
            assert ssum.numpy().ravel()[4] == np.float16(1.5 * R) and ssum.numpy().ravel()[7] == -np.inf
    # rows dense in the input, outputs strided (a column of a wider matrix)
    rng = np.random.default_rng(55)
    y = rng.integers(-9, 9, (500, 21)).astype(np.float32)
    wide = thc.Tensor.from_numpy(np.zeros((500, 3), np.float32))
    col = wide.narrow(1, 1, 1)
    col.sum(thc.Tensor.from_numpy(y), 1)
    assert thc.last_kernel() == "rows-lds"
    got = wide.numpy()
    assert_bit_equal(got[:, 1], y.sum(axis=1).astype(np.float32))
    assert not got[:, 0].any() and not got[:, 2].any()
    thc.force_64bit_index(True)
    try:
        out = thc.Tensor("float").sum(thc.Tensor.from_numpy(y), 1)
        assert thc.last_kernel() == "rows-lds"
        assert_bit_equal(out.numpy().ravel(), y.sum(axis=1).astype(np.float32))
    finally:
        thc.force_64bit_index(False)


@pytest.mark.parametrize("kind", ["float", "half"])
def test_small_dense_slices_are_staged_through_lds(thc, oracle, kind):
    """[O][R][C] inputs whose R x C slice is a few KiB: a workgroup stages a
    run of whole slices and a thread (or P threads, when outputs are few)
    takes each output. Ragged last runs, storage offsets, R = 1, one slice."""
    rng = np.random.default_rng(56)
    cases = [((1000, 8, 16), 1), ((500, 33, 2), 1), ((129, 7), 0), ((50, 100, 10), 1), ((3, 2, 5, 7), 1),
             ((3, 2, 5, 7), 2), ((77, 1, 9), 1), ((4100, 2, 3), 1), ((2, 200, 5), 1), ((1, 1000, 4), 1),
             ((300, 3, 130), 1)]
    for shape, dim in cases:
        n = int(np.prod(shape))
        for off in (0, 1, 3) if shape == (500, 33, 2) else (0,):
            st = [1] * len(shape)
            for d in range(len(shape) - 2, -1, -1):
                st[d] = st[d + 1] * shape[d + 1]
            dev, ref = dev_and_ref(thc, oracle, rng, (n + off, off, shape, tuple(st)), kind, "ints")
            # a reduced dim of length 1 counts as unit stride: the short-rows kernel takes it
            ek, eki = ("slab", "slab-index") if shape[dim] > 1 else ("rows-lds", "rows-index-lds")
            for name in ("sum", "norm2", "mean"):
                assert run_reduce(thc, oracle, name, dev, ref, dim, kind) == ek, (shape, dim, name)
            for which in ("max", "min"):
                assert run_minmax(thc, oracle, which, dev, ref, dim, kind) == eki, (shape, dim)
    thc.set_tuning("reduce.slab", 0)
    try:
        dev, ref = dev_and_ref(thc, oracle, rng, contiguous_geometry((500, 33, 2)), kind, "ints")
        assert run_reduce(thc, oracle, "sum", dev, ref, 1, kind).startswith("cols")
        assert run_minmax(thc, oracle, "max", dev, ref, 1, kind).startswith("cols-index")
    finally:
        thc.set_tuning("reduce.slab", 1)


def test_small_dense_slices_special_cases(thc, oracle):
    x = np.full((40, 6, 5), np.inf, np.float32)          # nothing beats min's start value
    x[3, 4, 2] = np.nan
    x[4, :, 1] = -1.0                                    # all tied: first index
    x[5, 2, 0] = x[5, 5, 0] = -3.0
    vals, idx = thc.Tensor("float"), thc.Tensor("long")
    vals.min(idx, thc.Tensor.from_numpy(x), 1)
    assert thc.last_kernel() == "slab-index"
    i, v = idx.numpy()[:, 0, :], vals.numpy()[:, 0, :]
    assert i[0, 0] == 1 and i[3, 2] == 5 and i[4, 1] == 1 and i[5, 0] == 3
    assert v[0, 0] == np.inf and np.isnan(v[3, 2]) and v[4, 1] == -1.0 and v[5, 0] == -3.0
    # outputs strided: a plane of a wider tensor
    rng = np.random.default_rng(57)
    y = rng.integers(-9, 9, (200, 9, 4)).astype(np.float32)
    wide = thc.Tensor.from_numpy(np.zeros((200, 3, 4), np.float32))
    plane = wide.narrow(1, 1, 1)
    plane.sum(thc.Tensor.from_numpy(y), 1)
    assert thc.last_kernel() == "slab"
    got = wide.numpy()
    assert_bit_equal(got[:, 1, :], y.sum(axis=1).astype(np.float32))
    assert not got[:, 0, :].any() and not got[:, 2, :].any()
    thc.force_64bit_index(True)
    try:
        out = thc.Tensor("float").sum(thc.Tensor.from_numpy(y), 1)
        assert thc.last_kernel() == "slab"
        assert_bit_equal(out.numpy()[:, 0, :], y.sum(axis=1).astype(np.float32))
    finally:
        thc.force_64bit_index(False)
    # var / std of small slices: staged once, swept twice in LDS
    z = (rng.standard_normal((300, 12, 6)) * 2 + 5).astype(np.float32)
    out = thc.Tensor("float").var(thc.Tensor.from_numpy(z), 1)
    assert thc.last_kernel() == "var-slab"
    np.testing.assert_allclose(out.numpy()[:, 0, :], z.astype(np.float64).var(axis=1, ddof=1), rtol=1e-5)


@pytest.mark.parametrize("kind", ["float", "half"])
def test_long_narrow_slices_reduce_in_chunks(thc, oracle, kind):
    """Few slices, each long and only a few (misaligned) columns wide: 32 KiB
    runs of rows are reduced to dense partials level by level (also with tiny
    runs, which takes four levels); ragged last chunks; the sum family."""
    rng = np.random.default_rng(58)
    dtype = np.float32 if kind == "float" else np.float16
    x = ((rng.integers(0, 40, (100003, 3)) == 0) * rng.integers(-2, 3, (100003, 3))).astype(dtype)  # fits half
    want = np.abs(x.astype(np.int64)).sum(axis=0, keepdims=True)
    # (first level: slices that start on 16-byte boundaries are read as flat runs of packs, "tall-flat";
    # switched off, the LDS-staged first level runs, "slab-chunked")
    for tall, expect in ((1, "tall-flat"), (0, "slab-chunked")):
        thc.set_tuning("reduce.slab.run_bytes", 512)
        thc.set_tuning("reduce.tall", tall)
        try:
            out = thc.Tensor(kind).norm(thc.Tensor.from_numpy(x), 1, 0)
            assert thc.last_kernel() == expect
        finally:
            thc.set_tuning("reduce.slab.run_bytes", 32768)
            thc.set_tuning("reduce.tall", 1)
        if kind == "float":
            assert_bit_equal(out.numpy(), want.astype(dtype))
        else:
            np.testing.assert_allclose(out.numpy().astype(np.float64), want, rtol=2e-3)
    for shape, dim in (((700001, 3), 0), ((3, 50001, 7), 1), ((120000, 10), 0), ((2, 9000, 33), 1), ((1, 300007, 5), 1),
                       ((2, 40000, 50), 1)):
        x = ((rng.integers(0, 40, shape) == 0) * rng.integers(-2, 3, shape)).astype(dtype)   # sums fit half
        dev, ref = thc.Tensor.from_numpy(x), oracle.View.of(x)
        vec = 4 if kind == "float" else 8
        outer = int(np.prod(shape[:dim]))
        flat = outer == 1 or (shape[dim] * int(np.prod(shape[dim + 1:]))) % vec == 0
        for name in ("sum", "norm1", "norm2", "mean"):
            k = run_reduce(thc, oracle, name, dev, ref, dim, kind)
            assert k == ("tall-flat" if flat else "slab-chunked"), (shape, name, k)
        out = thc.Tensor(kind).sum(dev, dim)                       # exact: small integers
        want = x.astype(np.int64).sum(axis=dim, keepdims=True)
        if np.abs(want).max() < (2048 if kind == "half" else 1 << 24):
            assert_bit_equal(out.numpy(), want.astype(dtype))
    # max / min without indices ride the same engine
    x = rng.standard_normal((90000, 5)).astype(np.float32)
    x[77777, 2] = np.nan
    vals, idx = thc.Tensor("float"), thc.Tensor("long")
    vals.max(idx, thc.Tensor.from_numpy(x), 0)                     # the indexed form has its own flat-pack kernel
    assert thc.last_kernel() == "tall-index"
    assert np.isnan(vals.numpy()[0, 2]) and idx.numpy()[0, 2] == 77778
    # rows of whole aligned packs (4-byte elements; on half the flat runs win there too), or many slices:
    # the column kernels stay
    dev, ref = dev_and_ref(thc, oracle, rng, contiguous_geometry((3, 50000, 8)), kind, "ints")
    assert run_reduce(thc, oracle, "sum", dev, ref, 1, kind).startswith("tall-flat" if kind == "half" else "cols")
    dev, ref = dev_and_ref(thc, oracle, rng, contiguous_geometry((300, 5000, 3)), kind, "ints")
    assert run_reduce(thc, oracle, "sum", dev, ref, 1, kind).startswith("cols")


def test_reductions_beyond_2pow31_elements(thc):
    """More than 2^31 elements in one tensor: the 64-bit index kernels of the
    row, column and whole-tensor reductions at their real size (8.6 GB), not
    forced. The data repeats a block of small integers, so every sum is exact
    in any order and can be predicted on the host; the extreme values are
    planted beyond offset 2^31 with a tie, whose lower index must be returned."""
    from tests.util import device_fill_from_block
    rng = np.random.default_rng(2 ** 31 % 1000)
    L = (1 << 20) + 17                                   # block length, coprime to the shapes used
    block = ((rng.integers(0, 8, L) == 0) * rng.integers(-2, 3, L)).astype(np.float32)
    n = (1 << 31) + 4099 * 4
    x = device_fill_from_block(thc, (n,), block)
    reps, rest = divmod(n, L)
    want_total = float(block.astype(np.int64).sum() * reps + block[:rest].astype(np.int64).sum())
    assert abs(want_total) < 2 ** 24
    assert x.sumall() == want_total
    # the entry point that allocates nothing serves up to 2^32 elements (more workgroups than sumall uses
    # beyond 2^31: another order of the partial sums, which integer-valued data does not notice)
    res = thc.Tensor("float").resize((1,)).fill(-1.0)
    x.sumall_no_alloc(res)
    thc.synchronize()
    assert res.numpy().tolist() == [want_total]
    # 1-D max / min with index: a long single row, split over workgroups and folded
    hi = (1 << 31) + 1234
    for pos in (hi, hi + 4096 + 3):
        x.narrow(0, pos, 1).fill(7.0)
        x.narrow(0, pos + 1, 1).fill(-7.0)
    v, i = thc.Tensor("float"), thc.Tensor("long")
    v.max(i, x, 0)
    assert v.numpy().tolist() == [7.0] and i.numpy().tolist() == [hi + 1]          # 1-based, first of the tie
    v.min(i, x, 0)
    assert v.numpy().tolist() == [-7.0] and i.numpy().tolist() == [hi + 2]
    assert x.maxall() == 7.0 and x.minall() == -7.0
    # 2-D views of the same storage: rows (reduced dim innermost) and columns (reduced dim strided)
    rows, cols = 4096, (1 << 19) + 4                      # 4096 x 524292 = 2^31 + 16384 elements (within the storage)
    assert rows * cols <= n
    m = x.view_as_strided(0, (rows, cols), (cols, 1))
    s = thc.Tensor("float").sum(m, 1)
    assert thc.last_kernel().startswith("rows")
    got = s.numpy().reshape(-1)
    cs = np.concatenate([[0], np.cumsum(np.tile(block.astype(np.int64), 2))])
    starts = (np.arange(rows, dtype=np.int64) * cols) % L
    full, part = divmod(cols, L)
    want = block.astype(np.int64).sum() * full + (cs[starts + part] - cs[starts])
    # the planted +7 / -7 pairs cancel in their rows except where a pair straddles a row end
    patched = np.zeros(rows, np.int64)
    for pos in (hi, hi + 4096 + 3):
        for q, val in ((pos, 7), (pos + 1, -7)):
            patched[q // cols] += val - int(block[q % L])
    assert np.array_equal(got.astype(np.int64), want + patched)
    c = thc.Tensor("float").sum(m, 0)
    assert thc.last_kernel().startswith("cols")
    assert c.shape == (1, cols)
    sample = np.array([0, 1, 5, 4099, 262144, cols - 2, cols - 1])
    offs = (np.arange(rows, dtype=np.int64)[:, None] * cols + sample[None, :])
    colwant = block[offs % L].astype(np.int64)
    for pos in (hi, hi + 4096 + 3):
        for q, val in ((pos, 7), (pos + 1, -7)):
            r, cc = divmod(q, cols)
            hit = np.flatnonzero(sample == cc)
            if hit.size:
                colwant[r, hit[0]] = val
    assert np.array_equal(c.numpy().reshape(-1)[sample].astype(np.int64), colwant.sum(axis=0))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half", "double", "int"])
def test_every_row_length_up_to_300_and_some_beyond(thc, kind):
    """Row reductions pick lanes per row, batch sizes and a partial last batch from the row length:
    every length from 1 to 300 and a few longer ones, rows back to back. Small integers, so sums
    are exact; max/min see ties (lowest index wins), and for the floating types one row with a
    NaN (first NaN wins) and one with zeros of both signs as the extreme (the first keeps its sign)."""
    rng = np.random.default_rng(77)
    dtype = {"float": np.float32, "half": np.float16, "double": np.float64, "int": np.int32}[kind]
    floating = kind in ("float", "half", "double")
    for R in list(range(1, 301)) + [383, 384, 500, 511, 512, 777, 1000, 1536, 2047, 4100]:
        rows = max(3, min(700, 40000 // R))
        x = rng.integers(-6, 7, (rows, R)).astype(dtype)
        if floating and R >= 3:
            x[1, R // 2] = np.nan
            x[1, R - 1] = np.nan
            x[2] = np.minimum(x[2], 0)
            x[2, R // 3] = -0.0
            x[2, R - 1] = 0.0
        dev = thc.Tensor.from_numpy(x)
        got = thc.Tensor(kind).sum(dev, 1).numpy().reshape(rows)
        want = x.astype(np.float64).sum(axis=1).astype(dtype) if floating else x.sum(axis=1, dtype=np.int64).astype(dtype)
        assert_bit_equal(got, want, "%s sum R=%d [%s]" % (kind, R, thc.last_kernel()))
        for which in ("max", "min"):
            v, i = thc.Tensor(kind), thc.Tensor("long")
            getattr(v, which)(i, dev, 1)
            gv, gi = v.numpy().reshape(rows), i.numpy().reshape(rows) - 1
            xf = x.astype(np.float64)
            wi = np.empty(rows, np.int64)
            for r in range(rows):
                nan = np.flatnonzero(np.isnan(xf[r]))
                wi[r] = nan[0] if nan.size else (np.argmax(xf[r]) if which == "max" else np.argmin(xf[r]))
            where = "%s %s R=%d [%s]" % (kind, which, R, thc.last_kernel())
            assert (gi == wi).all(), (where, np.flatnonzero(gi != wi)[:5])
            assert_bit_equal(gv, x[np.arange(rows), wi], where)
