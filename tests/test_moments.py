"""var / std / varall / stdall / dist (sibling reductions on the reduce engine:
generic/THCTensorMathReduce.cu:70-144,234-259). The oracle is pinned against
numpy's float64 var/std (ddof 0 and 1); the HIP path, which centres the data
first (two sweeps), must agree with it to 1e-5 relative."""
import numpy as np
import pytest

from tests.util import contiguous_geometry, fill_storage, random_geometry


def _np_view(st, off, size, stride):
    return np.lib.stride_tricks.as_strided(st[off:], shape=size, strides=tuple(4 * s for s in stride))


@pytest.mark.parametrize("seed", range(6))
def test_oracle_var_std_match_numpy(oracle, seed):
    rng = np.random.default_rng(seed)
    nd = int(rng.integers(1, 4))
    shape = tuple(int(x) for x in rng.integers(2, 9, nd))
    dim = int(rng.integers(0, nd))
    n, off, size, stride = random_geometry(rng, shape)
    st = (fill_storage(rng, n) * 3 + 5).astype(np.float32)
    src = oracle.View(st, off, size, stride)
    x = _np_view(st, off, size, stride).astype(np.float64)
    for kind, f, ddof in (("var", np.var, 1), ("var_biased", np.var, 0), ("std", np.std, 1),
                          ("std_biased", np.std, 0)):
        got = oracle.reduce_dim(kind, src, dim).numpy()
        np.testing.assert_allclose(got, f(x, axis=dim, ddof=ddof, keepdims=True), rtol=2e-6)
    assert abs(oracle.var_all(src) - x.var(ddof=1)) <= 1e-12 * x.var()
    assert abs(oracle.var_all(src, biased=True) - x.var()) <= 1e-12 * x.var()


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half"])
def test_gpu_var_std(thc, oracle, kind):
    rng = np.random.default_rng(7)
    tol = 1e-5 if kind == "float" else 2e-3
    dtype = np.float32 if kind == "float" else np.float16
    for shape, dim in (((64, 1024), 1), ((300, 7), 1), ((16, 500, 24), 1), ((9, 33), 0), ((5, 6, 7), 2)):
        geom = contiguous_geometry(shape) if len(shape) == 2 else random_geometry(rng, shape)
        st = (rng.standard_normal(geom[0]) * 2 + 3).astype(dtype)     # mean 3, sd 2
        dev = thc.Tensor.from_storage(st, *geom[1:], kind=kind)
        ref = oracle.View(st.copy(), *geom[1:])
        for biased in (0, 1):
            for name in ("var", "std"):
                out = getattr(thc.Tensor(kind), name)(dev, dim, biased)
                want = oracle.reduce_dim(name + ("_biased" if biased else ""), ref, dim).numpy()
                assert out.shape == want.shape
                np.testing.assert_allclose(out.numpy().astype(np.float64), want.astype(np.float64),
                                           rtol=tol, err_msg="%s %s dim %d" % (name, shape, dim))
        out = thc.Tensor(kind).var(dev, dim, 0, 0)
        assert out.shape == tuple(s for d, s in enumerate(shape) if d != dim)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half", "double"])
def test_gpu_varall_of_a_dense_tensor_is_one_read(thc, kind):
    """Welford per lane plus pairwise merges: sizes around the pack and batch
    boundaries, a storage offset (scalar loads), a large common offset, and an
    outlier in front, all against float64 numpy; the two-sweep form, reached
    with the kernel switched off or through a strided view, agrees."""
    rng = np.random.default_rng(81)
    dtype = {"float": np.float32, "half": np.float16, "double": np.float64}[kind]
    tol = {"float": 2e-5, "half": 2e-3, "double": 1e-12}[kind]
    for n in (1, 2, 5, 1023, 8192, 8193, 100003, (1 << 21) + 3):
        for off in (0, 1):
            x = (rng.standard_normal(n + off) * 0.5 + (3.0 if kind == "half" else 1000.0)).astype(dtype)
            x[off] = -7.0                                              # outlier first
            dev = thc.Tensor.from_storage(x, off, (n,), (1,), kind=kind)
            ref = x[off:].astype(np.float64)
            for biased in (0, 1):
                if n == 1 and not biased:
                    continue
                want = ref.var(ddof=0 if biased else 1)
                got = dev.varall(biased)
                assert thc.last_kernel() == "all-moments"
                assert abs(got - want) <= tol * max(want, 1e-30), (kind, n, off, biased, got, want)
    x = (rng.standard_normal((300, 70)) + 5).astype(dtype)
    dev = thc.Tensor.from_numpy(x)
    a = dev.varall(0)
    thc.set_tuning("reduce.all.moments", 0)
    try:
        b = dev.varall(0)
        assert thc.last_kernel() != "all-moments"
    finally:
        thc.set_tuning("reduce.all.moments", 1)
    c = dev.t().varall(0)                                            # not one dense run in logical order
    want = x.astype(np.float64).var(ddof=1)
    for v in (a, b, c):
        assert abs(v - want) <= tol * want


@pytest.mark.gpu
def test_gpu_varall_stdall_dist(thc, oracle):
    rng = np.random.default_rng(8)
    for shape in ((1000,), (257, 129), (1 << 20,)):
        geom = random_geometry(rng, shape) if len(shape) == 2 else contiguous_geometry(shape)
        st = (rng.standard_normal(geom[0]) * 2 + 10).astype(np.float32)
        dev = thc.Tensor.from_storage(st, *geom[1:])
        ref = oracle.View(st.copy(), *geom[1:])
        for biased in (0, 1):
            want = oracle.var_all(ref, bool(biased))
            assert abs(dev.varall(biased) - want) <= 1e-5 * want
            assert abs(dev.stdall(biased) - np.sqrt(want)) <= 1e-5 * np.sqrt(want)
        st2 = rng.standard_normal(geom[0]).astype(np.float32)
        other = thc.Tensor.from_storage(st2, *geom[1:])
        x = ref.numpy().astype(np.float64)
        y = oracle.View(st2.copy(), *geom[1:]).numpy().astype(np.float64)
        for p in (1.0, 2.0, 3.0):
            want = (np.abs(x - y) ** p).sum() ** (1 / p)
            assert abs(dev.dist(other, p) - want) <= 1e-5 * want
    e = thc.Tensor("float")
    with pytest.raises(thc.THCError, match="empty Tensor"):
        e.varall()


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half"])
def test_gpu_var_rows_single_read_and_fallback(thc, oracle, kind):
    """Rows that fit a lane group's registers take the one-read kernel; longer
    rows, ragged lengths and offsets that break 16-byte alignment take the
    two-sweep form. Both must agree with the oracle."""
    rng = np.random.default_rng(8)
    tol = 1e-5 if kind == "float" else 2e-3
    dtype = np.float32 if kind == "float" else np.float16
    vec = 4 if kind == "float" else 8
    for shape, expect in (((300, 1024), "var-rows"), ((7, 64 * vec * 8), "var-rows"), ((5, 8), "var-rows"),
                          ((3, 64 * vec * 8 + vec), "rows"), ((50, 1023), "var-rows-lds"), ((2, 40000), None)):
        x = (rng.standard_normal(shape) * 2 + 3).astype(dtype)
        dev, ref = thc.Tensor.from_numpy(x), oracle.View.of(x)
        for name, okind in (("var", "var"), ("std", "std")):
            for biased in (0, 1):
                out = getattr(thc.Tensor(kind), name)(dev, 1, biased=biased)
                if expect:
                    assert thc.last_kernel() == expect, (shape, thc.last_kernel())
                want = oracle.reduce_dim(okind + ("_biased" if biased else ""), ref, 1).numpy().astype(np.float64)
                np.testing.assert_allclose(out.numpy().astype(np.float64), want, rtol=tol, atol=tol * 1e-2)
    out = thc.Tensor(kind).var(thc.Tensor.from_numpy(np.ones((4, 16), dtype)), 1, keepdim=0)
    assert out.shape == (4,) and np.all(out.numpy() == 0)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half"])
def test_gpu_var_along_strided_dim_is_one_read_and_stable(thc, oracle, kind):
    """Welford along a strided dim: the large common offset (mean 1000 x the
    spread for float) must not cost accuracy, split and unsplit shapes."""
    rng = np.random.default_rng(9)
    tol = 1e-5 if kind == "float" else 2e-3
    dtype = np.float32 if kind == "float" else np.float16
    offset = 100.0 if kind == "float" else 4.0
    for shape, dim, expect in (((64, 512), 0, "var-cols"), ((6, 300, 40), 1, "var-cols"),
                               ((2, 8192, 96), 1, "var-cols-split"), ((129, 7), 0, "var-slab"),
                               ((3, 50, 8, 24), 1, "var-cols")):
        x = (rng.standard_normal(shape) * 0.1 + offset).astype(dtype)
        dev, ref = thc.Tensor.from_numpy(x), oracle.View.of(x)
        for name in ("var", "std"):
            for biased in (0, 1):
                out = getattr(thc.Tensor(kind), name)(dev, dim, biased=biased)
                k = thc.last_kernel()      # (half: long narrow slices of whole packs take the flat runs as well)
                assert k.startswith(expect.replace("-scalar", "")) or (kind == "half" and k == "var-tall"), (shape, k)
                want = oracle.reduce_dim(name + ("_biased" if biased else ""), ref, dim).numpy().astype(np.float64)
                np.testing.assert_allclose(out.numpy().astype(np.float64), want, rtol=tol * (8 if kind == "float" else 1),
                                           atol=0, err_msg="%s %s %s" % (shape, name, kind))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half", "double"])
def test_gpu_var_of_long_rows_is_one_read(thc, kind):
    """Rows too long for a lane group's registers (statistics over thousands of features) with enough
    rows for the chip: a wave per row runs (count, mean, M2) per lane and merges; against float64 numpy
    with a common offset of 40 sigma (8 for half), row lengths off the batch size, a strided row pitch."""
    rng = np.random.default_rng(84)
    dtype = {"float": np.float32, "half": np.float16, "double": np.float64}[kind]
    tol = {"float": 2e-5, "half": 4e-3, "double": 1e-12}[kind]
    centre = 4.0 if kind == "half" else 20.0
    vec = 16 // np.dtype(dtype).itemsize
    for rows, n, pitch in ((1500, 8192, 8192), (1100, 64 * vec * 8 + vec, 64 * vec * 8 + vec), (1030, 5000 // vec * vec, 6000 // vec * vec),
                           (2, 1024, 70000 // vec * vec)):
        store = (rng.standard_normal(rows * pitch) * 0.5 + centre).astype(dtype)
        dev = thc.Tensor.from_storage(store, 0, (rows, n), (pitch, 1), kind=kind)
        ref = store.reshape(rows, pitch)[:, :n].astype(np.float64)
        for name, fn in (("var", np.var), ("std", np.std)):
            for biased in (0, 1):
                out = getattr(thc.Tensor(kind), name)(dev, 1, biased=biased)
                if rows >= 1024:
                    assert thc.last_kernel() == "var-rows-long", (rows, n, thc.last_kernel())
                want = fn(ref, axis=1, ddof=0 if biased else 1, keepdims=True)
                np.testing.assert_allclose(out.numpy().astype(np.float64), want, rtol=tol, err_msg="%s %s %d x %d" % (kind, name, rows, n))
    x = (rng.standard_normal((1200, 4096)) + centre).astype(dtype)
    dev = thc.Tensor.from_numpy(x)
    a = thc.Tensor(kind).var(dev, 1).numpy()
    assert np.array_equal(a, thc.Tensor(kind).var(dev, 1).numpy())        # same bits on every run
    thc.set_tuning("reduce.var.long_rows", 0)
    try:
        b = thc.Tensor(kind).var(dev, 1).numpy()
        assert thc.last_kernel() != "var-rows-long"
    finally:
        thc.set_tuning("reduce.var.long_rows", 1)
    np.testing.assert_allclose(a.astype(np.float64), b.astype(np.float64), rtol=tol)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half", "double"])
def test_gpu_var_of_long_narrow_slices_reads_flat_packs(thc, kind):
    """Few long slices of narrow rows (batch statistics of a tall matrix) are read as flat runs of
    aligned packs with a running (count, mean, M2) per lane and column: against float64 numpy, with a
    common offset of 40 sigma (8 for half), column counts with every period of the pack pattern,
    slices with elements behind the last whole pack, several slices, and a first row that is an
    outlier (what a shifted one-pass sum would lose)."""
    rng = np.random.default_rng(83)
    dtype = {"float": np.float32, "half": np.float16, "double": np.float64}[kind]
    tol = {"float": 2e-5, "half": 4e-3, "double": 1e-12}[kind]
    centre = 4.0 if kind == "half" else 20.0
    vec = 16 // np.dtype(dtype).itemsize
    cases = [((200003, 3), 0), ((70001, 10), 0), ((30000, 33), 0), ((2, 40000, 7), 1), ((3, 16000, 5), 1),
             ((1, 50001, 9), 1), ((90001, 1, 6), 0), ((25000, 50), 0)]
    for shape, dim in cases:
        x = (rng.standard_normal(shape) * 0.5 + centre).astype(dtype)
        x[(0,) * len(shape)] = 60.0 if kind == "half" else 1e4
        dev = thc.Tensor.from_numpy(x)
        ref = x.astype(np.float64)
        inner = int(np.prod(shape[dim + 1:]))
        outer = int(np.prod(shape[:dim]))
        flat = inner % vec != 0 and (outer == 1 or (shape[dim] * inner) % vec == 0)
        for name, fn in (("var", np.var), ("std", np.std)):
            for biased in (0, 1):
                out = getattr(thc.Tensor(kind), name)(dev, dim, biased=biased)
                assert thc.last_kernel() == ("var-tall" if flat else "var-cols-split"), (shape, dim, thc.last_kernel())
                want = fn(ref, axis=dim, ddof=0 if biased else 1, keepdims=True)
                np.testing.assert_allclose(out.numpy().astype(np.float64), want, rtol=tol,
                                           err_msg="%s %s %s" % (kind, name, shape))
    x = (rng.standard_normal((70001, 10)) + centre).astype(dtype)
    dev = thc.Tensor.from_numpy(x)
    a = thc.Tensor(kind).var(dev, 0).numpy()
    thc.set_tuning("reduce.tall", 0)
    try:
        b = thc.Tensor(kind).var(dev, 0).numpy()
        assert thc.last_kernel() == "var-cols-split"
    finally:
        thc.set_tuning("reduce.tall", 1)
    np.testing.assert_allclose(a.astype(np.float64), b.astype(np.float64), rtol=tol)
    assert_same = thc.Tensor(kind).var(dev, 0).numpy()
    assert np.array_equal(a, assert_same)        # same bits on every run


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half", "double"])
def test_gpu_var_of_short_rows_and_small_slices_is_one_read(thc, kind):
    """Dense short rows and small R x C slices are staged in LDS and swept
    there twice (mean, squared deviations): row lengths around the group
    sizes, misaligned storage offsets, a common offset of 40 sigma, against float64
    numpy."""
    rng = np.random.default_rng(82)
    dtype = {"float": np.float32, "half": np.float16, "double": np.float64}[kind]
    tol = {"float": 2e-5, "half": 4e-3, "double": 1e-12}[kind]
    centre = 3.0 if kind == "half" else 20.0
    atol = {"float": 1e-6, "half": 2e-3, "double": 1e-14}[kind]    # rounding of the mean, squared-deviation scale
    cases = [((1000, 2), 1), ((777, 10), 1), ((300, 33), 1), ((64, 100), 1), ((9, 1001), 1), ((4, 5, 70), 2),
             ((500, 8, 16), 1), ((300, 33, 2), 1), ((129, 7), 0), ((40, 100, 10), 1), ((3, 2, 5, 7), 2)]
    for shape, dim in cases:
        n = int(np.prod(shape))
        for off in (0, 1, 3):
            x = (rng.standard_normal(n + off) * 0.5 + centre).astype(dtype)
            strides = [1] * len(shape)
            for d in range(len(shape) - 2, -1, -1):
                strides[d] = strides[d + 1] * shape[d + 1]
            dev = thc.Tensor.from_storage(x, off, shape, tuple(strides), kind=kind)
            ref = x[off:].reshape(shape).astype(np.float64)
            # rows that are whole aligned packs keep the register kernel
            expect = ("var-rows-lds", "var-rows") if dim == len(shape) - 1 else ("var-slab",)
            if shape == (300, 33) or (off % 2 and dim == len(shape) - 1):
                expect = ("var-rows-lds",)
            for name, fn in (("var", np.var), ("std", np.std)):
                for biased in (0, 1):
                    out = getattr(thc.Tensor(kind), name)(dev, dim, biased=biased)
                    assert thc.last_kernel() in expect, (shape, dim, off, thc.last_kernel())
                    want = fn(ref, axis=dim, ddof=0 if biased else 1, keepdims=True)
                    np.testing.assert_allclose(out.numpy().astype(np.float64), want, rtol=tol, atol=atol,
                                               err_msg="%s %s %s off %d" % (kind, name, shape, off))
