"""cumsum / cumprod (lib/THC/generic/THCTensorMathScan.cu:76-126). Oracle
pinned against numpy.cumsum/cumprod in float64 (and bit-exactly on
integer-valued data); HIP path against the oracle: integer-valued data
bit-exact, random data within 1e-5 of the running mass."""
import numpy as np
import pytest

from tests.util import assert_bit_equal, contiguous_geometry, fill_storage, random_geometry


@pytest.mark.parametrize("seed", range(6))
def test_oracle_scan_matches_numpy(oracle, seed):
    rng = np.random.default_rng(seed)
    nd = int(rng.integers(1, 4))
    shape = tuple(int(x) for x in rng.integers(1, 9, nd))
    dim = int(rng.integers(0, nd))
    n, off, size, stride = random_geometry(rng, shape)
    st = fill_storage(rng, n, dist="uniform")
    src = oracle.View(st, off, size, stride)
    x = src.numpy().astype(np.float64)
    np.testing.assert_allclose(oracle.scan_dim(src, dim).numpy(), np.cumsum(x, axis=dim), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(oracle.scan_dim(src, dim, product=True).numpy(), np.cumprod(x, axis=dim),
                               rtol=1e-6, atol=1e-30)
    xi = rng.integers(-9, 10, shape).astype(np.float32)
    assert_bit_equal(oracle.scan_dim(oracle.View.of(xi), dim).numpy(), np.cumsum(xi.astype(np.int64), axis=dim).astype(np.float32))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half"])
def test_gpu_scan_of_small_slices_goes_through_lds(thc, oracle, kind):
    """Short rows and small R x inner slices are scanned in LDS by a thread per
    column; input and output runs may sit at different misalignments."""
    rng = np.random.default_rng(18)
    dtype = np.float32 if kind == "float" else np.float16
    for shape, dim in (((5000, 10), 1), ((777, 33), 1), ((300, 8, 16), 1), ((1000, 33, 2), 1), ((41, 7), 0),
                       ((2, 3, 5, 7), 2), ((3, 500), 1), ((9, 1, 4), 1), ((1, 60, 60), 1)):
        n = int(np.prod(shape))
        for off in (0, 1, 3):
            st = [1] * len(shape)
            for d in range(len(shape) - 2, -1, -1):
                st[d] = st[d + 1] * shape[d + 1]
            x = rng.integers(-4, 5, n + off).astype(dtype)
            dev = thc.Tensor.from_storage(x, off, shape, tuple(st), kind=kind)
            got = thc.Tensor(kind).cumsum(dev, dim)
            assert thc.last_kernel() == "scan-slab", (shape, dim, thc.last_kernel())
            want = np.cumsum(x[off:].reshape(shape).astype(np.int64), axis=dim).astype(dtype)   # exact: small integers
            assert_bit_equal(got.numpy(), want, "%s %d off %d" % (shape, dim, off))
            dev.cumsum(dev, dim)                                         # in place, misaligned output
            assert_bit_equal(dev.numpy(), want)
            assert_bit_equal(dev.storage_numpy()[:off], x[:off])       # nothing written before the run
    thc.set_tuning("scan.slab", 0)
    try:
        x = rng.integers(-4, 5, (777, 33)).astype(dtype)
        got = thc.Tensor(kind).cumsum(thc.Tensor.from_numpy(x), 1)
        assert thc.last_kernel() == "scan-rows"
        assert_bit_equal(got.numpy(), np.cumsum(x.astype(np.int64), axis=1).astype(dtype))
    finally:
        thc.set_tuning("scan.slab", 1)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half", "int", "double"])
def test_gpu_long_scans_with_few_columns_run_in_chunks(thc, oracle, kind):
    """A scan that would occupy a handful of workgroups is cut into chunks of
    rows: chunk totals, their scan (recursively, here down to three levels with
    small chunks), then every chunk scans from its carry. Exact on small integers."""
    rng = np.random.default_rng(19)
    dtype = {"float": np.float32, "half": np.float16, "int": np.int32, "double": np.float64}[kind]
    for shape, dim, chunk in (((200000, 10), 0, 32768), ((3, 70001), 1, 32768), ((2, 50000, 7), 1, 32768),
                              ((1, 5000, 136), 1, 32768), ((100003, 3), 0, 512), ((2, 40000), 1, 256)):
        sparse = (rng.integers(0, 50, shape) == 0) * rng.integers(-2, 3, shape)     # running sums fit half
        x = sparse.astype(dtype)
        thc.set_tuning("scan.chunk_bytes", chunk)
        thc.set_tuning("scan.cols.split", 0)     # (wide rows would take the split column kernel,
        thc.set_tuning("scan.rows.split", 0)     #  long rows a wave per piece)
        try:
            got = thc.Tensor(kind).cumsum(thc.Tensor.from_numpy(x), dim)
            assert thc.last_kernel() == "scan-chunked", (shape, thc.last_kernel())
            results = [got]
            if kind in ("float", "half"):
                # the one-read form with look-back (off by default: slower), as it is and with readers
                # that never wait (a word that is still empty is computed by the reader itself)
                thc.set_tuning("scan.lookback", 1)
                for spin in (4096, 0):
                    thc.set_tuning("scan.lookback_spin", spin)
                    results.append(thc.Tensor(kind).cumsum(thc.Tensor.from_numpy(x), dim))
                    assert thc.last_kernel() == "scan-lookback", (shape, thc.last_kernel())
                # in place: the two-read form (a reader that gives up waiting would need another chunk's input)
                same = thc.Tensor.from_numpy(x)
                same.cumsum(same, dim)
                assert thc.last_kernel() == "scan-chunked"
                results.append(same)
        finally:
            thc.set_tuning("scan.chunk_bytes", 32768)
            thc.set_tuning("scan.cols.split", 1)
            thc.set_tuning("scan.rows.split", 1)
            thc.set_tuning("scan.lookback", 0)
            thc.set_tuning("scan.lookback_spin", 4096)
        want = np.cumsum(sparse, axis=dim)
        assert np.abs(want).max() < 2048
        for r in results:
            assert_bit_equal(r.numpy(), want.astype(dtype), "%s %s" % (kind, shape))
    rows, every = (150000, 1000) if kind == "double" else (40000, 2000)
    ones = np.ones((rows, 2), dtype)
    ones[::every] = 2
    got = thc.Tensor(kind).cumprod(thc.Tensor.from_numpy(ones), 0)
    assert thc.last_kernel() == "scan-chunked"
    want = np.cumprod(ones, axis=0, dtype=np.int64 if kind == "int" else np.float64)
    if kind == "half":
        assert_bit_equal(got.numpy()[:30000], want[:30000].astype(dtype))   # 2^15 still is a half
    else:
        assert_bit_equal(got.numpy(), want.astype(dtype))
    thc.set_tuning("scan.chunked", 0)
    thc.set_tuning("scan.rows.split", 0)
    try:
        x = rng.integers(-2, 3, (3, 70001)).astype(dtype)
        got = thc.Tensor(kind).cumsum(thc.Tensor.from_numpy(x), 1)
        assert thc.last_kernel() == "scan-rows"
    finally:
        thc.set_tuning("scan.chunked", 1)
        thc.set_tuning("scan.rows.split", 1)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half", "int", "double", "byte", "long"])
def test_gpu_few_long_rows_scan_in_pieces(thc, oracle, kind):
    """A 1-D cumsum (or a few long rows) is cut into pieces that scan side by side, a wave per piece:
    totals of the pieces, their scan, then every piece from its carry. Exact on small integers; row
    lengths that are and are not whole packs, storage offsets off the 16-byte grid, in place."""
    rng = np.random.default_rng(29)
    dtype = {"float": np.float32, "half": np.float16, "int": np.int32, "double": np.float64, "byte": np.uint8,
             "long": np.int64}[kind]
    for shape, dim, off, iters in (((1 << 20,), 0, 0, 8), ((1000003,), 0, 0, 8), ((3, 300000), 1, 0, 8),
                                   ((2, 1, 70001), 2, 1, 2), ((5, 40960), 1, 3, 1), ((1, 123457), 1, 0, 1)):
        n = int(np.prod(shape))
        if kind == "byte":
            sparse = (rng.integers(0, 6000, n + off) == 0) * rng.integers(0, 2, n + off)
        else:
            sparse = (rng.integers(0, 600, n + off) == 0) * rng.integers(-2, 3, n + off)     # running sums fit half
        x = sparse.astype(dtype)
        strides = [1] * len(shape)
        for d in range(len(shape) - 2, -1, -1):
            strides[d] = strides[d + 1] * shape[d + 1]
        thc.set_tuning("scan.rows.split_min_iters", iters)
        try:
            dev = thc.Tensor.from_storage(x, off, shape, tuple(strides), kind=kind)
            got = thc.Tensor(kind).cumsum(dev, dim)
            assert thc.last_kernel() == "scan-rows-split", (shape, thc.last_kernel())
            dev.cumsum(dev, dim)
            assert thc.last_kernel() == "scan-rows-split"
        finally:
            thc.set_tuning("scan.rows.split_min_iters", 8)
        want = np.cumsum(sparse[off:].reshape(shape), axis=dim)
        assert np.abs(want).max() < (256 if kind == "byte" else 2048)
        assert_bit_equal(got.numpy(), want.astype(dtype), "%s %s" % (kind, shape))
        assert_bit_equal(dev.numpy(), want.astype(dtype), "%s %s in place" % (kind, shape))
        assert_bit_equal(dev.storage_numpy()[:off], x[:off])       # nothing written before the rows
    if kind != "byte":
        ones = np.ones((2, 100000), dtype)
        ones[:, ::9000] = 2
        ones[1, 5::17000] = -1
        got = thc.Tensor(kind).cumprod(thc.Tensor.from_numpy(ones), 1)
        assert thc.last_kernel() == "scan-rows-split"
        assert_bit_equal(got.numpy(), np.cumprod(ones.astype(np.float64), axis=1).astype(dtype))
    if kind in ("float", "double"):
        x = rng.standard_normal(3000001).astype(dtype)
        got = thc.Tensor(kind).cumsum(thc.Tensor.from_numpy(x), 0).numpy().astype(np.float64)
        assert thc.last_kernel() == "scan-rows-split"
        want = np.cumsum(x.astype(np.float64))
        mass = np.cumsum(np.abs(x.astype(np.float64)))
        assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(np.abs(want), mass / 64))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half", "int", "double", "byte", "long"])
def test_gpu_long_scans_over_wide_rows_split_the_rows(thc, oracle, kind):
    """A long scan over rows wide enough for the column kernel's lanes, but with too few column tiles
    for the chip, cuts the rows into parts that scan side by side: totals of the parts, their scan,
    then every part from its carry. Exact on small integers; row counts that leave a short last
    part, widths that are and are not whole packs, several slices, in place."""
    rng = np.random.default_rng(23)
    dtype = {"float": np.float32, "half": np.float16, "int": np.int32, "double": np.float64, "byte": np.uint8,
             "long": np.int64}[kind]
    for shape, dim, min_rows in (((20000, 1000), 0, 256), ((3, 9001, 136), 1, 256), ((1, 30011, 257), 1, 256),
                                 ((2, 4099, 64), 1, 64), ((1500, 2000), 0, 64), ((70001, 100), 0, 256)):
        if kind == "byte":
            sparse = (rng.integers(0, 400, shape) == 0) * rng.integers(0, 2, shape)
        else:
            sparse = (rng.integers(0, 50, shape) == 0) * rng.integers(-2, 3, shape)     # running sums fit half
        x = sparse.astype(dtype)
        thc.set_tuning("scan.cols.split_min_rows", min_rows)
        thc.set_tuning("scan.cols.split_min_row_bytes", 1)      # (narrower rows are scanned in chunks by default,
        thc.set_tuning("scan.chunked", 0)                       #  and so are rows that are not whole packs)
        try:
            got = thc.Tensor(kind).cumsum(thc.Tensor.from_numpy(x), dim)
            assert thc.last_kernel() == "scan-cols-split", (shape, thc.last_kernel())
            same = thc.Tensor.from_numpy(x)
            same.cumsum(same, dim)
            assert thc.last_kernel() == "scan-cols-split"
        finally:
            thc.set_tuning("scan.cols.split_min_rows", 256)
            thc.set_tuning("scan.cols.split_min_row_bytes", 256)
            thc.set_tuning("scan.chunked", 1)
        want = np.cumsum(sparse, axis=dim)
        assert np.abs(want).max() < (256 if kind == "byte" else 2048)
        assert_bit_equal(got.numpy(), want.astype(dtype), "%s %s" % (kind, shape))
        assert_bit_equal(same.numpy(), want.astype(dtype), "%s %s in place" % (kind, shape))
    if kind != "byte":
        ones = np.ones((9000, 320), dtype)
        ones[::700] = 2
        ones[1::1300, ::7] = -1
        got = thc.Tensor(kind).cumprod(thc.Tensor.from_numpy(ones), 0)
        assert thc.last_kernel() == "scan-cols-split"
        assert_bit_equal(got.numpy(), np.cumprod(ones.astype(np.float64), axis=0).astype(dtype))
    if kind in ("float", "double"):
        x = rng.standard_normal((50000, 520)).astype(dtype)
        dev, ref = thc.Tensor.from_numpy(x), oracle.View.of(x)
        got = thc.Tensor(kind).cumsum(dev, 0).numpy().astype(np.float64)
        assert thc.last_kernel() == "scan-cols-split"
        want = oracle.scan_dim(ref, 0).numpy().astype(np.float64) if kind == "float" else np.cumsum(x, axis=0)
        mass = np.cumsum(np.abs(x.astype(np.float64)), axis=0)
        assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(np.abs(want), mass / 64))
    thc.set_tuning("scan.cols.split", 0)
    try:
        x = ((rng.integers(0, 50, (20000, 1000)) == 0) * 1).astype(dtype)
        got = thc.Tensor(kind).cumsum(thc.Tensor.from_numpy(x), 0)
        assert thc.last_kernel() in ("scan-cols", "scan-chunked")
        assert_bit_equal(got.numpy(), np.cumsum(x.astype(np.int64), axis=0).astype(dtype))
    finally:
        thc.set_tuning("scan.cols.split", 1)


@pytest.mark.gpu
@pytest.mark.parametrize("slab", [1, 0])
@pytest.mark.parametrize("kind", ["float", "half"])
def test_gpu_scan(thc, oracle, kind, slab):
    thc.set_tuning("scan.slab", slab)
    try:
        _gpu_scan_cases(thc, oracle, kind)
    finally:
        thc.set_tuning("scan.slab", 1)


def _gpu_scan_cases(thc, oracle, kind):
    rng = np.random.default_rng(17)
    dtype = np.float32 if kind == "float" else np.float16
    tol = 1e-5 if kind == "float" else 2e-3
    for shape, dim in (((7, 1000), 1), ((3, 257), 1), ((300, 5), 1), ((50, 64), 0), ((4, 33, 20), 1),
                       ((2, 3, 4, 130), 3), ((1,), 0), ((9000,), 0), ((6, 5, 1), 1), ((2, 1000, 24), 1),
                       ((3, 300, 7), 1), ((1, 5000, 136), 1), ((700, 2), 0), ((5, 2049), 1), ((2, 130, 8, 16), 1)):
        geom = random_geometry(rng, shape) if len(shape) == 3 else contiguous_geometry(shape)
        st = rng.uniform(-1, 1, geom[0]).astype(dtype)
        dev = thc.Tensor.from_storage(st, *geom[1:], kind=kind)
        ref = oracle.View(st.copy(), *geom[1:])
        got = thc.Tensor(kind).cumsum(dev, dim)
        assert got.shape == tuple(shape)
        want = oracle.scan_dim(ref, dim).numpy().astype(np.float64)
        mass = np.cumsum(np.abs(ref.numpy().astype(np.float64)), axis=dim)
        err = np.abs(got.numpy().astype(np.float64) - want) / np.maximum(np.abs(want), mass * 2.0 ** -6 + 1e-30)
        assert err.max() <= tol, (shape, dim, err.max())
        stp = rng.uniform(0.9, 1.1, geom[0]).astype(dtype)
        devp = thc.Tensor.from_storage(stp, *geom[1:], kind=kind)
        gotp = thc.Tensor(kind).cumprod(devp, dim).numpy().astype(np.float64)
        wantp = oracle.scan_dim(oracle.View(stp.copy(), *geom[1:]), dim, product=True).numpy().astype(np.float64)
        # (one step of half's subnormal grid where a product has decayed that far)
        np.testing.assert_allclose(gotp, wantp, rtol=max(tol, 2e-5) * 4, atol=6e-8 if kind == "half" else 0)
    xi = rng.integers(-9, 10, (37, 700)).astype(np.float32)
    for dim in (0, 1):
        got = thc.Tensor("float").cumsum(thc.Tensor.from_numpy(xi), dim)
        assert_bit_equal(got.numpy(), np.cumsum(xi.astype(np.int64), axis=dim).astype(np.float32))
    t = thc.Tensor.from_numpy(xi)
    t.cumsum(t, 1)                                               # in place
    assert_bit_equal(t.numpy(), np.cumsum(xi.astype(np.int64), axis=1).astype(np.float32))
    with pytest.raises(thc.THCError, match="out of range"):
        thc.Tensor("float").cumsum(thc.Tensor.from_numpy(xi), 2)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half", "int", "double"])
def test_gpu_scan_over_a_strided_dim_in_every_strip_width(thc, oracle, kind):
    """The scan over a non-innermost dim picks a strip width (8-64 lanes) and whether the next
    segment's packs are requested ahead from the shape and the chip; here each is forced in turn.
    Small integers: exact whatever the split; row counts off the segment size; an odd inner size
    takes the element-wise variant."""
    rng = np.random.default_rng(23)
    dtype = {"float": np.float32, "half": np.float16, "int": np.int32, "double": np.float64}[kind]
    thc.set_tuning("scan.chunked", 0)       # (few long slices would otherwise be cut into chunks of rows,
    thc.set_tuning("scan.slab", 0)          #  small ones scanned in LDS,
    thc.set_tuning("scan.cols.split", 0)    #  long ones over wide rows cut into parts of rows)
    try:
        for shape in ((3, 300, 520), (2, 129, 1024), (1, 64, 96), (2, 1000, 136), (1, 77, 515), (5, 1, 8192), (4, 9, 4100)):
            sparse = (rng.integers(0, 12, shape) == 0) * rng.integers(-2, 3, shape)
            x = thc.Tensor.from_numpy(sparse.astype(dtype))
            want = np.cumsum(sparse, axis=1)
            assert np.abs(want).max() < 2048
            for pf in (0, 1):
                for tx in (8, 16, 32, 64):
                    thc.set_tuning("scan.cols.prefetch", pf)
                    thc.set_tuning("scan.cols.min_tx", tx)
                    thc.set_tuning("scan.cols.max_tx", tx)
                    got = thc.Tensor(kind).cumsum(x, 1)
                    assert thc.last_kernel() == "scan-cols", (shape, thc.last_kernel())
                    assert_bit_equal(got.numpy(), want.astype(dtype), "%s %s pf=%d tx=%d" % (kind, shape, pf, tx))
    finally:
        thc.set_tuning("scan.chunked", 1)
        thc.set_tuning("scan.slab", 1)
        thc.set_tuning("scan.cols.split", 1)
        thc.set_tuning("scan.cols.prefetch", -1)
        thc.set_tuning("scan.cols.min_tx", 8)
        thc.set_tuning("scan.cols.max_tx", 64)
