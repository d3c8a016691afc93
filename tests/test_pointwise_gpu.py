"""Parity of the HIP apply engine with the CPU oracle, through the C ABI.

Method of cutorch's own suite (test/test.lua:232-323): the same seeded host
data is mirrored to the device with identical storage / offset / size /
stride, the op runs on both sides, and results are compared -- here bit for
bit over the WHOLE storage, so stray writes into holes are caught too
(copyRandomizedTest, test/test.lua:700-727).
Bar: add/sub/mul/div/cadd/addcmul/addcdiv and the scalar forms are bit-exact
(one correctly rounded binary32 operation per step, no fusion)."""
import numpy as np
import pytest

from tests.util import (assert_bit_equal, contiguous_geometry, device_fill_from_block, fill_storage,
                        random_geometry)

pytestmark = pytest.mark.gpu

BINARY = {"cadd1": ("add", 1.0), "cadd": ("cadd", 0.37), "csub1": ("sub", 1.0), "csub": ("cadd", -2.5),
          "cmul": ("mul", 0.0), "cdiv": ("div", 0.0)}


def run_binary(thc, oracle, name, geoms, rng, inplace=False, dist="normal", kind="float"):
    """geoms = [out, a, b] as (storage_len, offset, size, stride)."""
    dtype = np.float16 if kind == "half" else np.float32
    sts = [fill_storage(rng, g[0], dtype, dist) for g in geoms]
    if not inplace:
        sts[0][:] = np.nan
    dev = [thc.Tensor.from_storage(s, g[1], g[2], g[3], kind) for s, g in zip(sts, geoms)]
    ref = [oracle.View(s.copy(), g[1], g[2], g[3]) for s, g in zip(sts, geoms)]
    if inplace:
        dev[1], ref[1] = dev[0], ref[0]
    oop, v = BINARY[name]
    meth = name.rstrip("1")
    if meth in ("cadd", "csub"):
        value = 1.0 if name.endswith("1") else (0.37 if meth == "cadd" else 2.5)
        getattr(dev[0], meth)(dev[1], value, dev[2])
    else:
        getattr(dev[0], meth)(dev[1], dev[2])
    if kind == "half":          # a half tensor's scalar argument is a half too
        v = float(np.float16(v))
    oracle.pointwise(oop, ref[0], ref[1], ref[2], value=v)
    assert dev[0].shape == ref[1].size
    assert_bit_equal(dev[0].storage_numpy(), ref[0].storage, name)
    return thc.last_kernel()


@pytest.mark.parametrize("name", sorted(BINARY))
def test_contiguous_1d(thc, oracle, name):
    rng = np.random.default_rng(1)
    for n in (1, 3, 4, 1023, 1024, 4097, 100003):
        g = contiguous_geometry((n,))
        k = run_binary(thc, oracle, name, [g, g, g], rng, dist="uniform")
        assert k.startswith("contig")


def test_contiguous_config1_shape(thc, oracle):
    """c = a + b and c = a * b on 2^24 uniform[-1,1] elements (benchmark config 1)."""
    rng = np.random.default_rng(0xC0FFEE + 1)
    g = contiguous_geometry((1 << 24,))
    assert run_binary(thc, oracle, "cadd1", [g, g, g], rng, dist="uniform") == "contig"
    assert run_binary(thc, oracle, "cmul", [g, g, g], rng, dist="uniform") == "contig"


def test_misaligned_contiguous_views(thc, oracle):
    rng = np.random.default_rng(2)
    for off in (1, 2, 3, 5):
        g = (5000 + off, off, (5000,), (1,))
        g0 = contiguous_geometry((5000,))
        run_binary(thc, oracle, "cadd1", [g0, g, g0], rng)
        run_binary(thc, oracle, "cmul", [g, g0, g], rng)


@pytest.mark.parametrize("seed", range(40))
def test_random_strided_geometries(thc, oracle, seed):
    rng = np.random.default_rng(seed)
    nd = int(rng.integers(1, 6))
    shape = tuple(int(x) for x in rng.integers(1, 12, nd))
    geoms = [random_geometry(rng, shape, holes=rng.random() < 0.6, permute=rng.random() < 0.6)
             for _ in range(3)]
    name = sorted(BINARY)[seed % len(BINARY)]
    run_binary(thc, oracle, name, geoms, rng, inplace=(seed % 5 == 0))


@pytest.mark.parametrize("shift", [2, 1, 0])
@pytest.mark.parametrize("force64", [False, True])
@pytest.mark.parametrize("shape", [(64, 64), (70, 131), (257, 33), (8, 8), (5, 300, 7), (3, 40, 50),
                                   (128, 4, 96), (1, 200, 200), (2, 3, 65, 67)])
def test_transposed_operand_uses_tiles(thc, oracle, shape, force64, shift):
    """One operand's unit-stride dim is the first logical dim (a:t(), or a
    permute(3,2,1) view); out and b are contiguous. Rows that are not 16-byte
    aligned run on the line-aligned ragged variant (shift = 2), with it
    switched off on the shifted-window variant, and with that switched off
    too on the element-wise one."""
    rng = np.random.default_rng(sum(shape))
    thc.set_tuning("apply.tiled.ragged", 1 if shift == 2 else 0)
    thc.set_tuning("apply.tiled.shift", 1 if shift else 0)
    nd = len(shape)
    st, run = [0] * nd, 1
    for d in range(nd):            # dim 0 innermost in memory
        st[d] = run
        run *= shape[d]
    ga = (run, 0, shape, tuple(st))
    gc = contiguous_geometry(shape)
    thc.force_64bit_index(force64)
    try:
        k = run_binary(thc, oracle, "cadd1", [gc, ga, gc], rng)
        k2 = run_binary(thc, oracle, "cmul", [gc, gc, ga], rng)
        k3 = run_binary(thc, oracle, "cdiv", [ga, gc, gc], rng)   # transposed OUTPUT
    finally:
        thc.force_64bit_index(False)
        thc.set_tuning("apply.tiled.shift", 1)
        thc.set_tuning("apply.tiled.ragged", 1)
    dims = [s for s in shape if s != 1]
    if dims[0] >= 8 and dims[-1] >= 8:      # tiny tile dims fall back to the strided kernel
        assert k.startswith("tiled") and k2.startswith("tiled") and k3.startswith("tiled"), (k, k2, k3)
        if dims[0] % 4 or dims[-1] % 4:
            assert k == ("tiled-ragged", "tiled-shift", "tiled-scalar")[2 - shift], k
    else:
        assert k.startswith("strided"), (k, k2, k3)


@pytest.fixture
def no_ragged_tiles(thc):
    """Keeps 4-byte element types off the line-aligned ragged variant, so that the shifted-window
    variant (which otherwise serves the other element sizes only) runs."""
    thc.set_tuning("apply.tiled.ragged", 0)
    yield
    thc.set_tuning("apply.tiled.ragged", 1)


def run_exact(thc, name, geoms, rng, kind, inplace=False):
    """run_binary for any element type, on small integers (exact in every type) against numpy
    views of the same storages: name = cadd1 (a + b), cadd (a + 3 b) or cmul."""
    dtype = {"float": np.float32, "double": np.float64, "int": np.int32, "long": np.int64}[kind]
    sts = [rng.integers(-9, 10, g[0]).astype(dtype) for g in geoms]
    dev = [thc.Tensor.from_storage(s, g[1], g[2], g[3], kind) for s, g in zip(sts, geoms)]
    want = [s.copy() for s in sts]
    item = np.dtype(dtype).itemsize
    view = [np.lib.stride_tricks.as_strided(w[g[1]:], g[2], tuple(x * item for x in g[3])) for w, g in zip(want, geoms)]
    if inplace:
        dev[1], view[1] = dev[0], view[0]
    if name == "cmul":
        dev[0].cmul(dev[1], dev[2])
        view[0][...] = view[1] * view[2]
    else:
        value = 1 if name == "cadd1" else 3
        dev[0].cadd(dev[1], value, dev[2])
        view[0][...] = view[1] + value * view[2]
    assert_bit_equal(dev[0].storage_numpy(), want[0], "%s %s" % (kind, name))
    return thc.last_kernel()


@pytest.mark.parametrize("kind", ["float", "int", "double", "long"])
def test_line_aligned_ragged_tiles(thc, oracle, kind):
    """4- and 8-byte elements, rows that start anywhere in a cache line: tiles that cut every row at its
    own line boundaries. Sizes around the tile edges (64 x 128, up to 31 columns of slack; 32 x 64 and 15
    for 8-byte elements) and off the
    pack width, views 1..3 elements into their storage, storages that start rows at every offset
    within a line (pitches 129, 130, 161, 8193 mod 32), rows with gaps, a batch dim in front, a
    transposed output, two staged inputs and in-place use. Whole storages are compared, so a store
    outside the tensor's own elements fails the test."""
    rng = np.random.default_rng(81)
    for rows, cols in ((64, 128), (65, 129), (63, 127), (61, 125), (129, 257), (333, 515), (1001, 67), (9, 700),
                       (70, 97), (200, 161), (130, 130)):
        for off in (0, 1, 3, 17):
            ga = (rows * cols + off, off, (rows, cols), (1, rows))          # a:t()
            gc = (rows * cols + off, off, (rows, cols), (cols, 1))
            vec = 2 if kind in ("double", "long") else 4
            aligned = rows % vec == 0 and cols % vec == 0 and off % vec == 0
            want = "tiled" if aligned else "tiled-ragged"
            assert run_exact(thc, "cadd1", [gc, ga, gc], rng, kind) == want, (rows, cols, off)
            assert run_exact(thc, "cadd", [gc, gc, ga], rng, kind, inplace=True) == want, (rows, cols, off)
            assert run_exact(thc, "cadd1", [ga, ga, gc], rng, kind) == want, (rows, cols, off)   # transposed output
            # transposed output, two staged inputs: of 4-byte elements they would leave the ragged tiles one
            # workgroup per CU, so odd shapes take the shifted windows there
            k = run_exact(thc, "cmul", [ga, gc, gc], rng, kind)
            assert k == ("tiled" if aligned else ("tiled-ragged" if vec == 2 else "tiled-shift")), (rows, cols, off, k)
    # rows with gaps (a narrowed view of a wider matrix), transposed partner at another offset
    gout = (200 * 131 + 2, 2, (200, 127), (131, 1))
    ga = (127 * 203 + 1, 1, (200, 127), (1, 203))
    gb = (200 * 131 + 2, 2, (200, 127), (131, 1))
    assert run_exact(thc, "cadd", [gout, ga, gb], rng, kind) == "tiled-ragged"
    # b starts one element later than out: its packs would not be aligned, the element-wise variant runs
    gb = (200 * 131 + 3, 3, (200, 127), (131, 1))
    assert run_exact(thc, "cadd", [gout, ga, gb], rng, kind) == "tiled-scalar"
    # (for 8-byte elements out at offset 2 is pack-aligned and b at offset 3 is not: the same case)
    g3 = (7 * 130 * 401 + 5, 5, (7, 401, 130), (130 * 401, 1, 401))     # batch dim in front, p = 401
    gd = (7 * 401 * 130 + 5, 5, (7, 401, 130), (401 * 130, 130, 1))
    assert run_exact(thc, "cmul", [gd, g3, gd], rng, kind) == "tiled-ragged"


def test_line_aligned_ragged_tiles_with_three_inputs(thc, oracle):
    """addcmul on odd shapes with one, two and three transposed inputs: one staged input runs on the
    ragged tiles (41 KiB of LDS), two on the shifted windows, three on neither; 32- and 64-bit offsets."""
    rng = np.random.default_rng(83)
    rows, cols = 331, 203
    x, y, z = (rng.integers(-5, 6, (cols, rows)).astype(np.float32) for _ in range(3))     # used as x.t()
    u, v, w = (rng.integers(-5, 6, (rows, cols)).astype(np.float32) for _ in range(3))
    dev = {n: thc.Tensor.from_numpy(a) for n, a in dict(x=x, y=y, z=z, u=u, v=v, w=w).items()}
    for force64 in (False, True):
        thc.force_64bit_index(force64)
        try:
            out = thc.Tensor("float").addcmul(dev["u"], 2.0, dev["x"].t(), dev["v"])
            assert thc.last_kernel() == "tiled-ragged"
            assert_bit_equal(out.numpy(), u + 2.0 * x.T * v)
            out = thc.Tensor("float").addcmul(dev["u"], 2.0, dev["v"], dev["x"].t())
            assert thc.last_kernel() == "tiled-ragged"
            assert_bit_equal(out.numpy(), u + 2.0 * v * x.T)
            out = thc.Tensor("float").addcmul(dev["x"].t(), 2.0, dev["u"], dev["v"])
            assert thc.last_kernel() == "tiled-ragged"
            assert_bit_equal(out.numpy(), x.T + 2.0 * u * v)
            out = thc.Tensor("float").addcmul(dev["u"], 2.0, dev["x"].t(), dev["y"].t())
            assert thc.last_kernel() == "tiled-shift"                                        # two staged inputs
            assert_bit_equal(out.numpy(), u + 2.0 * x.T * y.T)
            out = thc.Tensor("float").addcmul(dev["x"].t(), 0.5, dev["y"].t(), dev["z"].t())
            assert thc.last_kernel().startswith("tiled") or thc.last_kernel().startswith("strided"), thc.last_kernel()
            assert_bit_equal(out.numpy(), x.T + 0.5 * y.T * z.T)
            dev["w"].addcmul(dev["w"], 2.0, dev["x"].t(), dev["v"])                          # in place
            assert thc.last_kernel() == "tiled-ragged"
            w = w + 2.0 * x.T * v
            assert_bit_equal(dev["w"].numpy(), w)
        finally:
            thc.force_64bit_index(False)


@pytest.mark.parametrize("kind", ["float", "half"])
def test_shifted_window_tiles_at_every_misalignment(thc, oracle, kind, no_ragged_tiles):
    """Sizes around the window edges (a tile spans 4 elements fewer than its
    window; 8 for half), views that start 1..3 elements into their storage,
    rows with gaps, and operands whose misalignments differ (those fall back
    to the element-wise variant). Whole storages are compared, so a store
    outside the tensor's own elements fails the test."""
    rng = np.random.default_rng(77)
    for rows, cols in ((60, 124), (61, 125), (59, 123), (121, 249), (333, 515), (1001, 67)):
        for off in (0, 1, 3):
            ga = (rows * cols + off, off, (rows, cols), (1, rows))          # a:t()
            gc = (rows * cols + off, off, (rows, cols), (cols, 1))
            k = run_binary(thc, oracle, "cadd1", [gc, ga, gc], rng, kind=kind)
            vec = 8 if kind == "half" else 4
            aligned = rows % vec == 0 and cols % vec == 0 and off == 0
            assert k == ("tiled" if aligned else "tiled-shift"), (rows, cols, off, k)
            k = run_binary(thc, oracle, "cmul", [ga, gc, gc], rng, kind=kind)   # transposed output
            assert k.startswith("tiled"), k
    # rows with gaps (a narrowed view of a wider matrix), transposed partner at another offset
    gout = (200 * 131 + 2, 2, (200, 127), (131, 1))
    ga = (127 * 203 + 1, 1, (200, 127), (1, 203))
    gb = (200 * 131 + 2, 2, (200, 127), (131, 1))
    assert run_binary(thc, oracle, "cadd", [gout, ga, gb], rng, kind=kind) == "tiled-shift"
    # b starts one element later than out: no common window
    gb = (200 * 131 + 3, 3, (200, 127), (131, 1))
    assert run_binary(thc, oracle, "cadd", [gout, ga, gb], rng, kind=kind) == "tiled-scalar"
    # b's rows drift against out's (row strides differ modulo the pack width)
    gb = (200 * 130 + 2, 2, (200, 127), (130, 1))
    assert run_binary(thc, oracle, "cadd", [gout, ga, gb], rng, kind=kind) == "tiled-scalar"


def test_shifted_window_tiles_with_two_staged_inputs(thc, oracle, no_ragged_tiles):
    rng = np.random.default_rng(78)
    x = rng.standard_normal((203, 331)).astype(np.float32)
    y = rng.standard_normal((203, 331)).astype(np.float32)
    z = rng.standard_normal((331, 203)).astype(np.float32)
    dx, dy, dz = (thc.Tensor.from_numpy(v) for v in (x, y, z))
    out = thc.Tensor("float").addcmul(dz, 0.5, dx.t(), dy.t())
    assert thc.last_kernel() == "tiled-shift"
    want = oracle.pointwise("addcmul", oracle.View.empty((331, 203)), oracle.View.of(z),
                            oracle.View(x.reshape(-1).copy(), 0, (331, 203), (1, 331)),
                            oracle.View(y.reshape(-1).copy(), 0, (331, 203), (1, 331)), value=0.5)
    assert_bit_equal(out.numpy(), want.numpy())
    out = thc.Tensor("float").cadd(dx.t(), 2.0, dy.t())      # both inputs staged, nothing direct but out
    assert_bit_equal(out.numpy(), (x.T + np.float32(2.0) * y.T).astype(np.float32))


def test_all_operands_transposed_alike_is_flat(thc, oracle):
    rng = np.random.default_rng(5)
    g = (60 * 80, 0, (60, 80), (1, 60))
    assert run_binary(thc, oracle, "cadd1", [g, g, g], rng) == "contig"


def test_operands_of_different_shape_pair_by_linear_index(thc, oracle):
    rng = np.random.default_rng(6)
    ga = contiguous_geometry((6, 20))
    gb = (120, 0, (10, 12), (1, 10))
    gout = contiguous_geometry((4, 30))
    sts = [fill_storage(rng, g[0]) for g in (gout, ga, gb)]
    dev = [thc.Tensor.from_storage(s, g[1], g[2], g[3]) for s, g in zip(sts, (gout, ga, gb))]
    ref = [oracle.View(s.copy(), g[1], g[2], g[3]) for s, g in zip(sts, (gout, ga, gb))]
    dev[0].cmul(dev[1], dev[2])                 # resizes out to a's shape
    assert dev[0].shape == (6, 20) and thc.last_kernel() == "generic"
    out_ref = oracle.View(ref[0].storage, 0, (6, 20))
    oracle.pointwise("mul", out_ref, ref[1], ref[2])
    assert_bit_equal(dev[0].storage_numpy(), out_ref.storage)


@pytest.mark.parametrize("name,oop", [("add", "addc"), ("sub", "subc"), ("mul", "mulc"), ("div", "divc")])
def test_scalar_forms(thc, oracle, name, oop):
    rng = np.random.default_rng(8)
    for shape, inplace in (((1000,), False), ((33, 47), True), ((9, 10, 11), False)):
        g_in = random_geometry(rng, shape)
        g_out = contiguous_geometry(shape)
        st_in, st_out = fill_storage(rng, g_in[0]), np.full(g_out[0], np.nan, np.float32)
        a = thc.Tensor.from_storage(st_in, *g_in[1:])
        ra = oracle.View(st_in.copy(), *g_in[1:])
        if inplace:
            out, rout = a, ra
        else:
            out = thc.Tensor.from_storage(st_out, *g_out[1:])
            rout = oracle.View(st_out.copy(), *g_out[1:])
        getattr(out, name)(a, 3.0)
        oracle.pointwise(oop, rout, ra, value=3.0)
        assert_bit_equal(out.storage_numpy(), rout.storage, name)


def test_scalar_divide_is_a_true_division(thc):
    x = np.arange(1, 2001, dtype=np.float32)
    t = thc.Tensor.from_numpy(x)
    out = thc.Tensor("float").div(t, 3.0)
    assert_bit_equal(out.numpy(), x / np.float32(3.0))
    assert np.any(x / np.float32(3.0) != x * (np.float32(1.0) / np.float32(3.0)))


@pytest.mark.parametrize("op", ["addcmul", "addcdiv"])
@pytest.mark.parametrize("value", [1.0, -0.75])
def test_addcmul_addcdiv(thc, oracle, op, value):
    rng = np.random.default_rng(9)
    for shape, inplace in (((4099,), False), ((64, 96), False), ((31, 65), True), ((6, 7, 8), False)):
        geoms = [contiguous_geometry(shape)] + [random_geometry(rng, shape) for _ in range(3)]
        if len(shape) == 2:   # the benchmark's pattern: src1 transposed
            geoms[2] = (shape[0] * shape[1], 0, shape, (1, shape[0]))
        sts = [fill_storage(rng, g[0]) for g in geoms]
        dev = [thc.Tensor.from_storage(s, *g[1:]) for s, g in zip(sts, geoms)]
        ref = [oracle.View(s.copy(), *g[1:]) for s, g in zip(sts, geoms)]
        if inplace:
            dev[0], ref[0] = dev[1], ref[1]
        getattr(dev[0], op)(dev[1], value, dev[2], dev[3])
        oracle.pointwise(op, ref[0], ref[1], ref[2], ref[3], value=value)
        assert_bit_equal(dev[0].storage_numpy(), ref[0].storage, op)


def test_unfused_multiply_add(thc):
    b = np.full(1024, 1 + 2.0 ** -12, dtype=np.float32)
    d = np.full(1024, -(1 + 2.0 ** -11), dtype=np.float32)
    out = thc.Tensor("float").addcmul(thc.Tensor.from_numpy(d), 1.0, thc.Tensor.from_numpy(b),
                                      thc.Tensor.from_numpy(b))
    assert np.all(out.numpy() == 0.0)          # an FMA would give 2^-24


def test_special_values(thc, oracle):
    a = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, 3e38, 1.0, -1e-40, 1e-39] * 13, dtype=np.float32)
    b = np.array([-0.0, 0.0, -np.inf, 2.0, 1.0, 1e-45, 3e38, 3.0, 1e-40, 0.5] * 13, dtype=np.float32)
    for name, oop in (("cadd", "add"), ("cmul", "mul"), ("cdiv", "div"), ("csub", "sub")):
        out = thc.Tensor("float")
        args = (thc.Tensor.from_numpy(a), 1.0, thc.Tensor.from_numpy(b)) if name in ("cadd", "csub") \
            else (thc.Tensor.from_numpy(a), thc.Tensor.from_numpy(b))
        getattr(out, name)(*args)
        r = oracle.View.empty(a.shape)
        oracle.pointwise(oop, r, oracle.View.of(a), oracle.View.of(b))
        got, want = out.numpy(), r.storage
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan)
        assert_bit_equal(got[~nan], want[~nan], name)   # denormals and signed zeros included


def test_overlapping_output_goes_through_a_dense_temporary(thc):
    # out is an expanded (stride 0) view: every row aliases the same 8 floats;
    # the reference semantics is "some writer wins" (THCApply.cuh:148-164)
    st = np.zeros(8, dtype=np.float32)
    out = thc.Tensor.from_storage(st, 0, (4, 8), (0, 1))
    a = thc.Tensor.from_numpy(np.arange(32, dtype=np.float32).reshape(4, 8))
    b = thc.Tensor.from_numpy(np.ones((4, 8), dtype=np.float32))
    out.cadd(a, 1.0, b)
    got = out.storage_numpy()
    cand = np.arange(32, dtype=np.float32).reshape(4, 8) + 1
    assert all(got[j] in cand[:, j] for j in range(8))


def test_empty_and_error_paths(thc):
    e = thc.Tensor("float")
    out = thc.Tensor("float").cadd(e, 1.0, e)            # zero-dim: no-op
    assert out.shape == ()
    a = thc.Tensor.from_numpy(np.zeros(6, np.float32))
    b = thc.Tensor.from_numpy(np.zeros(7, np.float32))
    with pytest.raises(thc.THCError, match="sizes do not match"):
        thc.Tensor("float").cadd(a, 1.0, b)
    with pytest.raises(thc.THCError, match="divide by zero"):
        thc.Tensor("float").div(a, 0.0)
    # the engine still works after an error was delivered
    assert np.all(thc.Tensor("float").cadd(a, 1.0, a).numpy() == 0)


def test_half_pointwise_rounds_once(thc, oracle):
    rng = np.random.default_rng(12)
    for shape in ((4096,), (33, 70), (130, 129)):
        gs = [contiguous_geometry(shape), random_geometry(rng, shape), contiguous_geometry(shape)]
        if len(shape) == 2:
            gs[1] = (shape[0] * shape[1], 0, shape, (1, shape[0]))
        for name in ("cadd1", "cmul", "cdiv", "cadd"):
            run_binary(thc, oracle, name, gs, rng, dist="uniform", kind="half")


def test_strided_copy_and_contiguous(thc):
    rng = np.random.default_rng(13)
    x = rng.standard_normal((37, 53)).astype(np.float32)
    t = thc.Tensor.from_numpy(x).t()
    assert not t.is_contiguous()
    assert_bit_equal(t.contiguous().numpy(), x.T)
    assert_bit_equal(t.numpy(), x.T)
    idx = thc.Tensor.from_numpy(np.arange(24, dtype=np.int64).reshape(4, 6)).t()
    assert np.array_equal(idx.contiguous().numpy(), np.arange(24).reshape(4, 6).T)


def test_large_transposed_roundtrip_property(thc):
    """Full benchmark size (8192x8192, a:t()): (a:t() * 1 + 0) transposed back
    equals a -- checked on the device, independent of the oracle."""
    n = 8192
    rng = np.random.default_rng(14)
    x = rng.standard_normal((n, n)).astype(np.float32)
    a = thc.Tensor.from_numpy(x)
    ones = thc.Tensor.from_numpy(np.ones((n, n), np.float32))
    out = thc.Tensor("float").cmul(a.t(), ones)
    assert thc.last_kernel() == "tiled"
    back = thc.Tensor("float").cmul(out.t(), ones)
    assert_bit_equal(back.numpy(), x)


def test_config2_full_size_against_the_oracle(thc, oracle):
    """The headline workload itself: out = a:t() * b + d (addcmul, value 1) on
    8192 x 8192 fp32 with the benchmark's seed, a viewed transposed; the whole
    output storage bit for bit against the CPU oracle (8 threads, ~0.1 s)."""
    n = 8192
    rng = np.random.default_rng(0xC0FFEE)
    a = rng.standard_normal((n, n), dtype=np.float32)
    b = rng.standard_normal((n, n), dtype=np.float32)
    d = rng.standard_normal((n, n), dtype=np.float32)
    out = thc.Tensor("float").addcmul(thc.Tensor.from_numpy(d), 1.0, thc.Tensor.from_numpy(a).t(),
                                      thc.Tensor.from_numpy(b))
    assert thc.last_kernel() == "tiled" and out.shape == (n, n)
    va = oracle.View(a.reshape(-1), 0, (n, n), (1, n))
    ref = oracle.View.empty((n, n))
    oracle.set_num_threads(8)
    try:
        oracle.pointwise("addcmul", ref, oracle.View(d.reshape(-1), 0, (n, n)), va,
                         oracle.View(b.reshape(-1), 0, (n, n)), value=1.0)
    finally:
        oracle.set_num_threads(1)
    assert_bit_equal(out.storage_numpy(), ref.storage, "config 2 at full size")
    # in place on d, as cutorch's addcmul(self == t) runs it
    dd = thc.Tensor.from_numpy(d)
    dd.addcmul(dd, 1.0, thc.Tensor.from_numpy(a).t(), thc.Tensor.from_numpy(b))
    assert_bit_equal(dd.storage_numpy(), ref.storage, "config 2 in place")


def test_config5_full_size_64bit_index_path(thc):
    """c = a + b on 2048 x 2048 x 520 fp32 (2.18e9 elements, 26 GB), a being a
    permute(3,2,1) view of a dense 520 x 2048 x 2048 tensor. The operands repeat
    a known block, so every element of the result can be predicted on the host:
    a[i,j,k] = blockA[(k*2048*2048 + j*2048 + i) % L], b[i,j,k] = blockB[(i*2048*520 + j*520 + k) % L].
    The WHOLE output is compared bit for bit, slab by slab (32 of the 2048
    (j,k) planes at a time, the closed form evaluated on host threads)."""
    from concurrent.futures import ThreadPoolExecutor
    rng = np.random.default_rng(0xC0FFEE + 5)
    L = (1 << 22) + 12345                          # block length coprime to the dims
    ba = rng.standard_normal(L).astype(np.float32)
    bb = rng.standard_normal(L).astype(np.float32)
    a = device_fill_from_block(thc, (520, 2048, 2048), ba)
    b = device_fill_from_block(thc, (2048, 2048, 520), bb)
    av = a.view_as_strided(0, (2048, 2048, 520), (1, 2048, 2048 * 2048))
    assert not av.is_contiguous()
    c = thc.Tensor("float").cadd(av, 1.0, b)
    assert thc.last_kernel().startswith("tiled") and c.shape == (2048, 2048, 520)
    j = np.arange(2048, dtype=np.int64)[:, None]
    k = np.arange(520, dtype=np.int64)[None, :]
    plane = 2048 * 520
    idx_a0 = ((k * 2048 * 2048 + j * 2048) % L).astype(np.int32)     # a's block index at i = 0
    bb2 = np.concatenate([bb, bb[:plane]])                           # a plane of b is one run of the block

    def mismatches(i0, got):
        assert got.shape == (32, 2048, 520) and got.dtype == np.float32
        bad = 0
        for d in range(got.shape[0]):
            i = i0 + d
            ia = idx_a0 + np.int32(i)
            ia -= np.int32(L) * (ia >= L)
            start = (i * plane) % L
            want = ba[ia] + bb2[start:start + plane].reshape(2048, 520)
            bad += int(np.count_nonzero(got[d].view(np.uint32) != want.view(np.uint32)))
        return bad

    step, pending, bad = 32, [], 0
    with ThreadPoolExecutor(max_workers=8) as pool:
        for i0 in range(0, 2048, step):
            pending.append(pool.submit(mismatches, i0, c.narrow(0, i0, step).numpy()))
            while len(pending) > 10:
                bad += pending.pop(0).result()
        for f in pending:
            bad += f.result()
    assert bad == 0, "%d of %d elements differ" % (bad, 2048 * plane)
    # a plane across i (fixed j): strided gather on the device side as well
    i = np.arange(2048, dtype=np.int64)[:, None]
    for jj in (0, 2047):
        want = ba[(k * 2048 * 2048 + jj * 2048 + i) % L] + bb[(i * 2048 * 520 + jj * 520 + k) % L]
        assert_bit_equal(c.select(1, jj).numpy(), want, "plane j=%d" % jj)


@pytest.mark.parametrize("kind", ["float", "half"])
def test_broadcast_operands_on_rows_that_are_not_pack_aligned(thc, kind):
    """x + bias where bias is a stride-0 view (row bias, column bias, a scalar, a
    middle-dim bias) and the rows of x are not 16-byte aligned: the dense
    operands stream as flat aligned packs, the broadcast one is gathered element
    by element. Aligned shapes keep the strided / tiled pack kernels; a
    permuted operand of full size never takes this route."""
    rng = np.random.default_rng(90)
    dtype = np.float32 if kind == "float" else np.float16
    for shape in ((333, 515), (61, 1001), (7, 9, 131), (1001,), (2, 3, 5, 67)):
        n = int(np.prod(shape))
        nd = len(shape)
        x = rng.integers(-8, 9, shape).astype(dtype)
        dx = thc.Tensor.from_numpy(x)
        for d in range(nd):
            bias = rng.integers(-8, 9, shape[d]).astype(dtype)
            strides = tuple(1 if k == d else 0 for k in range(nd))
            db = thc.Tensor.from_numpy(bias).view_as_strided(0, shape, strides)
            view = bias.reshape([shape[d] if k == d else 1 for k in range(nd)])
            if nd == 1:
                continue                                   # a 1-D "bias" is just a dense operand
            out = thc.Tensor(kind).cadd(dx, 1.0, db)
            assert thc.last_kernel() == "flat-gather", (shape, d, thc.last_kernel())
            assert_bit_equal(out.numpy(), (x + view).astype(dtype))
            out = thc.Tensor(kind).cmul(db, dx)             # broadcast operand first
            assert thc.last_kernel() == "flat-gather"
            assert_bit_equal(out.numpy(), (x * view).astype(dtype))
            if nd == 2:
                both = thc.Tensor(kind).addcmul(dx, 1.0, db, db)       # two gathered inputs
                assert thc.last_kernel() == "flat-gather"
                assert_bit_equal(both.numpy(), (x + view * view).astype(dtype))
        scalar = thc.Tensor.from_numpy(np.array([3], dtype)).view_as_strided(0, shape, (0,) * nd)
        acc = thc.Tensor.from_numpy(x.copy())
        acc.cadd(acc, 2.0, scalar)                          # in place on the dense operand
        assert thc.last_kernel() == "flat-gather"
        assert_bit_equal(acc.numpy(), (x + dtype(6)).astype(dtype))
    # aligned rows: the strided pack kernel is the faster one and stays
    x = rng.integers(-8, 9, (64, 256)).astype(dtype)
    bias = rng.integers(-8, 9, 256).astype(dtype)
    db = thc.Tensor.from_numpy(bias).view_as_strided(0, (64, 256), (0, 1))
    out = thc.Tensor(kind).cadd(thc.Tensor.from_numpy(x), 1.0, db)
    assert thc.last_kernel() == "strided"
    assert_bit_equal(out.numpy(), (x + bias).astype(dtype))
    # a transposed operand of the output's own size is not a broadcast
    y = rng.integers(-8, 9, (515, 333)).astype(dtype)
    out = thc.Tensor(kind).cadd(thc.Tensor.from_numpy(y).t(), 1.0, thc.Tensor.from_numpy(y.T.copy()))
    assert thc.last_kernel().startswith("tiled")
    assert_bit_equal(out.numpy(), (y.T + y.T).astype(dtype))
    thc.set_tuning("apply.flatmix", 0)
    try:
        x = rng.integers(-8, 9, (333, 515)).astype(dtype)
        bias = rng.integers(-8, 9, 515).astype(dtype)
        db = thc.Tensor.from_numpy(bias).view_as_strided(0, (333, 515), (0, 1))
        out = thc.Tensor(kind).cadd(thc.Tensor.from_numpy(x), 1.0, db)
        assert thc.last_kernel() in ("strided-scalar", "strided-unaligned")     # (packs for 4- and 8-byte elements)
        assert_bit_equal(out.numpy(), (x + bias).astype(dtype))
    finally:
        thc.set_tuning("apply.flatmix", 1)


@pytest.mark.parametrize("kind", ["float", "half", "int", "double"])
def test_rows_of_a_few_elements_with_a_repeated_operand(thc, kind):
    """(N, 3) scaled by a column, (N, 2, 5) plus a per-N offset: the output and one input are one dense
    run, the other input is the output's own order with dims repeated (stride 0) and as large as N; under
    rows of a few elements it is gathered beside the flat packs instead of going element by element."""
    rng = np.random.default_rng(78)
    dtype = {"float": np.float32, "half": np.float16, "int": np.int32, "double": np.float64}[kind]
    for shape, rep_strides in (((70001, 3), (1, 0)), ((4099, 2, 5), (1, 0, 0)), ((3001, 4, 3), (4, 1, 0)), ((50000, 7), (1, 0))):
        x = rng.integers(-4, 5, shape).astype(dtype)
        small_shape = tuple(n if st else 1 for n, st in zip(shape, rep_strides))
        rep = rng.integers(-3, 4, small_shape).astype(dtype)
        dx = thc.Tensor.from_numpy(x)
        drep = thc.Tensor.from_numpy(rep.reshape(-1)).view_as_strided(0, shape, rep_strides)
        flat = kind in ("float", "half")          # (the other types' functors have no flat + gathered kernel)
        out = thc.Tensor(kind).cmul(dx, drep)
        assert not flat or thc.last_kernel() == "flat-gather", (kind, shape, thc.last_kernel())
        assert_bit_equal(out.numpy(), (x * rep).astype(dtype))
        acc = thc.Tensor.from_numpy(x.copy())
        acc.cadd(acc, 2, drep)                                   # in place on the dense operand
        assert not flat or thc.last_kernel() == "flat-gather"
        assert_bit_equal(acc.numpy(), (x + dtype(2) * rep).astype(dtype))
    thc.set_tuning("apply.flatmix.repeated", 0)
    try:
        x = rng.integers(-4, 5, (5000, 3)).astype(dtype)
        col = rng.integers(-3, 4, (5000, 1)).astype(dtype)
        out = thc.Tensor(kind).cmul(thc.Tensor.from_numpy(x), thc.Tensor.from_numpy(col.reshape(-1)).view_as_strided(0, (5000, 3), (1, 0)))
        assert thc.last_kernel() != "flat-gather"
        assert_bit_equal(out.numpy(), (x * col).astype(dtype))
    finally:
        thc.set_tuning("apply.flatmix.repeated", 1)


@pytest.mark.parametrize("kind", ["float", "int", "double", "long", "half", "byte"])
def test_strided_rows_off_the_16_byte_grid(thc, kind):
    """Views whose rows start off the 16-byte grid and have odd lengths (x[:, 1:-2] of a wider matrix):
    the elements move as packs at element-aligned addresses with a partial last pack per row (rows
    shorter than four packs element by element). In place and out of place, one to three inputs, every
    operand at its own offset; the whole destination storage is compared."""
    rng = np.random.default_rng(77)
    dtype = {"float": np.float32, "int": np.int32, "double": np.float64, "long": np.int64, "half": np.float16,
             "byte": np.uint8}[kind]
    wide = True      # (packs at element-aligned addresses for every element size)
    for rows, cols, pitch, offs in ((37, 101, 128, (1, 3, 2, 5)), (64, 8187, 8200, (3, 1, 1, 2)), (5, 16, 19, (1, 2, 3, 0)),
                                    (3, 7, 9, (1, 1, 1, 1)), (200, 33, 40, (0, 1, 2, 3)), (6, 700, 4097, (5, 6, 7, 9))):
        lo, hi = (0, 5) if kind == "byte" else (-4, 5)
        hosts = [rng.integers(lo, hi, rows * pitch + 16).astype(dtype) for _ in range(4)]
        def view(i):
            return thc.Tensor.from_storage(hosts[i], offs[i], (rows, cols), (pitch, 1), kind=kind)
        def host_view(i):
            return np.lib.stride_tricks.as_strided(hosts[i][offs[i]:], (rows, cols), (pitch * dtype().itemsize, dtype().itemsize))
        expect = "strided-unaligned" if wide and cols >= 4 * (16 // dtype().itemsize) else "strided-scalar"
        # two inputs, out of place
        out = view(0)
        out.cadd(view(1), 2, view(2))
        k = thc.last_kernel()
        want = hosts[0].copy()
        np.lib.stride_tricks.as_strided(want[offs[0]:], (rows, cols), (pitch * dtype().itemsize, dtype().itemsize))[...] = \
            (host_view(1) + dtype(2) * host_view(2)).astype(dtype)
        assert k in (expect, "strided"), (kind, rows, cols, k)
        assert_bit_equal(out.storage_numpy(), want, "%s cadd %dx%d %s" % (kind, rows, cols, k))
        # one input, in place
        acc = view(3)
        acc.mul(acc, 3)
        want3 = hosts[3].copy()
        np.lib.stride_tricks.as_strided(want3[offs[3]:], (rows, cols), (pitch * dtype().itemsize, dtype().itemsize))[...] = \
            (host_view(3) * dtype(3)).astype(dtype)
        assert_bit_equal(acc.storage_numpy(), want3, "%s mul in place %dx%d" % (kind, rows, cols))
        # copy between views at different offsets, and a fill
        dst = view(0)
        dst.copy(view(2))
        want0 = hosts[0].copy()
        np.lib.stride_tricks.as_strided(want0[offs[0]:], (rows, cols), (pitch * dtype().itemsize, dtype().itemsize))[...] = host_view(2)
        assert_bit_equal(dst.storage_numpy(), want0, "%s copy %dx%d %s" % (kind, rows, cols, thc.last_kernel()))
        f = view(1)
        f.fill(2)
        want1 = hosts[1].copy()
        np.lib.stride_tricks.as_strided(want1[offs[1]:], (rows, cols), (pitch * dtype().itemsize, dtype().itemsize))[...] = dtype(2)
        assert_bit_equal(f.storage_numpy(), want1, "%s fill %dx%d %s" % (kind, rows, cols, thc.last_kernel()))
    if kind == "float":
        # three inputs, and a comparison into a Byte tensor (4 elements per pack on both sides)
        rows, cols, pitch = 50, 1001, 1024
        hs = [rng.integers(-4, 5, rows * pitch + 8).astype(np.float32) for _ in range(4)]
        vs = [thc.Tensor.from_storage(h, o, (rows, cols), (pitch, 1)) for h, o in zip(hs, (1, 2, 3, 1))]
        hv = [np.lib.stride_tricks.as_strided(h[o:], (rows, cols), (pitch * 4, 4)) for h, o in zip(hs, (1, 2, 3, 1))]
        vs[0].addcmul(vs[1], 2.0, vs[2], vs[3])
        assert thc.last_kernel() == "strided-unaligned"
        want = hs[0].copy()
        np.lib.stride_tricks.as_strided(want[1:], (rows, cols), (pitch * 4, 4))[...] = hv[1] + np.float32(2) * hv[2] * hv[3]
        assert_bit_equal(vs[0].storage_numpy(), want)
        mstore = np.full(rows * pitch + 8, 9, np.uint8)
        mask = thc.Tensor.from_storage(mstore, 4, (rows, cols), (pitch, 1), kind="byte")
        mask.compare_tensor("lt", vs[2], vs[3])
        wantm = mstore.copy()
        np.lib.stride_tricks.as_strided(wantm[4:], (rows, cols), (pitch, 1))[...] = (hv[2] < hv[3]).astype(np.uint8)
        assert_bit_equal(mask.storage_numpy(), wantm, "lt into bytes %s" % thc.last_kernel())


@pytest.mark.parametrize("band", [1, 2, 3, 8])
def test_shifted_window_tiles_in_bands_along_p(thc, oracle, band, no_ragged_tiles):
    """The shifted-window variant walks its tiles in bands of `band` tiles along
    p (p fastest inside a band): whole bands, a ragged last band, and shapes
    too short in p for banding must all cover every tile exactly once."""
    rng = np.random.default_rng(91)
    thc.set_tuning("apply.tiled.group_p", band)
    try:
        for rows, cols in ((333, 515), (400, 130), (1001, 67), (61, 125), (977, 251)):
            ga = (rows * cols + 1, 1, (rows, cols), (1, rows))           # a:t(), one element into its storage
            gc = contiguous_geometry((rows, cols))
            assert run_binary(thc, oracle, "cadd", [gc, ga, gc], rng) == "tiled-shift"
        g3 = (7 * 130 * 401, 0, (7, 401, 130), (130 * 401, 1, 401))      # batch dim in front, p = 401
        assert run_binary(thc, oracle, "cmul", [contiguous_geometry((7, 401, 130)), g3,
                                                contiguous_geometry((7, 401, 130))], rng) == "tiled-shift"
    finally:
        thc.set_tuning("apply.tiled.group_p", 8)


@pytest.mark.parametrize("cap", [1, 7, 64])
def test_tiled_variants_with_several_tiles_per_workgroup(thc, oracle, cap):
    """With the grid capped below the number of tiles a workgroup walks several tiles and reuses its
    LDS slabs: every tiled variant (pack, fused q, ragged, shifted windows, element-wise) must still
    cover every tile exactly once."""
    rng = np.random.default_rng(93)
    thc.set_tuning("apply.tiled.max_grid", cap)
    try:
        gc = contiguous_geometry((320, 512))
        assert run_binary(thc, oracle, "cadd", [gc, (320 * 512, 0, (320, 512), (1, 320)), gc], rng) == "tiled"
        gp = (40 * 24 * 520, 0, (520, 24, 40), (1, 520, 520 * 24))
        assert run_binary(thc, oracle, "cadd", [contiguous_geometry((520, 24, 40)), gp,
                                                contiguous_geometry((520, 24, 40))], rng) == "tiled-fused"
        go = contiguous_geometry((333, 515))
        ga = (333 * 515 + 1, 1, (333, 515), (1, 333))
        assert run_binary(thc, oracle, "cadd", [go, ga, go], rng) == "tiled-ragged"
        assert run_binary(thc, oracle, "cadd", [go, ga, go], rng, kind="half") == "tiled-shift"
        thc.set_tuning("apply.tiled.ragged", 0)
        assert run_binary(thc, oracle, "cadd", [go, ga, go], rng) == "tiled-shift"
        thc.set_tuning("apply.tiled.shift", 0)
        assert run_binary(thc, oracle, "cadd", [go, ga, go], rng) == "tiled-scalar"
    finally:
        thc.set_tuning("apply.tiled.max_grid", 1 << 22)
        thc.set_tuning("apply.tiled.ragged", 1)
        thc.set_tuning("apply.tiled.shift", 1)


@pytest.mark.parametrize("band", [1, 2, 3, 16])
def test_aligned_tiles_in_bands_along_p(thc, oracle, band):
    """The pack variant of the tiled kernel can walk its tiles in bands along p too (the default
    for single-input ops): whole bands, a ragged last band, a batch dim in front, fused q."""
    rng = np.random.default_rng(92)
    thc.set_tuning("apply.tiled.group_p_vec", band)
    thc.set_tuning("apply.skinny", 0)          # (copies with a dim of at most 256 bytes would leave the tiled kernel)
    try:
        for rows, cols in ((320, 512), (448, 132), (1000, 64), (2304, 128)):
            ga = (rows * cols, 0, (rows, cols), (1, rows))               # a:t()
            gc = contiguous_geometry((rows, cols))
            assert run_binary(thc, oracle, "cadd", [gc, ga, gc], rng) == "tiled"
            src = thc.Tensor.from_numpy(rng.integers(-99, 100, (cols, rows)).astype(np.float32))
            out = thc.Tensor("float").resize((rows, cols)).copy(src.t())
            assert thc.last_kernel() == "tiled"
            assert_bit_equal(out.numpy(), src.numpy().T)
        g3 = (5 * 128 * 400, 0, (5, 400, 128), (128 * 400, 1, 400))      # batch dim in front, p = 400
        assert run_binary(thc, oracle, "cmul", [contiguous_geometry((5, 400, 128)), g3,
                                                contiguous_geometry((5, 400, 128))], rng) == "tiled"
        gp = (40 * 24 * 520, 0, (520, 24, 40), (1, 520, 520 * 24))       # permute(3,2,1): q fuses two dims
        assert run_binary(thc, oracle, "cadd", [contiguous_geometry((520, 24, 40)), gp,
                                                contiguous_geometry((520, 24, 40))], rng) == "tiled-fused"
    finally:
        thc.set_tuning("apply.tiled.group_p_vec", -1)
        thc.set_tuning("apply.skinny", 1)


@pytest.mark.parametrize("kind", ["float", "int"])
def test_addcmul_when_self_is_a_factor(thc, oracle, kind):
    """addcmul(self, t, v, src1, src2) with self being src1 (or src2) and not t:
    the reference first copies t into self and then accumulates in place
    (generic/THCTensorMathPointwise.cu:586-590), so the factor that is self
    already holds t's values: self = t + v * t * src2."""
    rng = np.random.default_rng(17)
    dtype = np.float32 if kind == "float" else np.int32
    t = rng.integers(-6, 7, (33, 65)).astype(dtype)
    a = rng.integers(-6, 7, (33, 65)).astype(dtype)
    b = rng.integers(-6, 7, (33, 65)).astype(dtype)
    for which in ("src1", "src2"):
        dt, da, db = thc.Tensor.from_numpy(t), thc.Tensor.from_numpy(a), thc.Tensor.from_numpy(b)
        if which == "src1":
            da.addcmul(dt, 2, da, db)
            got, want = da.numpy(), t + 2 * t * b
        else:
            db.addcmul(dt, 2, da, db)
            got, want = db.numpy(), t + 2 * a * t
        assert_bit_equal(got, want.astype(dtype), which)
        # a view on self's storage counts as well (here: self transposed twice)
        dt, da, db = thc.Tensor.from_numpy(t), thc.Tensor.from_numpy(a), thc.Tensor.from_numpy(b)
        alias = da.t().t()
        da.addcdiv(dt, 3, alias, thc.Tensor.from_numpy(np.ones_like(t)))
        assert_bit_equal(da.numpy(), (t + 3 * t).astype(dtype), "aliasing view")
    # self == t stays the one-pass in-place form
    dt, da, db = thc.Tensor.from_numpy(t), thc.Tensor.from_numpy(a), thc.Tensor.from_numpy(b)
    dt.addcmul(dt, 2, da, db)
    assert_bit_equal(dt.numpy(), (t + 2 * a * b).astype(dtype), "in place on t")


def test_streaming_store_variants_give_the_same_bits(thc, oracle):
    """Outputs of 64 MiB and more are stored with the streaming hint; the knobs
    force that policy onto small shapes so that every kernel's streaming-store
    form (flat, strided, flat + gathered, tiled, shifted-window, scans) is
    compared with the oracle as well."""
    rng = np.random.default_rng(31)
    knobs = ("apply.contig.nt_store", "apply.indexed.nt_store", "apply.tiled.nt_store", "scan.nt_store")
    for k in knobs:
        thc.set_tuning(k, 1)
    try:
        g = contiguous_geometry((100003,))
        assert run_binary(thc, oracle, "cadd", [g, g, g], rng) == "contig"
        gp = (64 * 200, 0, (64, 192), (200, 1))                      # padded rows, pack aligned
        assert run_binary(thc, oracle, "cmul", [gp, gp, contiguous_geometry((64, 192))], rng) == "strided"
        ga = (130 * 96, 0, (96, 130), (1, 96))                       # a:t(): rows not pack aligned everywhere
        assert run_binary(thc, oracle, "cadd1", [contiguous_geometry((96, 130)), ga, contiguous_geometry((96, 130))],
                          rng).startswith("tiled")
        ga = (128 * 256, 0, (256, 128), (1, 256))
        assert run_binary(thc, oracle, "cdiv", [contiguous_geometry((256, 128)), ga, contiguous_geometry((256, 128))],
                          rng) == "tiled"
        go = (333 * 515 + 1, 1, (333, 515), (1, 333))
        assert run_binary(thc, oracle, "cadd", [contiguous_geometry((333, 515)), go, contiguous_geometry((333, 515))],
                          rng) == "tiled-ragged"
        x = rng.integers(-8, 9, (333, 515)).astype(np.float32)
        bias = rng.integers(-8, 9, 515).astype(np.float32)
        db = thc.Tensor.from_numpy(bias).view_as_strided(0, (333, 515), (0, 1))
        out = thc.Tensor("float").cadd(thc.Tensor.from_numpy(x), 1.0, db)
        assert thc.last_kernel() == "flat-gather"
        assert_bit_equal(out.numpy(), x + bias)
        for shape, dim, kernel in (((1200, 3000), 1, "scan-rows"), ((64, 40, 512), 1, "scan-cols")):
            xi = rng.integers(-9, 10, shape).astype(np.float32)
            got = thc.Tensor("float").cumsum(thc.Tensor.from_numpy(xi), dim)
            assert thc.last_kernel() == kernel, thc.last_kernel()
            assert_bit_equal(got.numpy(), np.cumsum(xi.astype(np.int64), axis=dim).astype(np.float32))
    finally:
        for k in knobs:
            thc.set_tuning(k, -1)
