"""Helpers shared by the parity tests: random strided geometries in the spirit
of cutorch's createHoledTensorWithSizes / copyRandomizedTest
(test/test.lua:81-175,543-727) and bitwise comparison of whole storages."""
import numpy as np


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[a.itemsize])


def assert_bit_equal(got, want, what=""):
    got, want = np.ascontiguousarray(got), np.ascontiguousarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    bad = np.flatnonzero(bits(got).reshape(-1) != bits(want).reshape(-1))
    if bad.size:
        i = int(bad[0])
        raise AssertionError("%s: %d of %d elements differ, first at %d: got %r want %r" % (
            what, bad.size, got.size, i, got.reshape(-1)[i], want.reshape(-1)[i]))


def random_geometry(rng, shape, holes=True, permute=True, max_offset=3):
    """(storage_len, offset, size, stride) of a non-overlapping view with the
    logical `shape`: dims laid out in a random memory order, optionally padded
    so that the view has holes."""
    nd = len(shape)
    order = list(rng.permutation(nd)) if permute else list(range(nd))
    padded = [int(s + (rng.integers(0, 3) if holes else 0)) for s in shape]
    stride = [0] * nd
    run = 1
    for d in reversed(order):          # last in `order` is innermost in memory
        stride[d] = run
        run *= padded[d]
    offset = int(rng.integers(0, max_offset + 1)) if max_offset else 0
    return run + offset, offset, tuple(int(s) for s in shape), tuple(stride)


def contiguous_geometry(shape):
    stride, run = [], 1
    for s in reversed(shape):
        stride.append(run)
        run *= int(s)
    return run, 0, tuple(int(s) for s in shape), tuple(reversed(stride))


def fill_storage(rng, n, dtype=np.float32, dist="normal"):
    if dist == "normal":
        a = rng.standard_normal(n)
    elif dist == "uniform":
        a = rng.uniform(-1.0, 1.0, n)
    else:
        a = rng.integers(-8, 9, n).astype(np.float64)
    return a.astype(dtype)


def rel_err_rows(got, want, scale):
    """max over outputs of |got-want| / scale (scale > 0 elementwise)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return float(np.max(np.abs(got - want) / scale)) if got.size else 0.0


def device_fill_from_block(thc, shape, block):
    """Device tensor of `shape` whose storage repeats the host array `block`
    (device-to-device copies): sets up multi-GB operands in seconds. The
    element at storage offset o is block[o % block.size]."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    t = thc.Tensor("float").resize(shape)
    n = int(np.prod(shape))
    blk = thc.Tensor.from_numpy(block)
    base, done = t.data_ptr(), 0
    while done < n:
        m = min(block.size, n - done)
        assert hip.hipMemcpy(base + 4 * done, blk.data_ptr(), 4 * m, 3) == 0
        done += m
    return t
