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


def holed_geometry(rng, shape, holes=True, swaps=10, inflate=(4, 15)):
    """(storage_len, offset, size, stride) of a view with the logical `shape`,
    built the way cutorch's suite builds its hardest operands
    (createHoledTensorWithSizes + randomlyTranspose, test/test.lua:81-98,647-661):
    a dense allocation in which up to three dims are inflated by 4..15 elements,
    narrowed back to size at a random start (holes on both sides of the view),
    seen through `swaps` random transpositions. The transpositions are applied
    to the allocation's dim order so that the view comes out with `shape`."""
    nd = len(shape)
    perm = list(range(nd))                      # perm[k] = logical dim stored at allocation position k
    for _ in range(swaps):
        a, b = int(rng.integers(0, nd)), int(rng.integers(0, nd))
        perm[a], perm[b] = perm[b], perm[a]
    alloc = [int(shape[d]) for d in perm]
    start = [0] * nd
    if holes:
        for _ in range(3):
            k = int(rng.integers(0, nd))
            alloc[k] += int(rng.integers(inflate[0], inflate[1] + 1))
        for k in range(nd):
            start[k] = int(rng.integers(0, alloc[k] - int(shape[perm[k]]) + 1))
    astride, run = [0] * nd, 1
    for k in reversed(range(nd)):
        astride[k] = run
        run *= alloc[k]
    offset = sum(s * st for s, st in zip(start, astride))
    stride = [0] * nd
    for k, d in enumerate(perm):
        stride[d] = astride[k]
    return run, offset, tuple(int(s) for s in shape), tuple(stride)


def refactorised_shape(rng, shape, moves=10):
    """A shape with the same element count: `moves` times a prime factor of a
    random dim becomes a new dim or is multiplied into another dim
    (constructOutput of copyRandomizedTest, test/test.lua:584-622)."""
    out = [int(s) for s in shape]
    for _ in range(moves):
        d = int(rng.integers(0, len(out)))
        n, f, factors = out[d], 2, []
        while n > 1:
            while n % f == 0:
                factors.append(f)
                n //= f
            f += 1
        if not factors:
            continue
        f = factors[int(rng.integers(0, len(factors)))]
        out[d] //= f
        if rng.random() < 0.5 and len(out) < 25:
            out.insert(int(rng.integers(0, len(out) + 1)), f)
        else:
            out[int(rng.integers(0, len(out)))] *= f
    return tuple(out)
