"""Dense tensors of many shapes through every reduction / scan kernel family.

Which kernel serves a dense reduction depends on the lengths around the
reduced dim (short rows, small slices, tall narrow slices, aligned or not), so
this sweep draws shapes from a grid of awkward lengths and checks sum, max
(+index), min (+index), mean and cumsum against numpy on small-integer data,
where every partial sum is exact in the element type: results must match bit
for bit whatever order the kernel adds in."""
import numpy as np
import pytest

from tests.util import assert_bit_equal

pytestmark = pytest.mark.gpu

LENGTHS = [1, 2, 3, 4, 5, 7, 8, 10, 15, 16, 17, 31, 33, 64, 100, 127, 128, 130, 250, 257, 511, 1000, 1025, 4099]
SEEN = set()      # kernel families the sweep reached
DTYPES = {"float": np.float32, "half": np.float16, "int": np.int32, "double": np.float64, "byte": np.uint8,
          "long": np.int64}


def draw_shape(rng, budget=300000):
    nd = int(rng.integers(1, 4))
    while True:
        shape = tuple(int(rng.choice(LENGTHS)) for _ in range(nd))
        if np.prod(shape) <= budget:
            return shape


@pytest.mark.parametrize("seed", range(80))
def test_dense_shapes_against_numpy(thc, seed):
    rng = np.random.default_rng(9000 + seed)
    kind = ["float", "half", "int", "double", "byte", "long"][seed % 6]
    dtype = DTYPES[kind]
    shape = draw_shape(rng)
    if seed % 7 == 0:                      # one long dim next to short ones
        shape = (int(rng.choice([40000, 70001, 131072])),) + tuple(int(rng.choice([1, 3, 10, 16])) for _ in range(1))
        if seed % 14 == 0:
            shape = shape[::-1]
    n = int(np.prod(shape))
    # sparse small values: |running sums| stay below 2048 (exact in half) and 255 (byte)
    dense = rng.integers(0, 3, shape) if kind == "byte" else rng.integers(-2, 3, shape)
    keep = rng.random(shape) < min(1.0, (100.0 if kind == "byte" else 800.0) / max(shape))
    x = (dense * keep).astype(dtype)
    off = int(rng.integers(0, 4))
    storage = np.zeros(n + off, dtype)
    storage[off:] = x.reshape(-1)
    strides = [1] * len(shape)
    for d in range(len(shape) - 2, -1, -1):
        strides[d] = strides[d + 1] * shape[d + 1]
    dev = thc.Tensor.from_storage(storage, off, shape, tuple(strides), kind=kind)
    wide = x.astype(np.int64)
    for dim in range(len(shape)):
        what = "%s %s dim %d off %d" % (kind, shape, dim, off)
        out = thc.Tensor(kind).sum(dev, dim)
        k = thc.last_kernel()
        SEEN.add(k)
        assert_bit_equal(out.numpy(), wide.sum(axis=dim, keepdims=True).astype(dtype), what + " sum " + k)
        for which, arg, red in (("max", np.argmax, np.max), ("min", np.argmin, np.min)):
            vals, idx = thc.Tensor(kind), thc.Tensor("long")
            getattr(vals, which)(idx, dev, dim)
            k = thc.last_kernel()
            SEEN.add(k)
            assert_bit_equal(vals.numpy(), red(x, axis=dim, keepdims=True), what + " " + which + " " + k)
            assert np.array_equal(idx.numpy(), np.expand_dims(arg(x, axis=dim), dim) + 1), what + " arg" + which + " " + k
        out = thc.Tensor(kind).cumsum(dev, dim)
        k = thc.last_kernel()
        SEEN.add(k)
        assert_bit_equal(out.numpy(), np.cumsum(wide, axis=dim).astype(dtype), what + " cumsum " + k)
    assert_bit_equal(dev.storage_numpy(), storage)      # inputs untouched


def test_dense_shape_sweep_reached_every_kernel_family():
    if len(SEEN) == 0:
        pytest.skip("the sweep did not run in this process")
    want = {"rows", "rows-lds", "rows-index-lds", "slab", "slab-index", "cols", "cols-index",
            "scan-slab", "scan-chunked", "scan-rows", "scan-cols"}
    assert want <= SEEN, sorted(want - SEEN)


@pytest.mark.parametrize("kind", ["byte", "char", "short", "half", "int", "float", "long", "double"])
def test_transposed_copies_of_every_element_size_at_odd_shapes(thc, kind):
    """out:copy(a:t()) for 1-, 2-, 4- and 8-byte elements on shapes that leave no
    row 16-byte aligned (the shifted-window tiles) and with both tensors 1..3
    elements into their storages; the whole output storage is compared."""
    rng = np.random.default_rng(9100)
    dtype = {"char": np.int8, "short": np.int16}.get(kind) or DTYPES[kind]
    for rows, cols in ((61, 125), (333, 515), (130, 1001), (17, 9), (250, 64)):
        for off_in, off_out in ((0, 0), (1, 3), (2, 1)):
            n = rows * cols
            src = rng.integers(0, 100, n + off_in).astype(dtype)
            dst = np.full(n + off_out, 7, dtype)
            want = dst.copy()
            want[off_out:] = src[off_in:].reshape(cols, rows).T.reshape(-1)
            # (a dim short enough for the tall-and-skinny copy takes that kernel unless it is switched off)
            for skinny in (1, 0):
                a = thc.Tensor.from_storage(src, off_in, (rows, cols), (1, rows), kind=kind)     # a = b:t()
                out = thc.Tensor.from_storage(dst, off_out, (rows, cols), (cols, 1), kind=kind)
                thc.set_tuning("apply.skinny", skinny)
                try:
                    out.copy(a)
                finally:
                    thc.set_tuning("apply.skinny", 1)
                k = thc.last_kernel()
                assert k.startswith("tiled") or (skinny and k == "skinny"), (kind, rows, cols, k)
                assert_bit_equal(out.storage_numpy(), want, "%s %dx%d +%d/+%d %s" % (kind, rows, cols, off_in, off_out, k))


def test_reductions_and_scans_are_reproducible_run_to_run(thc):
    """No atomics, fixed fold orders: the same call on the same data returns
    the same bits, on every kernel family (split ones included)."""
    rng = np.random.default_rng(9200)
    for shape, dim in (((3, 1 << 18), 1), ((2, 8192, 96), 1), ((65536, 33), 1), ((4096, 8, 16), 1),
                       ((300001, 3), 0), ((8191, 513), 0), ((1024, 1024), 1), ((200000, 10), 0)):
        x = thc.Tensor.from_numpy(rng.standard_normal(shape).astype(np.float32))
        first = {}
        for rep in range(3):
            got = {"sum": thc.Tensor("float").sum(x, dim).numpy(), "norm": thc.Tensor("float").norm(x, 2.0, dim).numpy(),
                   "std": thc.Tensor("float").std(x, dim).numpy(), "cumsum": thc.Tensor("float").cumsum(x, dim).numpy(),
                   "sumall": np.float32(x.sumall()), "varall": np.float32(x.varall())}
            for k, v in got.items():
                if rep == 0:
                    first[k] = v
                else:
                    assert_bit_equal(np.asarray(v), np.asarray(first[k]), "%s %s rep %d" % (k, shape, rep))
