"""Copies between a dense (long x short) layout and its planar counterpart (the short dim selecting a
plane, the long dim at unit stride): tall-and-skinny transposes and NCHW <-> NHWC conversions with few
channels (lib/THC/THCTensorCopy.cu:26-122 runs them through the one strided apply). Bit-exact against
numpy on every element size, in both directions, with pack-aligned and unaligned sides, ragged last
tiles, batch dims, and the storage around the destination untouched."""
import numpy as np
import pytest

from tests.util import assert_bit_equal

KINDS = {"float": np.float32, "half": np.float16, "byte": np.uint8, "double": np.float64, "short": np.int16,
         "long": np.int64}


def values(rng, n, dtype):
    if np.dtype(dtype).kind == "f":
        return rng.integers(-1000, 1000, n).astype(dtype)
    info = np.iinfo(dtype)
    return rng.integers(max(info.min, -30000), min(info.max, 30000), n).astype(dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", sorted(KINDS))
def test_tall_skinny_transposes_both_directions(thc, kind):
    rng = np.random.default_rng(41)
    dtype = KINDS[kind]
    for long_n, short_n in ((100000, 3), (65536, 4), (70001, 5), (4099, 16), (30000, 31), (1000, 2), (64, 7)):
        if short_n * np.dtype(dtype).itemsize > 256:
            continue
        # (odd storage offsets: packs at element-aligned addresses; with the knob, the element-wise variants)
        thc.set_tuning("apply.skinny.aligned_packs_only", 1 if long_n in (70001, 4099) else 0)
        for off in (0, 1):
            planar = values(rng, short_n * long_n + off, dtype)
            src = thc.Tensor.from_storage(planar, off, (long_n, short_n), (1, long_n), kind=kind)     # (short, long):t()
            dst = thc.Tensor(kind).resize((long_n, short_n))
            dst.copy(src)
            assert thc.last_kernel() == "skinny", (kind, long_n, short_n, thc.last_kernel())
            want = planar[off:].reshape(short_n, long_n).T
            assert_bit_equal(dst.numpy(), np.ascontiguousarray(want), "%s gather %d x %d off %d" % (kind, long_n, short_n, off))
            # the other direction: dense rows scattered into planes, into the middle of a larger storage
            dense = values(rng, long_n * short_n + off, dtype)
            dsrc = thc.Tensor.from_storage(dense, off, (short_n, long_n), (1, short_n), kind=kind)    # (long, short):t()
            guard = values(rng, short_n * long_n + 2 * 5 + off, dtype)
            ddst = thc.Tensor.from_storage(guard, 5 + off, (short_n, long_n), (long_n, 1), kind=kind)
            ddst.copy(dsrc)
            assert thc.last_kernel() == "skinny", (kind, long_n, short_n, thc.last_kernel())
            want = dense[off:].reshape(long_n, short_n).T
            assert_bit_equal(ddst.numpy(), np.ascontiguousarray(want), "%s scatter %d x %d off %d" % (kind, long_n, short_n, off))
            after = ddst.storage_numpy()
            assert_bit_equal(after[:5 + off], guard[:5 + off])
            assert_bit_equal(after[5 + off + short_n * long_n:], guard[5 + off + short_n * long_n:])
    thc.set_tuning("apply.skinny.aligned_packs_only", 0)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["float", "half", "byte"])
def test_image_layout_conversions(thc, kind):
    """NCHW -> NHWC and back for 3, 4 and 16 channels: (h, w) collapse to one long dim, n stays a batch
    dim; a padded plane stride on the planar side; round trip returns the input."""
    rng = np.random.default_rng(42)
    dtype = KINDS[kind]
    for n, c, h, w, pad in ((5, 3, 37, 53, 0), (2, 4, 64, 64, 0), (3, 16, 20, 24, 0), (2, 3, 33, 40, 8)):
        plane = h * w + pad
        store = values(rng, n * c * plane, dtype)
        nchw = store.reshape(n, c, plane)[:, :, :h * w].reshape(n, c, h, w)
        src = thc.Tensor.from_storage(store, 0, (n, h, w, c), (c * plane, w, 1, plane), kind=kind)   # NHWC view of NCHW
        nhwc = thc.Tensor(kind).resize((n, h, w, c))
        nhwc.copy(src)
        assert thc.last_kernel() == "skinny", (kind, c, thc.last_kernel())
        assert_bit_equal(nhwc.numpy(), np.ascontiguousarray(nchw.transpose(0, 2, 3, 1)))
        back_view = nhwc.view_as_strided(0, (n, c, h, w), (h * w * c, 1, w * c, c))                    # NCHW view of NHWC
        back = thc.Tensor(kind).resize((n, c, h, w))
        back.copy(back_view)
        assert thc.last_kernel() == "skinny", (kind, c, thc.last_kernel())
        assert_bit_equal(back.numpy(), np.ascontiguousarray(nchw))


@pytest.mark.gpu
def test_skinny_copy_declines_what_it_does_not_cover(thc):
    rng = np.random.default_rng(43)
    x = rng.standard_normal((300, 200)).astype(np.float32)
    dst = thc.Tensor("float").resize((200, 300))
    dst.copy(thc.Tensor.from_numpy(x).t())                 # both dims long: the tiled kernel
    assert thc.last_kernel() != "skinny"
    assert_bit_equal(dst.numpy(), np.ascontiguousarray(x.T))
    thc.set_tuning("apply.skinny", 0)
    try:
        y = rng.standard_normal((3, 5000)).astype(np.float32)
        d2 = thc.Tensor("float").resize((5000, 3))
        d2.copy(thc.Tensor.from_numpy(y).t())
        assert thc.last_kernel() != "skinny"
        assert_bit_equal(d2.numpy(), np.ascontiguousarray(y.T))
    finally:
        thc.set_tuning("apply.skinny", 1)


@pytest.mark.gpu
@pytest.mark.parametrize("src_kind,dst_kind", [("byte", "float"), ("float", "byte"), ("byte", "half"), ("half", "byte"),
                                               ("half", "float"), ("float", "half"), ("float", "double"),
                                               ("double", "float")])
def test_converting_copies_between_image_layouts(thc, src_kind, dst_kind):
    """Type-converting copies of the same layouts (lib/THC/THCTensorCopy.cu:26-122 converts inside the
    apply): a byte HWC image into float CHW planes and back, tall-and-skinny transposes; values that
    every type involved represents exactly, so numpy's astype is the expected result bit for bit."""
    rng = np.random.default_rng(44)
    sdt, ddt = KINDS.get(src_kind, np.float32), KINDS.get(dst_kind, np.float32)
    for n, c, h, w in ((3, 3, 37, 53), (2, 4, 64, 64), (1, 16, 20, 24)):
        hwc = rng.integers(0, 200, (n, h, w, c)).astype(sdt)
        src = thc.Tensor.from_numpy(hwc)
        chw_view = src.view_as_strided(0, (n, c, h, w), (h * w * c, 1, w * c, c))       # NCHW view of the NHWC data
        out = thc.Tensor(dst_kind).resize((n, c, h, w))
        out.copy_from(chw_view)
        assert thc.last_kernel() == "skinny", (src_kind, dst_kind, thc.last_kernel())
        assert_bit_equal(out.numpy(), np.ascontiguousarray(hwc.transpose(0, 3, 1, 2)).astype(ddt))
        chw = rng.integers(0, 200, (n, c, h, w)).astype(sdt)
        src2 = thc.Tensor.from_numpy(chw)
        hwc_view = src2.view_as_strided(0, (n, h, w, c), (c * h * w, w, 1, h * w))       # NHWC view of the NCHW data
        out2 = thc.Tensor(dst_kind).resize((n, h, w, c))
        out2.copy_from(hwc_view)
        assert thc.last_kernel() == "skinny", (src_kind, dst_kind, thc.last_kernel())
        assert_bit_equal(out2.numpy(), np.ascontiguousarray(chw.transpose(0, 2, 3, 1)).astype(ddt))
    for long_n, short_n, off in ((70001, 3, 1), (4099, 5, 0)):
        planar = rng.integers(0, 200, short_n * long_n + off).astype(sdt)
        src = thc.Tensor.from_storage(planar, off, (long_n, short_n), (1, long_n), kind=src_kind)
        dst = thc.Tensor(dst_kind).resize((long_n, short_n))
        dst.copy_from(src)
        assert thc.last_kernel() == "skinny"
        assert_bit_equal(dst.numpy(), np.ascontiguousarray(planar[off:].reshape(short_n, long_n).T).astype(ddt))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", sorted(KINDS))
def test_batches_of_small_transposed_matrices(thc, kind):
    """(B, P, Q) <- (B, Q, P) transposed per matrix, P and Q below 64: tiles of whole matrices that are one
    contiguous run on both sides. Square and oblong matrices, batch counts off the tile size, an outer
    batch dim with padding between its rows, storage offsets off the 16-byte grid, whole destination
    storage compared."""
    rng = np.random.default_rng(45)
    dtype = KINDS[kind]
    for b, p, q in ((1000, 4, 4), (5003, 3, 3), (777, 8, 8), (300, 16, 16), (129, 32, 32), (65, 5, 7), (40, 63, 2), (2500, 2, 3)):
        thc.set_tuning("apply.skinny.aligned_packs_only", 1 if b in (5003, 300) else 0)
        for off_in, off_out in ((0, 0), (1, 3)):
            src = values(rng, b * p * q + off_in, dtype)
            dst = values(rng, b * p * q + off_out + 4, dtype)
            a = thc.Tensor.from_storage(src, off_in, (b, p, q), (p * q, 1, p), kind=kind)        # per-matrix transpose
            out = thc.Tensor.from_storage(dst, off_out, (b, p, q), (p * q, q, 1), kind=kind)
            out.copy(a)
            assert thc.last_kernel() == "small-transpose", (kind, b, p, q, thc.last_kernel())
            want = dst.copy()
            want[off_out:off_out + b * p * q] = src[off_in:].reshape(b, q, p).transpose(0, 2, 1).reshape(-1)
            assert_bit_equal(out.storage_numpy(), want, "%s %dx%dx%d +%d/+%d" % (kind, b, p, q, off_in, off_out))
    thc.set_tuning("apply.skinny.aligned_packs_only", 0)
    # an outer batch dim whose rows are padded on both sides
    o, b, p, q, pad_in, pad_out = 3, 50, 6, 5, 16, 32
    src = values(rng, o * (b * p * q + pad_in), dtype)
    dst = values(rng, o * (b * p * q + pad_out), dtype)
    a = thc.Tensor.from_storage(src, 0, (o, b, p, q), (b * p * q + pad_in, p * q, 1, p), kind=kind)
    out = thc.Tensor.from_storage(dst, 0, (o, b, p, q), (b * p * q + pad_out, p * q, q, 1), kind=kind)
    out.copy(a)
    assert thc.last_kernel() == "small-transpose"
    want = dst.copy().reshape(o, -1)
    want[:, :b * p * q] = src.reshape(o, -1)[:, :b * p * q].reshape(o, b, q, p).transpose(0, 1, 3, 2).reshape(o, -1)
    assert_bit_equal(out.storage_numpy(), want.reshape(-1))
    thc.set_tuning("apply.small_transpose", 0)
    try:
        x = values(rng, 200 * 4 * 4, dtype)
        out = thc.Tensor(kind).resize((200, 4, 4))
        out.copy(thc.Tensor.from_storage(x, 0, (200, 4, 4), (16, 1, 4), kind=kind))
        assert thc.last_kernel() != "small-transpose"
        assert_bit_equal(out.numpy(), x.reshape(200, 4, 4).transpose(0, 2, 1))
    finally:
        thc.set_tuning("apply.small_transpose", 1)
