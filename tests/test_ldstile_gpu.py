"""The general LDS-tile kernel of the apply engine: every op family and element
type with a transposed input and / or a transposed output, on shapes that are
whole aligned packs and on shapes that are not (odd sizes, odd pitches, views
at odd offsets), holes on both sides of every view.

The reference runs every type and op through its one strided apply
(lib/THC/THCApply.cuh:426-640); the method is that of its copyRandomizedTest
(test/test.lua:543-727): the whole storage is compared, so untouched elements
must stay untouched. Everything here is compared bit for bit with the oracle
(transcendental functions within the stated ulp bound)."""
import numpy as np
import pytest

from tests.util import assert_bit_equal

INT_KINDS = ["byte", "char", "short", "int", "long"]
ALL_KINDS = INT_KINDS + ["double", "float", "half"]


def storage_of(rng, oracle, kind, n, small=False, nonzero=False):
    dt = oracle.NP_OF[kind]
    if kind in ("double", "float", "half"):
        a = rng.uniform(-4, 4, n).astype(dt)
        if nonzero:
            a[a == 0] = dt(1.5)
        return a
    info = np.iinfo(dt)
    if small:
        a = rng.integers(0, 6, n).astype(dt)
    else:
        a = rng.integers(max(info.min, -30000), min(info.max, 30000) + 1, n).astype(dt)
    if nonzero:
        a[(a == 0) | (a == np.array(-1, np.int64).astype(dt))] = 3
    return a


def geometry(shape, order, pad, offset):
    """(storage_len, offset, size, stride): dims nest in memory as `order` says
    (last entry = unit stride), every dim but the unit-stride one padded by
    pad[d] elements of its run (holes), the view starting `offset` elements in."""
    nd = len(shape)
    stride, run = [0] * nd, 1
    for j, d in enumerate(reversed(order)):
        stride[d] = run
        run = run * shape[d] + (pad[d] if j < nd - 1 else 0)
    return run + offset + 3, offset, tuple(shape), tuple(stride)


def pair(thc, oracle, st, geom, kind):
    return thc.Tensor.from_storage(st, *geom[1:], kind=kind), oracle.View(st.copy(), *geom[1:])


# (shape, aligned): aligned shapes are multiples of 16 in every size, pitch and offset, so that
# they are whole packs for every element type; the others are odd everywhere
SHAPES_2D = [((208, 144), True), ((64, 512), True), ((48, 1040), True), ((201, 137), False), ((300, 701), False),
             ((1031, 67), False), ((9, 8), False)]


def operand_geoms(rng, shape, aligned, transposed):
    """Geometries of output, a, b, c for `shape`; `transposed` names the operands (0 = output)
    whose unit-stride dim is dim 0 instead of the last one."""
    nd = len(shape)
    geoms = []
    for k in range(4):
        order = list(range(nd))
        if k in transposed:
            order = order[::-1]
        step = 16 if aligned else 1
        pad = [int(rng.integers(0, 3)) * step + (0 if aligned else int(rng.integers(0, 2))) for _ in range(nd)]
        offset = int(rng.integers(0, 3)) * step + (0 if aligned else int(rng.integers(0, 4)))
        geoms.append(geometry(shape, order, pad, offset))
    return geoms


def expect_kernel(thc, shape, aligned, kind=None):
    k = thc.last_kernel()
    assert k.startswith("lds-tile") or k.startswith("tiled"), (k, shape, kind)
    if min(shape[0], shape[-1]) >= 8 and not aligned:
        assert k in ("lds-tile-shift", "tiled-shift", "tiled-ragged", "tiled-scalar"), (k, shape, kind)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ALL_KINDS)
def test_two_input_ops_with_transposed_operands(thc, oracle, kind):
    rng = np.random.default_rng(301)
    ops = ["add", "mul", "div", "fn:cmax", "fn:cmin"] + (["fn:cbitxor", "fn:cremainder"] if kind in INT_KINDS else [])
    names = {"add": "cadd", "mul": "cmul", "div": "cdiv"}
    for (shape, aligned) in SHAPES_2D:
        for transposed in ((1,), (2,), (1, 2), (0,), (0, 1)):
            op = ops[int(rng.integers(0, len(ops)))]
            go, ga, gb, _ = operand_geoms(rng, shape, aligned, transposed)
            da, ra = pair(thc, oracle, storage_of(rng, oracle, kind, ga[0]), ga, kind)
            db, rb = pair(thc, oracle, storage_of(rng, oracle, kind, gb[0], nonzero=op in ("div", "fn:cremainder")), gb, kind)
            do, ro = pair(thc, oracle, storage_of(rng, oracle, kind, go[0]), go, kind)
            name = names.get(op, op.replace("fn:", ""))
            if name == "cadd":
                do.cadd(da, 1, db)
            else:
                do.binary(name, da, db)
            expect_kernel(thc, shape, aligned, kind)
            if kind in ("float", "half"):
                oracle.pointwise(op, ro, ra, rb, value=1.0)
            else:
                oracle.typed_pointwise(op, ro, ra, rb, value=1)
            assert_bit_equal(do.storage_numpy(), ro.storage, "%s %s %s t=%s" % (kind, op, shape, transposed))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ALL_KINDS)
def test_one_and_three_input_ops_with_transposed_operands(thc, oracle, kind):
    rng = np.random.default_rng(302)
    for (shape, aligned) in SHAPES_2D:
        for transposed in ((1,), (0,), (1, 3), (0, 2)):
            go, ga, gb, gc = operand_geoms(rng, shape, aligned, transposed)
            da, ra = pair(thc, oracle, storage_of(rng, oracle, kind, ga[0]), ga, kind)
            db, rb = pair(thc, oracle, storage_of(rng, oracle, kind, gb[0]), gb, kind)
            dc, rc = pair(thc, oracle, storage_of(rng, oracle, kind, gc[0], nonzero=True), gc, kind)
            do, ro = pair(thc, oracle, storage_of(rng, oracle, kind, go[0]), go, kind)
            fl = kind in ("float", "half")
            ref = oracle.pointwise if fl else oracle.typed_pointwise
            # one input: abs (the math family) and a scalar op
            if kind != "byte":
                do.unary("abs", da)
                ref("fn:abs", ro, ra)
                assert_bit_equal(do.storage_numpy(), ro.storage, "%s abs %s t=%s" % (kind, shape, transposed))
            do.mul(da, 3)
            ref("mulc", ro, ra, value=3)
            assert_bit_equal(do.storage_numpy(), ro.storage, "%s mulc %s t=%s" % (kind, shape, transposed))
            # three inputs
            if 3 in transposed or 2 in transposed:
                do.addcdiv(da, 2, db, dc)
                ref("addcdiv", ro, ra, rb, rc, value=2)
                assert_bit_equal(do.storage_numpy(), ro.storage, "%s addcdiv %s t=%s" % (kind, shape, transposed))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ALL_KINDS)
def test_odd_shapes_with_inputs_on_the_outputs_pack_grid(thc, oracle, kind):
    """The common case of an odd shape: the output and the inputs that are not transposed are dense
    tensors of one shape, pitch and base alignment, so their rows start equally far from 16-byte
    boundaries (the kernel then reads those inputs from LDS pack by pack). Also mixed: a third input
    of another pitch and offset, a transposed output whose dense input shares its grid, and the same
    ops with the fast path switched off."""
    rng = np.random.default_rng(308)
    fl = kind in ("float", "half")
    ref = oracle.pointwise if fl else oracle.typed_pointwise
    for same_grid in (1, 0):
        thc.set_tuning("apply.ldstile.same_grid", same_grid)
        try:
            for shape in ((201, 137), (300, 701), (77, 1003), (9, 8)):
                for offset in (0, 3):
                    dense = geometry(shape, [0, 1], [0, 0], offset)
                    dense_t = geometry(shape, [1, 0], [0, 0], offset)
                    other = geometry(shape, [0, 1], [5, 0], offset + 1)
                    for go, ga, gb, gc in ((dense, dense_t, dense, dense), (dense, dense_t, dense, other),
                                           (dense_t, dense, dense_t, dense_t)):
                        da, ra = pair(thc, oracle, storage_of(rng, oracle, kind, ga[0]), ga, kind)
                        db, rb = pair(thc, oracle, storage_of(rng, oracle, kind, gb[0]), gb, kind)
                        dc, rc = pair(thc, oracle, storage_of(rng, oracle, kind, gc[0]), gc, kind)
                        do, ro = pair(thc, oracle, storage_of(rng, oracle, kind, go[0]), go, kind)
                        do.binary("cmax", da, db)
                        assert thc.last_kernel().startswith("lds-tile"), thc.last_kernel()
                        ref("fn:cmax", ro, ra, rb)
                        assert_bit_equal(do.storage_numpy(), ro.storage, "%s cmax %s off %d grid %d" % (kind, shape, offset, same_grid))
                        if kind not in ("float", "half"):       # (their addcmul runs on the specialised tiled kernels)
                            do.addcmul(dc, 2, da, db)
                            assert thc.last_kernel().startswith("lds-tile"), thc.last_kernel()
                            ref("addcmul", ro, rc, ra, rb, value=2)
                            assert_bit_equal(do.storage_numpy(), ro.storage, "%s addcmul %s off %d grid %d" % (kind, shape, offset, same_grid))
        finally:
            thc.set_tuning("apply.ldstile.same_grid", 1)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ALL_KINDS)
def test_comparisons_with_transposed_operands(thc, oracle, kind):
    rng = np.random.default_rng(303)
    cmps = ["lt", "gt", "le", "ge", "eq", "ne"]
    for (shape, aligned) in SHAPES_2D:
        for transposed, same_type in (((1,), False), ((2,), True), ((0,), False), ((0, 2), True), ((1, 2), False)):
            cmp = cmps[int(rng.integers(0, 6))]
            go, ga, gb, _ = operand_geoms(rng, shape, aligned, transposed)
            okind = kind if same_type else "byte"
            da, ra = pair(thc, oracle, storage_of(rng, oracle, kind, ga[0], small=kind in INT_KINDS), ga, kind)
            db, rb = pair(thc, oracle, storage_of(rng, oracle, kind, gb[0], small=kind in INT_KINDS), gb, kind)
            do, ro = pair(thc, oracle, storage_of(rng, oracle, okind, go[0]), go, okind)
            do.compare_tensor(cmp, da, db, same_type=same_type)
            oracle.typed_compare(cmp, ro, ra, rb)
            assert_bit_equal(do.storage_numpy(), ro.storage, "%s %s tensor %s t=%s" % (kind, cmp, shape, transposed))
            if 1 in transposed or 0 in transposed:
                do.compare_value(cmp, da, 2, same_type=same_type)
                expect_kernel(thc, shape, aligned, kind)
                oracle.typed_compare(cmp, ro, ra, value=2)
                assert_bit_equal(do.storage_numpy(), ro.storage, "%s %s value %s t=%s" % (kind, cmp, shape, transposed))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["half", "float", "double"])
def test_transcendental_family_with_transposed_operands(thc, oracle, kind):
    """exp / log / tanh (one input) and atan2 / cpow (two inputs): the device's libm against the
    host's, 4 ulp of the element type (half results are rounded from fp32: 1 ulp)."""
    rng = np.random.default_rng(304)
    dt = oracle.NP_OF[kind]
    eps = {"half": 2.0 ** -10, "float": 2.0 ** -23, "double": 2.0 ** -52}[kind]
    ref = oracle.typed_pointwise if kind == "double" else oracle.pointwise
    for (shape, aligned) in SHAPES_2D[:5]:
        for transposed in ((1,), (0,), (1, 2)):
            go, ga, gb, _ = operand_geoms(rng, shape, aligned, transposed)
            sa = (np.abs(rng.uniform(0.1, 3, ga[0]))).astype(dt)
            da, ra = pair(thc, oracle, sa, ga, kind)
            db, rb = pair(thc, oracle, rng.uniform(-2, 2, gb[0]).astype(dt), gb, kind)
            do, ro = pair(thc, oracle, np.zeros(go[0], dt), go, kind)
            for fn in ("exp", "log", "tanh"):
                do.unary(fn, da)
                ref("fn:" + fn, ro, ra)
                got, want = do.storage_numpy().astype(np.float64), ro.storage.astype(np.float64)
                assert np.all(np.abs(got - want) <= 4 * eps * np.maximum(np.abs(want), 1e-30)), (kind, fn, shape)
            for fn in ("atan2", "cpow"):
                do.binary(fn, da, db)
                expect_kernel(thc, shape, aligned, kind)
                ref("fn:" + fn, ro, ra, rb)
                got, want = do.storage_numpy().astype(np.float64), ro.storage.astype(np.float64)
                assert np.all(np.abs(got - want) <= 4 * eps * np.maximum(np.abs(want), 1e-30)), (kind, fn, shape)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["short", "half", "double", "byte"])
def test_permuted_3d_operands_and_batch_dims(thc, oracle, kind):
    """Tiles inside a batch: 3-D operands whose permutations differ, with holes."""
    rng = np.random.default_rng(305)
    fl = kind in ("float", "half")
    ref = oracle.pointwise if fl else oracle.typed_pointwise
    for shape in ((6, 80, 96), (5, 71, 93), (40, 3, 150)):
        aligned = shape[1] % 16 == 0
        for orders in (((0, 1, 2), (2, 1, 0), (0, 1, 2)), ((0, 1, 2), (0, 2, 1), (0, 1, 2)), ((1, 0, 2), (0, 2, 1), (2, 0, 1)),
                       ((2, 1, 0), (0, 1, 2), (0, 1, 2))):
            geoms = []
            for order in orders:
                step = 16 if aligned else 1
                pad = [int(rng.integers(0, 2)) * step for _ in range(3)]
                geoms.append(geometry(shape, list(order), pad, int(rng.integers(0, 2)) * step))
            go, ga, gb = geoms
            da, ra = pair(thc, oracle, storage_of(rng, oracle, kind, ga[0]), ga, kind)
            db, rb = pair(thc, oracle, storage_of(rng, oracle, kind, gb[0]), gb, kind)
            do, ro = pair(thc, oracle, storage_of(rng, oracle, kind, go[0]), go, kind)
            do.binary("cmax", da, db)
            ref("fn:cmax", ro, ra, rb)
            assert_bit_equal(do.storage_numpy(), ro.storage, "%s cmax %s %s" % (kind, shape, orders))
            m, rm = pair(thc, oracle, np.zeros(go[0], np.uint8), go, "byte")
            m.compare_tensor("le", da, db)
            oracle.typed_compare("le", rm, ra, rb)
            assert_bit_equal(m.storage_numpy(), rm.storage, "%s le %s %s" % (kind, shape, orders))


@pytest.mark.gpu
def test_many_tiles_bands_and_capped_grid(thc, oracle):
    """More tiles than the persistent grid holds (every workgroup walks several tiles with the next
    tile's loads in flight), ragged last band, grid capped to one workgroup per CU and to one in all."""
    rng = np.random.default_rng(306)
    for kind, shape in (("short", (1100, 2100)), ("int", (2500, 1300)), ("half", (777, 3001))):
        aligned = False
        go, ga, gb, _ = operand_geoms(rng, shape, aligned, (1,))
        da, ra = pair(thc, oracle, storage_of(rng, oracle, kind, ga[0]), ga, kind)
        db, rb = pair(thc, oracle, storage_of(rng, oracle, kind, gb[0], nonzero=True), gb, kind)
        want = None
        for cap in (8, 1, 0):
            do, ro = pair(thc, oracle, storage_of(rng, oracle, kind, go[0]), go, kind)
            if cap == 0:
                thc.set_tuning("apply.ldstile.max_grid", 3)
            else:
                thc.set_tuning("apply.ldstile.max_per_cu", cap)
            try:
                do.binary("cmin", da, db)
                assert thc.last_kernel().startswith("lds-tile"), thc.last_kernel()
            finally:
                thc.set_tuning("apply.ldstile.max_per_cu", 8)
                thc.set_tuning("apply.ldstile.max_grid", -1)
            if want is None:
                ref = oracle.pointwise if kind == "half" else oracle.typed_pointwise
                ref("fn:cmin", ro, ra, rb)
                want = ro
            got = do.numpy()
            assert_bit_equal(got, want.numpy(), "%s cmin %s cap %d" % (kind, shape, cap))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["short", "half", "int", "float", "double", "byte"])
def test_streamed_store_form_gives_the_same_bits(thc, oracle, kind):
    """Large outputs leave the kernel as nontemporal stores; the knob forces that form onto small aligned
    and odd shapes, with transposed inputs and with a transposed output."""
    rng = np.random.default_rng(307)
    thc.set_tuning("apply.tiled.nt_store", 1)
    try:
        for (shape, aligned) in (((208, 144), True), ((201, 137), False), ((300, 701), False), ((64, 512), True)):
            for transposed in ((1,), (0,), (1, 2)):
                go, ga, gb, _ = operand_geoms(rng, shape, aligned, transposed)
                da, ra = pair(thc, oracle, storage_of(rng, oracle, kind, ga[0]), ga, kind)
                db, rb = pair(thc, oracle, storage_of(rng, oracle, kind, gb[0]), gb, kind)
                do, ro = pair(thc, oracle, storage_of(rng, oracle, kind, go[0]), go, kind)
                do.binary("cmax", da, db)
                assert thc.last_kernel().startswith("lds-tile"), thc.last_kernel()
                if kind in ("float", "half"):
                    oracle.pointwise("fn:cmax", ro, ra, rb)
                else:
                    oracle.typed_pointwise("fn:cmax", ro, ra, rb)
                assert_bit_equal(do.storage_numpy(), ro.storage, "%s %s t=%s" % (kind, shape, transposed))
    finally:
        thc.set_tuning("apply.tiled.nt_store", -1)


def conv_values(rng, oracle, src, dst, n):
    """Source values that convert to `dst` without leaving its range (out-of-range float -> integer
    conversions are undefined in C)."""
    sdt = oracle.NP_OF[src]
    if src in ("double", "float", "half"):
        lim = {"byte": (0, 200), "char": (-100, 100)}.get(dst, (-1000, 1000))
        return rng.uniform(lim[0], lim[1], n).astype(sdt)
    info = np.iinfo(sdt)
    lo, hi = max(info.min, -30000), min(info.max, 30000)
    if dst == "half":
        lo, hi = max(lo, -2000), min(hi, 2000)
    return rng.integers(lo, hi + 1, n).astype(sdt)


@pytest.mark.gpu
@pytest.mark.parametrize("src", ALL_KINDS)
def test_converting_copies_of_transposed_and_strided_operands(thc, oracle, src):
    """dst = (type) src in one pass for every pair of element types: transposed source, transposed
    destination, both strided alike (holes), aligned and odd shapes, whole destination storage compared
    (lib/THC/THCTensorCopy.cu:26-122, method of test/test.lua:700-727)."""
    rng = np.random.default_rng(307)
    for dst in ALL_KINDS:
        if dst == src:
            continue
        for (shape, aligned) in (((208, 144), True), ((201, 137), False), ((40, 1100), False), ((64, 512), True)):
            for transposed in ((1,), (0,), ()):
                go, gs, _, _ = operand_geoms(rng, shape, aligned, transposed)
                ds, rs = pair(thc, oracle, conv_values(rng, oracle, src, dst, gs[0]), gs, src)
                dd, rd = pair(thc, oracle, storage_of(rng, oracle, dst, go[0]), go, dst)
                dd.copy_from(ds)
                k = thc.last_kernel()
                if transposed:      # (a short dim of at most 256 bytes: the tall-and-skinny copy, for some pairs)
                    assert k.startswith("lds-tile") or k == "skinny", (k, src, dst, shape)
                else:
                    assert k.startswith("strided") or k in ("convert", "contig", "contig-scalar"), (k, src, dst, shape)
                oracle.typed_convert(rd, rs)
                assert_bit_equal(dd.storage_numpy(), rd.storage, "%s -> %s %s t=%s" % (src, dst, shape, transposed))


@pytest.mark.gpu
def test_converting_copy_between_different_shapes_and_overlapping_destination(thc, oracle):
    rng = np.random.default_rng(308)
    x = rng.uniform(-100, 100, (12, 35)).astype(np.float32)
    d = thc.Tensor.from_numpy(x)
    out = thc.Tensor("int").resize((5, 84))           # same element count, different shape
    out.copy_from(d.t())
    assert_bit_equal(out.numpy().reshape(-1), x.T.reshape(-1).astype(np.int32))
    # a destination that addresses elements twice (through a dense temporary): every element ends up
    # with one of the values written to it, which one is not defined; the rest of the storage stays
    st = np.zeros(40, np.float64)
    dst = thc.Tensor.from_storage(st, 0, (6, 10), (5, 1), kind="double")
    src = thc.Tensor.from_numpy(np.arange(60, dtype=np.int16).reshape(6, 10))
    dst.copy_from(src)
    got = dst.storage_numpy()
    cand = [set() for _ in range(40)]
    for i in range(6):
        for j in range(10):
            cand[5 * i + j].add(float(10 * i + j))
    for o in range(40):
        assert got[o] in (cand[o] or {0.0}), (o, got[o], cand[o])
