"""Strided operands the way cutorch's own suite builds its hardest ones
(test/test.lua:81-175,543-727): 6 to 10 dims, holes on both sides of the view
(inflate + narrow), ten random transpositions, shapes re-factorised between
input and output, up to the 25-dim limit of THCTensorInfo.cuh:10-16 (26 must
raise). Apply, copy and reductions are compared with the CPU oracle through
the C ABI; pointwise results and copies bit for bit over the WHOLE output
storage, whose holes are NaN-filled beforehand."""
import numpy as np
import pytest

from tests.test_reduce_gpu import REDUCERS, dev_and_ref, run_reduce
from tests.util import assert_bit_equal, fill_storage, holed_geometry, refactorised_shape

pytestmark = pytest.mark.gpu


def deep_shape(rng, lo=6, hi=10, max_elems=150000):
    nd = int(rng.integers(lo, hi + 1))
    while True:
        shape = tuple(int(x) for x in rng.integers(1, 6, nd))
        if 1 < int(np.prod(shape)) <= max_elems:
            return shape


def mirror(thc, oracle, storage, geom, kind="float"):
    return (thc.Tensor.from_storage(storage, geom[1], geom[2], geom[3], kind),
            oracle.View(storage.copy(), geom[1], geom[2], geom[3]))


OPS = ("cadd", "cmul", "cdiv", "addcmul", "add", "copy")


def run_op(op, dev, ref, oracle):
    if op == "cadd":
        dev[0].cadd(dev[1], 0.37, dev[2])
        oracle.pointwise("cadd", ref[0], ref[1], ref[2], value=0.37)
    elif op == "cmul":
        dev[0].cmul(dev[1], dev[2])
        oracle.pointwise("mul", ref[0], ref[1], ref[2])
    elif op == "cdiv":
        dev[0].cdiv(dev[1], dev[2])
        oracle.pointwise("div", ref[0], ref[1], ref[2])
    elif op == "addcmul":
        dev[0].addcmul(dev[1], -1.5, dev[2], dev[3])
        oracle.pointwise("addcmul", ref[0], ref[1], ref[2], ref[3], value=-1.5)
    elif op == "add":
        dev[0].add(dev[1], 2.25)
        oracle.pointwise("addc", ref[0], ref[1], value=2.25)
    else:
        dev[0].copy(dev[1])
        oracle.pointwise("copy", ref[0], ref[1])


@pytest.mark.parametrize("seed", range(36))
def test_apply_on_deep_holed_transposed_operands(thc, oracle, seed):
    rng = np.random.default_rng(9000 + seed)
    shape = deep_shape(rng)
    op = OPS[seed % len(OPS)]
    nin = {"addcmul": 3, "add": 1, "copy": 1}.get(op, 2)
    geoms = [holed_geometry(rng, shape, holes=rng.random() < 0.7, swaps=10 if rng.random() < 0.7 else 0)
             for _ in range(nin + 1)]
    sts = [fill_storage(rng, g[0], np.float32, "normal") for g in geoms]
    sts[0][:] = np.nan
    pairs = [mirror(thc, oracle, s, g) for s, g in zip(sts, geoms)]
    dev, ref = [p[0] for p in pairs], [p[1] for p in pairs]
    thc.force_64bit_index(seed % 4 == 3)
    try:
        run_op(op, dev, ref, oracle)
    finally:
        thc.force_64bit_index(False)
    assert dev[0].shape == shape and dev[0].strides == geoms[0][3]      # the view itself is untouched
    assert_bit_equal(dev[0].storage_numpy(), ref[0].storage, "%s %s" % (op, shape))


@pytest.mark.parametrize("seed", range(30))
def test_copy_and_apply_between_refactorised_shapes(thc, oracle, seed):
    """Input and output agree in element count only (elements pair by logical
    linear index, THCApply.cuh:434-439): up to 10 dims of up to 25 each on one
    side, prime factors moved between dims or into new dims on the other."""
    rng = np.random.default_rng(9500 + seed)
    nd = int(rng.integers(1, 11))
    while True:
        in_shape = tuple(int(x) for x in rng.integers(1, 26, nd))
        if int(np.prod(in_shape)) <= 200000:
            break
    out_shape = refactorised_shape(rng, in_shape)
    assert int(np.prod(out_shape)) == int(np.prod(in_shape))
    gi = holed_geometry(rng, in_shape, holes=rng.random() < 0.5, swaps=10 if rng.random() < 0.5 else 0)
    go = holed_geometry(rng, out_shape, holes=rng.random() < 0.5, swaps=10 if rng.random() < 0.5 else 0)
    si = np.full(gi[0], -150.0, np.float32)
    so = np.full(go[0], np.nan, np.float32)
    din, rin = mirror(thc, oracle, si, gi)
    lin = np.arange(1, int(np.prod(in_shape)) + 1, dtype=np.float32).reshape(in_shape)
    din.copy(thc.Tensor.from_numpy(lin))                     # 1..n in logical order, holes keep -150
    oracle.pointwise("copy", rin, oracle.View.of(lin))
    assert_bit_equal(din.storage_numpy(), rin.storage, "fill of the input view")
    dout, rout = mirror(thc, oracle, so, go)
    dout.copy(din)
    oracle.pointwise("copy", rout, rin)
    assert_bit_equal(dout.storage_numpy(), rout.storage, "copy %s -> %s" % (in_shape, out_shape))
    assert_bit_equal(dout.numpy().reshape(-1), lin.reshape(-1), "logical order")
    dout.cadd(dout, 0.5, din)                                 # apply with mismatched shapes, in place
    oracle.pointwise("cadd", rout, rout, rin, value=0.5)
    assert_bit_equal(dout.storage_numpy(), rout.storage, "cadd %s += %s" % (out_shape, in_shape))


@pytest.mark.parametrize("seed", range(24))
def test_reductions_on_deep_holed_transposed_inputs(thc, oracle, seed):
    rng = np.random.default_rng(9800 + seed)
    shape = deep_shape(rng, max_elems=60000)
    geom = holed_geometry(rng, shape, holes=rng.random() < 0.7, swaps=10 if rng.random() < 0.7 else 0)
    dev, ref = dev_and_ref(thc, oracle, rng, geom)
    for dim in sorted(set(int(d) for d in rng.integers(0, len(shape), 3))):
        run_reduce(thc, oracle, REDUCERS[(seed + dim) % len(REDUCERS)][0], dev, ref, dim)
        v, i = thc.Tensor("float"), thc.Tensor("long")
        (v.max if (seed + dim) % 2 else v.min)(i, dev, dim)
        rv, ri = oracle.minmax_dim("max" if (seed + dim) % 2 else "min", ref, dim)
        assert_bit_equal(v.numpy(), rv.numpy(), "values dim %d %s" % (dim, shape))
        assert np.array_equal(i.numpy(), ri.numpy()), ("indices", dim, shape)
    got, want = dev.sumall(), oracle.reduce_all("sum", ref)
    assert abs(got - want) <= 1e-5 * max(abs(want), float(np.abs(ref.numpy()).sum()) / 64)


def test_25_dims_work_and_26_raise(thc, oracle):
    """THCTensorInfo.cuh:10-16: MAX_CUTORCH_DIMS = 25."""
    rng = np.random.default_rng(9999)
    shape = tuple([2] * 12 + [1] * 5 + [3, 2, 1, 2, 1, 1, 2, 1])           # 25 dims, 98304 elements
    assert len(shape) == 25
    ga = holed_geometry(rng, shape, holes=True, swaps=10)
    gb = holed_geometry(rng, shape, holes=False, swaps=10)
    go = holed_geometry(rng, shape, holes=True, swaps=0)
    sts = [fill_storage(rng, g[0], np.float32, "normal") for g in (go, ga, gb)]
    sts[0][:] = np.nan
    pairs = [mirror(thc, oracle, s, g) for s, g in zip(sts, (go, ga, gb))]
    dev, ref = [p[0] for p in pairs], [p[1] for p in pairs]
    dev[0].cmul(dev[1], dev[2])
    oracle.pointwise("mul", ref[0], ref[1], ref[2])
    assert_bit_equal(dev[0].storage_numpy(), ref[0].storage, "25-dim cmul")
    flat = thc.Tensor("float").resize((int(np.prod(shape)),))
    flat.copy(dev[1])
    assert_bit_equal(flat.numpy(), ref[1].numpy().reshape(-1), "25-dim copy")
    for dim in (0, 12, 17, 24):
        run_reduce(thc, oracle, "sum", dev[1], ref[1], dim)
        v, i = thc.Tensor("float"), thc.Tensor("long")
        v.max(i, dev[1], dim)
        rv, ri = oracle.minmax_dim("max", ref[1], dim)
        assert_bit_equal(v.numpy(), rv.numpy(), "25-dim max")
        assert np.array_equal(i.numpy(), ri.numpy())
    got, want = dev[1].sumall(), oracle.reduce_all("sum", ref[1])
    assert abs(got - want) <= 1e-5 * float(np.abs(ref[1].numpy()).sum())
    # one dim more: every engine refuses with the reference's message
    shape26 = shape + (1,)
    x = thc.Tensor("float").resize(shape26)
    y = thc.Tensor("float").resize(shape26)
    for call in (lambda: thc.Tensor("float").cmul(x, y), lambda: thc.Tensor("float").sum(x, 3),
                 lambda: x.sumall(), lambda: thc.Tensor("float").max(thc.Tensor("long"), x, 3)):
        with pytest.raises(thc.THCError, match="too many"):
            call()
