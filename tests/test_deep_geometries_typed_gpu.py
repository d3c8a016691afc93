"""The deep-geometry generators of tests/test_deep_geometries_gpu.py (method of
cutorch's own suite, test/test.lua:81-175,543-727: 6 to 10 dims, holes on both
sides of the view, ten random transpositions, shapes re-factorised between
input and output) for the element types beyond float: half, byte, int, long
and double, for apply, same-type copy, type-converting copy and the
reductions with indices. Pointwise results, copies and conversions are
compared bit for bit over the WHOLE output storage; integer reductions bit for
bit, floating ones within the tolerance of their type."""
import numpy as np
import pytest

from tests.test_deep_geometries_gpu import deep_shape
from tests.util import assert_bit_equal, holed_geometry, refactorised_shape

pytestmark = pytest.mark.gpu

KINDS = ["half", "byte", "int", "long", "double"]
NP = {"half": np.float16, "byte": np.uint8, "int": np.int32, "long": np.int64, "double": np.float64,
      "float": np.float32, "short": np.int16, "char": np.int8}


def values(rng, kind, n, nonzero=False, lo=None, hi=None):
    dt = NP[kind]
    if kind in ("half", "double", "float"):
        a = rng.uniform(-4 if lo is None else lo, 4 if hi is None else hi, n).astype(dt)
        if nonzero:
            a[np.abs(a) < 0.25] = dt(1.5)
        return a
    info = np.iinfo(dt)
    a = rng.integers(max(info.min, -20000 if lo is None else lo), min(info.max, 20000 if hi is None else hi) + 1, n).astype(dt)
    if nonzero:
        a[(a == 0) | (a == np.array(-1, np.int64).astype(dt))] = 3
    return a


def mirror(thc, oracle, storage, geom, kind):
    return (thc.Tensor.from_storage(storage, geom[1], geom[2], geom[3], kind),
            oracle.View(storage.copy(), geom[1], geom[2], geom[3]))


OPS = ("cadd", "cmul", "cdiv", "addcmul", "add", "copy", "cmax", "lt")


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("seed", range(16))
def test_typed_apply_on_deep_holed_transposed_operands(thc, oracle, kind, seed):
    rng = np.random.default_rng(11000 + seed)
    shape = deep_shape(rng)
    op = OPS[seed % len(OPS)]
    nin = {"addcmul": 3, "add": 1, "copy": 1}.get(op, 2)
    geoms = [holed_geometry(rng, shape, holes=rng.random() < 0.7, swaps=10 if rng.random() < 0.7 else 0)
             for _ in range(nin + 1)]
    okind = "byte" if op == "lt" else kind
    sts = [values(rng, okind, geoms[0][0])] + [values(rng, kind, g[0], nonzero=(op == "cdiv")) for g in geoms[1:]]
    pairs = [mirror(thc, oracle, sts[0], geoms[0], okind)] + [mirror(thc, oracle, s, g, kind) for s, g in zip(sts[1:], geoms[1:])]
    dev, ref = [p[0] for p in pairs], [p[1] for p in pairs]
    fl = kind == "half"
    pw = oracle.pointwise if fl else oracle.typed_pointwise
    v = 3 if kind in ("byte", "int", "long") else 0.5
    thc.force_64bit_index(seed % 4 == 3)
    try:
        if op == "cadd":
            dev[0].cadd(dev[1], v, dev[2])
            pw("cadd", ref[0], ref[1], ref[2], value=v)
        elif op == "cmul":
            dev[0].cmul(dev[1], dev[2])
            pw("mul", ref[0], ref[1], ref[2])
        elif op == "cdiv":
            dev[0].cdiv(dev[1], dev[2])
            pw("div", ref[0], ref[1], ref[2])
        elif op == "addcmul":
            dev[0].addcmul(dev[1], v, dev[2], dev[3])
            pw("addcmul", ref[0], ref[1], ref[2], ref[3], value=v)
        elif op == "add":
            dev[0].add(dev[1], v)
            pw("addc", ref[0], ref[1], value=v)
        elif op == "copy":
            dev[0].copy(dev[1])
            pw("copy", ref[0], ref[1])
        elif op == "cmax":
            dev[0].binary("cmax", dev[1], dev[2])
            pw("fn:cmax", ref[0], ref[1], ref[2])
        else:
            dev[0].compare_tensor("lt", dev[1], dev[2])
            oracle.typed_compare("lt", ref[0], ref[1], ref[2])
    finally:
        thc.force_64bit_index(False)
    assert dev[0].shape == shape and dev[0].strides == geoms[0][3]
    assert_bit_equal(dev[0].storage_numpy(), ref[0].storage, "%s %s %s" % (kind, op, shape))


CONVERSIONS = [("float", "half"), ("half", "float"), ("float", "double"), ("double", "float"), ("int", "long"),
               ("long", "int"), ("float", "byte"), ("byte", "float"), ("double", "int"), ("short", "half"),
               ("half", "char"), ("long", "double")]


@pytest.mark.parametrize("pair", CONVERSIONS, ids=lambda p: "%s-to-%s" % p)
@pytest.mark.parametrize("seed", range(6))
def test_converting_copy_on_deep_and_refactorised_geometries(thc, oracle, pair, seed):
    """dst = (type) src with both sides deep, holed and transposed; on odd seeds the two shapes agree
    in element count only (elements pair by logical linear index, lib/THC/THCTensorCopy.cu:26-31)."""
    src, dst = pair
    rng = np.random.default_rng(12000 + seed)
    in_shape = deep_shape(rng, max_elems=80000)
    out_shape = refactorised_shape(rng, in_shape) if seed % 2 else in_shape
    gi = holed_geometry(rng, in_shape, holes=rng.random() < 0.6, swaps=10 if rng.random() < 0.7 else 0)
    go = holed_geometry(rng, out_shape, holes=rng.random() < 0.6, swaps=10 if rng.random() < 0.7 else 0)
    lim = {"byte": (0, 200), "char": (-100, 100)}.get(dst, (-1000, 1000))
    if src == "byte":
        lim = (0, 200)
    si = values(rng, src, gi[0], lo=lim[0], hi=lim[1])
    so = values(rng, dst, go[0])
    din, rin = mirror(thc, oracle, si, gi, src)
    dout, rout = mirror(thc, oracle, so, go, dst)
    thc.force_64bit_index(seed % 3 == 2)
    try:
        dout.copy_from(din)
    finally:
        thc.force_64bit_index(False)
    oracle.typed_convert(rout, rin)
    assert_bit_equal(dout.storage_numpy(), rout.storage, "%s -> %s %s -> %s" % (src, dst, in_shape, out_shape))


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("seed", range(8))
def test_typed_reductions_on_deep_holed_transposed_inputs(thc, oracle, kind, seed):
    rng = np.random.default_rng(13000 + seed)
    shape = deep_shape(rng, max_elems=60000)
    geom = holed_geometry(rng, shape, holes=rng.random() < 0.7, swaps=10 if rng.random() < 0.7 else 0)
    # small values with many ties: max/min must return the lowest index among equals
    st = values(rng, kind, geom[0], lo=-3, hi=3) if kind not in ("half", "double") else np.round(values(rng, kind, geom[0]))
    dev, ref = mirror(thc, oracle, st, geom, kind)
    for dim in sorted(set(int(d) for d in rng.integers(0, len(shape), 3))):
        out = thc.Tensor(kind).sum(dev, dim)
        if kind == "half":
            want = oracle.reduce_dim("sum", ref, dim).numpy().astype(np.float64)
            mass = np.abs(ref.numpy().astype(np.float64)).sum(axis=dim, keepdims=True)
            assert np.all(np.abs(out.numpy().astype(np.float64) - want) <= 2e-3 * np.maximum(np.abs(want), mass / 64)), (dim, shape)
        elif kind == "double":
            want = oracle.typed_reduce_dim("sum", ref, dim).numpy()
            mass = np.abs(ref.numpy()).sum(axis=dim, keepdims=True)
            assert np.all(np.abs(out.numpy() - want) <= 1e-13 * np.maximum(mass, 1e-300)), (dim, shape)
        else:
            assert_bit_equal(out.numpy(), oracle.typed_reduce_dim("sum", ref, dim).numpy(), "sum dim %d %s" % (dim, shape))
        which = "max" if (seed + dim) % 2 else "min"
        v, i = thc.Tensor(kind), thc.Tensor("long")
        getattr(v, which)(i, dev, dim)
        if kind == "half":
            rv, ri = oracle.minmax_dim(which, ref, dim)
        else:
            rv, ri = oracle.typed_minmax_dim(which, ref, dim)
        assert_bit_equal(v.numpy(), rv.numpy(), "%s %s values dim %d %s" % (kind, which, dim, shape))
        assert np.array_equal(i.numpy(), ri.numpy()), (kind, which, "indices", dim, shape)
    if kind in ("byte", "int", "long"):
        assert dev.sumall() == oracle.typed_reduce_all("sum", ref)
        assert dev.maxall() == oracle.typed_reduce_all("max", ref)
