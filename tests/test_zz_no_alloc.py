"""THCudaTensor_sumallNoAlloc: the whole-tensor sum for callers that cannot
allocate (its partials live in a fixed device array). It must give exactly
what THCudaTensor_sumall gives, call after call, whatever the previous call
left in the shared array; and it must refuse what it cannot serve without a
temporary."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _bits(x):
    return np.array([x], np.float32).view(np.uint32)[0]


def _no_alloc(thc, t, res):
    res.fill(-123.0)                      # a stale result cannot pass for a new one
    t.sumall_no_alloc(res)
    thc.synchronize()
    return res.numpy()[0]


def test_two_calls_in_a_row_match_sumall(thc):
    rng = np.random.default_rng(77)
    res = thc.Tensor("float").resize((1,))
    big = rng.uniform(-1, 1, (1 << 24) + 4099).astype(np.float32)   # 512 workgroups + a ragged tail
    small = rng.uniform(-1, 1, 70001).astype(np.float32)            # 9 workgroups: fewer partials than before
    tb, ts = thc.Tensor.from_numpy(big), thc.Tensor.from_numpy(small)
    got_b = _no_alloc(thc, tb, res)
    got_s = _no_alloc(thc, ts, res)
    assert thc.last_kernel() == "all-noalloc"
    want_b, want_s = tb.sumall(), ts.sumall()
    assert _bits(got_b) == _bits(want_b), (got_b, want_b)
    assert _bits(got_s) == _bits(want_s), (got_s, want_s)
    # and against the mathematics: 1e-5 relative to the mass of the summands
    for got, x in ((got_b, big), (got_s, small)):
        ref = float(np.sum(x, dtype=np.float64))
        assert abs(got - ref) <= 1e-5 * max(abs(ref), float(np.abs(x).sum()) / 64)
    # again, big after small, on integer-valued data every order sums exactly
    ints = rng.integers(-8, 9, (1 << 22) + 3).astype(np.float32)
    ti = thc.Tensor.from_numpy(ints)
    assert _no_alloc(thc, ti, res) == float(ints.astype(np.float64).sum())


def test_shapes_offsets_and_empty(thc):
    rng = np.random.default_rng(78)
    res = thc.Tensor("float").resize((1,))
    x = rng.standard_normal((37, 129, 11)).astype(np.float32)
    t = thc.Tensor.from_numpy(x)
    assert _bits(_no_alloc(thc, t, res)) == _bits(t.sumall())
    flat = thc.Tensor.from_numpy(x.reshape(-1))
    odd = flat.narrow(0, 1, x.size - 2)                 # not 16-byte aligned: scalar loads
    assert _bits(_no_alloc(thc, odd, res)) == _bits(odd.sumall())
    one = flat.narrow(0, 5, 1)
    assert _no_alloc(thc, one, res) == x.reshape(-1)[5]
    assert _no_alloc(thc, thc.Tensor("float"), res) == 0.0   # empty tensor: the init value
    thc.force_64bit_index(True)
    try:
        assert _bits(_no_alloc(thc, t, res)) == _bits(t.sumall())
    finally:
        thc.force_64bit_index(False)


def test_rejects_what_needs_a_temporary_or_is_too_large(thc):
    res = thc.Tensor("float").resize((1,))
    res.fill(7.0)
    t = thc.Tensor.from_numpy(np.ones((8, 16), np.float32))
    with pytest.raises(thc.THCError, match="contiguous"):
        t.t().sumall_no_alloc(res)
    # a contiguous geometry of 2^32 + 65536 elements claimed over a small storage (the size field is
    # edited in place): refused before any launch
    huge = thc.Tensor("float").resize((2, 65536))
    huge.h.contents.size[0] = 65537
    try:
        with pytest.raises(thc.THCError, match="exceed the limit"):
            huge.sumall_no_alloc(res)
    finally:
        huge.h.contents.size[0] = 2
    with pytest.raises(thc.THCError, match="result"):
        thc.lib().THCudaTensor_sumallNoAlloc(thc.state(), t.h, C.c_void_p(0))
        thc._check()
    thc.synchronize()
    assert res.numpy()[0] == 7.0                      # nothing was launched


def test_does_not_allocate(thc):
    """Neither the caching allocator's pool nor the driver's free memory moves."""
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    t = thc.Tensor.from_numpy(np.arange(1 << 20, dtype=np.float32))
    res = thc.Tensor("float").resize((1,))
    t.sumall_no_alloc(res)
    thc.synchronize()
    f0, tot = C.c_size_t(0), C.c_size_t(0)
    assert hip.hipMemGetInfo(C.byref(f0), C.byref(tot)) == 0
    cached0 = thc.cached_memory()[0]
    for _ in range(10):
        t.sumall_no_alloc(res)
    thc.synchronize()
    f1 = C.c_size_t(0)
    assert hip.hipMemGetInfo(C.byref(f1), C.byref(tot)) == 0
    assert f1.value == f0.value and thc.cached_memory()[0] == cached0
    assert res.numpy()[0] == t.sumall()
