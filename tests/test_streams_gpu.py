"""The engine launches on the caller's current stream (thread-local, as
THCState_getCurrentStream / setStream in lib/THC/THCGeneral.c:516-546) and
keeps its scratch per stream (THCGeneral.c:677-712)."""
import ctypes as C
import threading

import numpy as np
import pytest

from tests.util import assert_bit_equal

pytestmark = pytest.mark.gpu


@pytest.fixture()
def streams(thc):
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
    hip.hipStreamDestroy.argtypes = [C.c_void_p]
    hip.hipStreamSynchronize.argtypes = [C.c_void_p]
    made = []
    for _ in range(2):
        s = C.c_void_p()
        assert hip.hipStreamCreate(C.byref(s)) == 0          # default priority
        made.append(s)
    yield hip, made
    thc.lib().THCState_setCurrentStream(thc.state(), None)
    thc.synchronize()
    for s in made:
        hip.hipStreamDestroy(s)


def test_ops_follow_the_current_stream(thc, oracle, streams):
    hip, (s1, s2) = streams
    lib, st = thc.lib(), thc.state()
    rng = np.random.default_rng(61)
    a = rng.standard_normal((512, 384)).astype(np.float32)
    b = rng.standard_normal((384, 512)).astype(np.float32)
    big = rng.integers(-8, 9, (3, 1 << 18)).astype(np.float32)      # split reduction: uses the stream's scratch
    da, db, dbig = thc.Tensor.from_numpy(a), thc.Tensor.from_numpy(b), thc.Tensor.from_numpy(big)
    thc.synchronize()
    want_mul = a * b.T
    want_sum = big.astype(np.int64).sum(axis=1, keepdims=True).astype(np.float32)
    for stream in (s1, s2, None, s1):
        lib.THCState_setCurrentStream(st, stream)
        assert lib.THCState_getCurrentStream(st) == (stream.value if stream else None)
        out = thc.Tensor("float").cmul(da, db.t())
        sums = thc.Tensor("float").sum(dbig, 1)
        assert thc.last_kernel() == "rows-split"
        total = dbig.sumall()                                        # waits on the current stream itself
        assert total == float(big.astype(np.int64).sum())
        if stream:
            assert hip.hipStreamSynchronize(stream) == 0
        else:
            thc.synchronize()
        assert_bit_equal(out.numpy(), want_mul)
        assert_bit_equal(sums.numpy(), want_sum)


def test_current_stream_is_per_thread(thc, streams):
    hip, (s1, _) = streams
    lib, st = thc.lib(), thc.state()
    lib.THCState_setCurrentStream(st, s1)
    seen = {}

    def worker():
        seen["stream"] = lib.THCState_getCurrentStream(st)           # a fresh thread starts on the default stream
        x = thc.Tensor.from_numpy(np.arange(1000, dtype=np.float32))
        seen["sum"] = x.sumall()

    t = threading.Thread(target=worker)
    t.start()
    t.join()
    assert seen["stream"] is None and seen["sum"] == 499500.0
    assert lib.THCState_getCurrentStream(st) == s1.value


def test_concurrent_host_threads_on_their_own_streams(thc, streams):
    """Four host threads, each on its own stream (two created here, two more
    below), run pointwise ops, split and chunked reductions and scans, *all reductions
    and temporaries (caching allocator) at the same time; every result must be
    exact."""
    hip, (s1, s2) = streams
    lib, st = thc.lib(), thc.state()
    extra = []
    for _ in range(2):
        s = C.c_void_p()
        assert hip.hipStreamCreate(C.byref(s)) == 0
        extra.append(s)
    errors = []

    def worker(idx, stream):
        try:
            lib.THCState_setCurrentStream(st, stream)
            rng = np.random.default_rng(700 + idx)
            for it in range(25):
                a = rng.integers(-8, 9, (64, 333)).astype(np.float32)
                b = rng.integers(-8, 9, (333, 64)).astype(np.float32)
                big = rng.integers(-4, 5, (2, 1 << 17)).astype(np.float32)
                da, db, dbig = thc.Tensor.from_numpy(a), thc.Tensor.from_numpy(b), thc.Tensor.from_numpy(big)
                out = thc.Tensor("float").addcmul(da, 2.0, da, db.t())       # tiled kernel
                sums = thc.Tensor("float").sum(dbig, 1)                        # split reduction (stream scratch)
                mx, ix = thc.Tensor("float"), thc.Tensor("long")
                mx.max(ix, out, 1)
                total = dbig.sumall()                                          # blocks on this stream only
                cont = db.t().contiguous()                                     # temporary through the allocator
                tall = rng.integers(-2, 3, (40000, 3)).astype(np.float32)      # chunked kernels: partials and carries
                dtall = thc.Tensor.from_numpy(tall)                            # live in this stream's scratch
                colsum = thc.Tensor("float").sum(dtall, 0)
                assert thc.last_kernel() == "tall-flat"
                run = thc.Tensor("float").cumsum(dtall, 0)
                assert thc.last_kernel() == "scan-chunked"
                var = dtall.varall()
                assert np.array_equal(colsum.numpy().ravel(), tall.astype(np.int64).sum(axis=0).astype(np.float32))
                assert np.array_equal(run.numpy(), np.cumsum(tall.astype(np.int64), axis=0).astype(np.float32))
                assert abs(var - tall.astype(np.float64).var(ddof=1)) <= 1e-5 * var, (idx, it, "varall")
                want = a + 2.0 * (a * b.T)
                assert np.array_equal(out.numpy(), want), (idx, it, "addcmul")
                assert np.array_equal(sums.numpy().ravel(), big.astype(np.int64).sum(axis=1).astype(np.float32))
                assert total == float(big.astype(np.int64).sum()), (idx, it, "sumall")
                assert np.array_equal(ix.numpy().ravel(), want.argmax(axis=1) + 1), (idx, it, "argmax")
                assert np.array_equal(cont.numpy(), b.T)
        except Exception as e:                                                  # noqa: BLE001
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(i, s)) for i, s in enumerate([s1, s2] + extra)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    thc.synchronize()
    for s in extra:
        hip.hipStreamDestroy(s)
    assert not errors, errors


def test_async_copies_between_pinned_host_memory_and_a_stream(thc, streams):
    """copyAsyncFromHost / copyAsyncToHost (the raw-pointer forms of copyAsyncCPU / copyAsyncCuda,
    generic/THCTensorCopy.c:104-164): queued on the current stream in order with the kernels around
    them, no host wait; contiguity and size are argument errors as in the reference."""
    hip, (s1, _) = streams
    lib, st = thc.lib(), thc.state()
    hip.hipHostMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t, C.c_uint]
    hip.hipHostFree.argtypes = [C.c_void_p]
    n = (1 << 20) + 3
    src, dst = C.c_void_p(), C.c_void_p()
    assert hip.hipHostMalloc(C.byref(src), 4 * n, 0) == 0 and hip.hipHostMalloc(C.byref(dst), 4 * n, 0) == 0
    try:
        hsrc = np.ctypeslib.as_array(C.cast(src, C.POINTER(C.c_float)), (n,))
        hdst = np.ctypeslib.as_array(C.cast(dst, C.POINTER(C.c_float)), (n,))
        rng = np.random.default_rng(63)
        hsrc[:] = rng.standard_normal(n).astype(np.float32)
        hdst[:] = -1.0
        lib.THCState_setCurrentStream(st, s1)
        t = thc.Tensor("float").resize((n,))
        t.copy_async_from_host(src.value, n)             # H2D, then a kernel, then D2H: one stream, in order
        t.mul(t, 2.0)
        t.copy_async_to_host(dst.value, n)
        assert hip.hipStreamSynchronize(s1) == 0
        assert_bit_equal(hdst, hsrc * np.float32(2.0))
        with pytest.raises(thc.THCError, match="sizes do not match"):
            t.copy_async_from_host(src.value, n - 1)
        m = thc.Tensor("float").resize((64, 32))
        with pytest.raises(thc.THCError, match="Target tensor must be contiguous"):
            m.t().copy_async_from_host(src.value, 64 * 32)
        with pytest.raises(thc.THCError, match="Source tensor must be contiguous"):
            m.t().copy_async_to_host(dst.value, 64 * 32)
        thc.Tensor("float").copy_async_from_host(src.value, 0)      # empty: nothing to do
    finally:
        lib.THCState_setCurrentStream(st, None)
        thc.synchronize()
        hip.hipHostFree(src)
        hip.hipHostFree(dst)
