"""Caching device allocator (role of lib/THC/THCCachingAllocator.cpp): freed
blocks are parked per stream and size class and handed out again, so resizes
and temporaries stop paying for hipMalloc/hipFree."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_blocks_are_reused_and_accounted(thc):
    lib, st = thc.lib(), thc.state()
    assert lib.THCState_isCachingAllocatorEnabled(st) == 1
    n = 3 * 1024 * 1024 + 17                      # 12 MiB + a bit: rounds up to 128 KiB granules
    a = thc.Tensor("float").resize((n,))
    p1 = a.data_ptr()
    free0, total, _ = thc.cached_memory()
    del a
    free1, _, largest = thc.cached_memory()
    rounded = -(-4 * n // (128 * 1024)) * 128 * 1024
    assert free1 == free0 + rounded and largest >= rounded and total > 0
    b = thc.Tensor("float").resize((n - 1000,))   # a little smaller: still served by the parked block
    assert b.data_ptr() == p1
    c = thc.Tensor("float").resize((n,))          # the block is taken: this one is fresh
    assert c.data_ptr() != p1
    # small sizes use 512-byte granules
    s1 = thc.Tensor("float").resize((100,))
    q = s1.data_ptr()
    del s1
    s2 = thc.Tensor("float").resize((128,))
    assert s2.data_ptr() == q


def test_results_are_unaffected_by_reuse(thc):
    rng = np.random.default_rng(5)
    for _ in range(5):                             # temporaries and outputs recycle the same blocks
        x = rng.standard_normal((257, 129)).astype(np.float32)
        t = thc.Tensor.from_numpy(x)
        out = thc.Tensor("float").cadd(t.t(), 1.0, thc.Tensor.from_numpy(x.T.copy()))
        assert np.array_equal(out.numpy(), x.T + x.T)
        assert np.array_equal(t.t().contiguous().numpy(), x.T)


def test_plain_allocator_can_be_selected(thc):
    lib = thc.lib()
    st = C.c_void_p(lib.THCState_alloc())
    lib.THCudaInit(st)
    assert lib.THCState_isCachingAllocatorEnabled(st) == 0
    lib.THCudaTensor_newWithSize1d.restype = C.POINTER(thc._Tensor)
    t = lib.THCudaTensor_newWithSize1d(st, 1000)
    assert t.contents.storage.contents.size == 1000
    lib.THCudaTensor_free(st, t)
    lib.THCudaShutdown(st)
    lib.THCState_free(st)


@pytest.fixture()
def nonblocking_streams(thc):
    """Two streams that do not synchronise with the default stream."""
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamCreateWithFlags.argtypes = [C.POINTER(C.c_void_p), C.c_uint]
    hip.hipStreamDestroy.argtypes = [C.c_void_p]
    hip.hipStreamSynchronize.argtypes = [C.c_void_p]
    made = []
    for _ in range(2):
        s = C.c_void_p()
        assert hip.hipStreamCreateWithFlags(C.byref(s), 1) == 0      # hipStreamNonBlocking, default priority
        made.append(s)
    yield hip, made
    for s in made:
        assert hip.hipStreamSynchronize(s) == 0
    thc.lib().THCState_setCurrentStream(thc.state(), None)
    thc.synchronize()
    for s in made:
        hip.hipStreamDestroy(s)


def _still_busy(hip, stream):
    """True while work queued on `stream` has not completed. An assertion about a block being held back
    is only meaningful while the other stream is still busy: the caller reads the quantity first and
    asserts only if the stream was still busy afterwards (on a fast GPU or a slow host the queue may
    have drained, and then nothing needs to be held back any more)."""
    hip.hipStreamQuery.argtypes = [C.c_void_p]
    busy = hip.hipStreamQuery(stream) != 0
    hip.hipGetLastError()                             # "not ready" is not an error to leave behind
    return busy


def _busy(thc, w, launches):
    """Queues `launches` passes over the 1 GiB tensor w on the current stream (a few ms of work)."""
    for _ in range(launches):
        w.add(w, 1.0)


def test_block_used_on_another_stream_is_held_back(thc, nonblocking_streams):
    """Allocated under stream A, read by work queued on stream B, freed: the block may not serve a new
    request on A (which would overwrite it at once) until B's work has completed."""
    hip, (sa, sb) = nonblocking_streams
    lib, st = thc.lib(), thc.state()
    lib.THCAmd_cachingAllocatorPendingBlocks.restype = C.c_size_t
    n = (1 << 24) + 12345
    lib.THCState_setCurrentStream(st, sa)
    x = thc.Tensor("float").resize((n,)).fill(1.0)
    px = x.data_ptr()
    assert hip.hipStreamSynchronize(sa) == 0
    lib.THCState_setCurrentStream(st, sb)
    w = thc.Tensor("float").resize((1 << 28,)).fill(0.0)
    r = thc.Tensor("float").resize((n,))
    _busy(thc, w, 40)                                  # stream B is busy for a while ...
    r.copy(x)                                          # ... and only then reads x
    del x                                              # freed while B's copy has not even started
    pending = lib.THCAmd_cachingAllocatorPendingBlocks()
    lib.THCState_setCurrentStream(st, sa)
    z = thc.Tensor("float").resize((n,))
    pz = z.data_ptr()
    if _still_busy(hip, sb):
        assert pending == 1 and pz != px               # not handed out while B may still read it
    z.fill(7.0)                                        # runs on A at once, concurrently with B
    assert hip.hipStreamSynchronize(sa) == 0 and hip.hipStreamSynchronize(sb) == 0
    assert np.all(r.numpy() == 1.0)
    assert lib.THCAmd_cachingAllocatorPendingBlocks() == 0
    z2 = thc.Tensor("float").resize((n,))             # B has caught up: the block is back in A's pool
    assert z2.data_ptr() == px
    assert w.narrow(0, 12345, 4).numpy().tolist() == [40.0] * 4


def test_record_stream_entry_point_and_resize_on_another_stream(thc, nonblocking_streams):
    hip, (sa, sb) = nonblocking_streams
    lib, st = thc.lib(), thc.state()
    lib.THCAmd_cachingAllocatorPendingBlocks.restype = C.c_size_t
    lib.THCCachingAllocator_recordStream.argtypes = [C.c_void_p, C.c_void_p]
    lib.THCState_setCurrentStream(st, sb)
    w = thc.Tensor("float").resize((1 << 28,)).fill(0.0)
    # a host that launches its own work on B reports the use itself
    lib.THCState_setCurrentStream(st, sa)
    y = thc.Tensor("float").resize((1 << 22,)).fill(2.0)
    py = y.data_ptr()
    lib.THCState_setCurrentStream(st, sb)
    _busy(thc, w, 20)
    lib.THCCachingAllocator_recordStream(C.c_void_p(py), sb)
    lib.THCState_setCurrentStream(st, sa)
    del y
    pending = lib.THCAmd_cachingAllocatorPendingBlocks()
    other = thc.Tensor("float").resize((1 << 22,))
    if _still_busy(hip, sb):
        assert pending == 1 and other.data_ptr() != py
    assert hip.hipStreamSynchronize(sb) == 0
    assert lib.THCAmd_cachingAllocatorPendingBlocks() == 0
    # resize on a stream other than the block's own: the old block is copied from on B, then freed
    lib.THCState_setCurrentStream(st, sa)
    t = thc.Tensor.from_numpy(np.arange(1 << 20, dtype=np.float32))
    pt = t.data_ptr()
    assert hip.hipStreamSynchronize(sa) == 0
    lib.THCState_setCurrentStream(st, sb)
    _busy(thc, w, 20)
    t.resize((1 << 21,))                               # storage grows: copy of the old contents queued on B
    assert t.data_ptr() != pt
    lib.THCState_setCurrentStream(st, sa)
    q = thc.Tensor("float").resize((1 << 20,))
    pq = q.data_ptr()
    if _still_busy(hip, sb):
        assert pq != pt                                # the source of B's pending copy is not recycled on A
    q.fill(-1.0)
    assert hip.hipStreamSynchronize(sa) == 0 and hip.hipStreamSynchronize(sb) == 0
    assert np.array_equal(t.numpy()[:1 << 20], np.arange(1 << 20, dtype=np.float32))


def test_no_alloc_entry_point_reports_its_input(thc, nonblocking_streams):
    """THCudaTensor_sumallNoAlloc launches on the current stream without waiting: an input allocated
    under stream A and summed on stream B must be held back when freed, like any other operand."""
    hip, (sa, sb) = nonblocking_streams
    lib, st = thc.lib(), thc.state()
    lib.THCAmd_cachingAllocatorPendingBlocks.restype = C.c_size_t
    n = (1 << 22) + 77
    lib.THCState_setCurrentStream(st, sa)
    x = thc.Tensor("float").resize((n,)).fill(0.5)
    px = x.data_ptr()
    assert hip.hipStreamSynchronize(sa) == 0
    lib.THCState_setCurrentStream(st, sb)
    w = thc.Tensor("float").resize((1 << 28,)).fill(0.0)
    res = thc.Tensor("float").resize((1,)).fill(0.0)
    _busy(thc, w, 30)
    x.sumall_no_alloc(res)                             # queued on B behind the busy work
    del x
    pending = lib.THCAmd_cachingAllocatorPendingBlocks()
    lib.THCState_setCurrentStream(st, sa)
    z = thc.Tensor("float").resize((n,))
    pz = z.data_ptr()
    if _still_busy(hip, sb):
        assert pending == 1 and pz != px
    z.fill(-3.0)                                       # would corrupt the sum if the block had been handed out
    assert hip.hipStreamSynchronize(sa) == 0 and hip.hipStreamSynchronize(sb) == 0
    assert res.numpy().tolist() == [0.5 * n]
    assert lib.THCAmd_cachingAllocatorPendingBlocks() == 0


def test_host_copy_waits_for_a_nonblocking_stream(thc, nonblocking_streams):
    """copyFromHost runs on the null stream; it must not overtake work queued on a non-blocking current stream."""
    hip, (sa, _) = nonblocking_streams
    lib, st = thc.lib(), thc.state()
    lib.THCState_setCurrentStream(st, sa)
    w = thc.Tensor("float").resize((1 << 28,)).fill(0.0)
    t = thc.Tensor("float").resize((1 << 20,)).fill(0.0)
    tv = thc.Tensor("float").resize((1024, 2048)).fill(0.0).t()     # a strided destination (staged through a temporary)
    _busy(thc, w, 20)
    t.add(t, 1.0)
    tv.add(tv, 1.0)
    fives = np.full(1 << 20, 5.0, np.float32)
    t._fn("copyFromHost")(t._st, t.h, fives.ctypes.data_as(C.c_void_p))
    tv._fn("copyFromHost")(tv._st, tv.h, np.full((2048, 1024), 5.0, np.float32).ctypes.data_as(C.c_void_p))
    assert hip.hipStreamSynchronize(sa) == 0
    assert np.all(t.numpy() == 5.0) and np.all(tv.numpy() == 5.0)
