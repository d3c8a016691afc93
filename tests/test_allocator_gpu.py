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
