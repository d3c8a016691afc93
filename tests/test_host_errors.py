"""Error delivery of the C ABI, exercised on a machine without a GPU: the
library's exceptions must reach the TH handler (THCGeneral.c:714-726 routes
every CUDA error through THError) and the default handler must print and abort."""
import ctypes as C
import subprocess
import sys

import pytest

import cutorch_amd


def _gpu_present():
    try:
        hip = C.CDLL("libamdhip64.so")
        n = C.c_int(0)
        return hip.hipGetDeviceCount(C.byref(n)) == 0 and n.value > 0
    except OSError:
        return False


needs_no_gpu = pytest.mark.skipif(_gpu_present(), reason="checks the no-device error path")


@needs_no_gpu
def test_init_without_device_reports_through_handler():
    lib = cutorch_amd.lib()
    st = lib.THCState_alloc()
    lib.THCudaInit(C.c_void_p(st))
    msg = lib.THCAmd_lastError()
    assert msg and b"no HIP-capable device" in msg
    lib.THCAmd_clearLastError()
    assert lib.THCAmd_lastError() is None
    # an allocation on the uninitialised state fails cleanly as well
    lib.THCudaTensor_newWithSize1d.restype = C.c_void_p
    t = lib.THCudaTensor_newWithSize1d(C.c_void_p(st), 16)
    assert t is None and b"hip runtime error" in lib.THCAmd_lastError()
    lib.THCAmd_clearLastError()
    lib.THCState_free(C.c_void_p(st))


def test_argument_errors_carry_the_argument_number():
    lib = cutorch_amd.lib()
    seen = []
    cb = C.CFUNCTYPE(None, C.c_int, C.c_char_p, C.c_void_p)(lambda a, m, d: seen.append((a, m)))
    lib.THSetArgErrorHandler(cb, None)
    try:
        st = lib.THCState_alloc()
        t = lib.THCudaTensor_new(C.c_void_p(st))       # empty tensor: no device memory involved
        lib.THCudaTensor_size.restype = C.c_long
        lib.THCudaTensor_size.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        assert lib.THCudaTensor_size(st, t, 3) == 0
        assert seen == [(2, b"out of range")]
        lib.THCudaTensor_free(C.c_void_p(st), t)
        lib.THCState_free(C.c_void_p(st))
    finally:
        lib.THSetArgErrorHandler(cutorch_amd._err_cb[1], None)
        lib.THCAmd_clearLastError()


def test_empty_tensor_views_need_no_device():
    lib = cutorch_amd.lib()
    st = C.c_void_p(lib.THCState_alloc())
    t = lib.THCudaTensor_new(st)
    assert lib.THCudaTensor_nElement(st, t) == 0 and lib.THCudaTensor_isContiguous(st, t) == 1
    assert t.contents.nDimension == 0 and not t.contents.storage
    lib.THCudaTensor_free(st, t)
    lib.THCState_free(st)


def test_default_handler_prints_and_aborts():
    code = ("import ctypes as C, cutorch_amd; l=cutorch_amd.lib(); l.THSetErrorHandler(None,None);"
            "l.THSetArgErrorHandler(None,None); st=C.c_void_p(l.THCState_alloc()); t=l.THCudaTensor_new(st);"
            "l.THCudaTensor_size.argtypes=[C.c_void_p,C.c_void_p,C.c_int]; l.THCudaTensor_size(st,t,7)")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True,
                       cwd=cutorch_amd._HERE + "/..")
    assert r.returncode == -6, r                      # SIGABRT
    assert "THC error: invalid argument 2: out of range" in r.stderr
