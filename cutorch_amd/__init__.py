"""ctypes binding of libTHC.so (the MI355X-native apply/reduce engine).

The library is the product; this module is the thin host-side mirror of the
Lua-visible interface (`torch.CudaTensor` methods add / cmul / sum / max ...,
TensorMath.lua:1510-1520,1562-1571,1810-1849,2179-2189) used by the tests
and the benchmark. Every method is one call into the C ABI declared in
include/THC.h; nothing here computes. Loading fails loudly if the library has
not been built (`python -m cutorch_amd.build`): there is no fallback path.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libTHC.so")

c_long_p = C.POINTER(C.c_long)


class _Storage(C.Structure):
    _fields_ = [("data", C.c_void_p), ("size", C.c_ssize_t), ("refcount", C.c_int),
                ("flag", C.c_char), ("allocator", C.c_void_p), ("allocatorContext", C.c_void_p),
                ("view", C.c_void_p), ("device", C.c_int)]


class _Tensor(C.Structure):
    _fields_ = [("size", c_long_p), ("stride", c_long_p), ("nDimension", C.c_int),
                ("storage", C.POINTER(_Storage)), ("storageOffset", C.c_ssize_t),
                ("refcount", C.c_int), ("flag", C.c_char)]


_lib = None
_state = None
_err_cb = None


class THCError(RuntimeError):
    pass


def lib():
    """The loaded libTHC.so (loads on first use)."""
    global _lib, _err_cb
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is missing: run `python -m cutorch_amd.build`" % LIB_PATH)
        _lib = C.CDLL(LIB_PATH)
        _declare(_lib)
        # Handlers that return: the failed entry point returns to us and the
        # message is picked up from THCAmd_lastError by _check().
        _err_cb = (C.CFUNCTYPE(None, C.c_char_p, C.c_void_p)(lambda m, d: None),
                   C.CFUNCTYPE(None, C.c_int, C.c_char_p, C.c_void_p)(lambda a, m, d: None))
        _lib.THSetErrorHandler(_err_cb[0], None)
        _lib.THSetArgErrorHandler(_err_cb[1], None)
    return _lib


def _check():
    msg = _lib.THCAmd_lastError()
    if msg:
        text = msg.decode()
        _lib.THCAmd_clearLastError()
        raise THCError(text)


def state():
    """The process-wide THCState (THCState_alloc + THCudaInit on first use)."""
    global _state
    if _state is None:
        l = lib()
        st = l.THCState_alloc()
        # as cutorch's init.c:1037-1042: caching allocator unless THC_CACHING_ALLOCATOR=0
        if os.environ.get("THC_CACHING_ALLOCATOR", "1") != "0":
            l.THCState_setDeviceAllocator(C.c_void_p(st), l.THCCachingAllocator_get())
        l.THCudaInit(st)
        _check()
        _state = st
    return _state


_TYPES = {
    "float": ("THCudaTensor", "THCudaStorage", C.c_float, np.float32),
    "half": ("THCudaHalfTensor", "THCudaHalfStorage", C.c_uint16, np.float16),
    "long": ("THCudaLongTensor", "THCudaLongStorage", C.c_long, np.int64),
    "byte": ("THCudaByteTensor", "THCudaByteStorage", C.c_ubyte, np.uint8),
    "char": ("THCudaCharTensor", "THCudaCharStorage", C.c_byte, np.int8),
    "short": ("THCudaShortTensor", "THCudaShortStorage", C.c_short, np.int16),
    "int": ("THCudaIntTensor", "THCudaIntStorage", C.c_int, np.int32),
    "double": ("THCudaDoubleTensor", "THCudaDoubleStorage", C.c_double, np.float64),
}
_COPY_SUFFIX = {"byte": "Byte", "char": "Char", "short": "Short", "int": "Int", "long": "Long",
                "float": "Float", "double": "Double", "half": "Half"}
_FLOAT_KINDS = ("float", "half")


def _declare(l):
    P = C.c_void_p
    l.THCState_alloc.restype = P
    l.THCCachingAllocator_get.restype = P
    l.THCState_setDeviceAllocator.argtypes = [P, P]
    l.THCState_isCachingAllocatorEnabled.argtypes = [P]
    l.THCudaMemGetInfoCached.argtypes = [P, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t),
                                         C.POINTER(C.c_size_t)]
    l.THCudaInit.argtypes = [P]
    l.THCudaShutdown.argtypes = [P]
    l.THCState_free.argtypes = [P]
    l.THCAmd_lastError.restype = C.c_char_p
    l.THCAmd_lastKernel.restype = C.c_char_p
    l.THCAmd_setTuning.argtypes = [C.c_char_p, C.c_long]
    l.THCAmd_getTuning.argtypes = [C.c_char_p]
    l.THCAmd_getTuning.restype = C.c_long
    l.THCAmd_getNumComputeUnits.argtypes = [P]
    l.THCState_getCurrentStream.argtypes = [P]
    l.THCState_getCurrentStream.restype = P
    l.THCState_setCurrentStream.argtypes = [P, P]
    l.THC_float2half.argtypes = [C.c_float]
    l.THC_float2half.restype = C.c_uint16
    l.THC_half2float.argtypes = [C.c_uint16]
    l.THC_half2float.restype = C.c_float
    l.THCAmd_collapseDims.argtypes = [C.c_int, c_long_p, c_long_p, C.c_int, c_long_p, c_long_p,
                                      C.POINTER(C.c_int)]
    l.THCAmd_overlappingIndices.argtypes = [C.c_int, c_long_p, c_long_p]
    l.THCAmd_canUse32BitIndexMath.argtypes = [C.c_int, c_long_p, c_long_p]
    l.THCAmd_indexToOffset.argtypes = [C.c_int, c_long_p, c_long_p, C.c_long]
    l.THCAmd_indexToOffset.restype = C.c_long
    l.THCAmd_jointCollapse.argtypes = [C.c_int, C.c_int, c_long_p, c_long_p, c_long_p, c_long_p]
    TP = C.POINTER(_Tensor)
    SP = C.POINTER(_Storage)
    for kind, (T, S, creal, _) in _TYPES.items():
        def f(name, res, *args):
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = list(args)
        f(S + "_newWithSize", SP, P, C.c_ssize_t)
        f(S + "_free", None, P, SP)
        f(S + "_copyFromHost", None, P, SP, P, C.c_ssize_t)
        f(S + "_copyToHost", None, P, P, SP, C.c_ssize_t)
        f(S + "_size", C.c_ssize_t, P, SP)
        f(T + "_new", TP, P)
        f(T + "_newWithSize1d", TP, P, C.c_long)
        f(T + "_newWithTensor", TP, P, TP)
        f(T + "_newContiguous", TP, P, TP)
        f(T + "_newClone", TP, P, TP)
        f(T + "_newTranspose", TP, P, TP, C.c_int, C.c_int)
        f(T + "_newNarrow", TP, P, TP, C.c_int, C.c_long, C.c_long)
        f(T + "_newSelect", TP, P, TP, C.c_int, C.c_long)
        f(T + "_resizeNd", None, P, TP, C.c_int, c_long_p, c_long_p)
        f(T + "_setStorageNd", None, P, TP, SP, C.c_ssize_t, C.c_int, c_long_p, c_long_p)
        f(T + "_free", None, P, TP)
        f(T + "_copy", None, P, TP, TP)
        f(T + "_copyFromHost", None, P, TP, P)
        f(T + "_copyToHost", None, P, P, TP)
        f(T + "_copyAsyncFromHost", None, P, TP, P, C.c_ssize_t)
        f(T + "_copyAsyncToHost", None, P, P, C.c_ssize_t, TP)
        f(T + "_isContiguous", C.c_int, P, TP)
        f(T + "_nElement", C.c_ssize_t, P, TP)
        f(T + "_data", P, P, TP)
        f(T + "_squeeze1d", None, P, TP, TP, C.c_int)
        for other in _TYPES:
            f(T + "_copyCuda" + _COPY_SUFFIX[other], None, P, TP, TP)
        for cmp in ("lt", "gt", "le", "ge", "eq", "ne"):
            f(T + "_" + cmp + "Value", None, P, TP, TP, creal)
            f(T + "_" + cmp + "ValueT", None, P, TP, TP, creal)
            f(T + "_" + cmp + "Tensor", None, P, TP, TP, TP)
            f(T + "_" + cmp + "TensorT", None, P, TP, TP, TP)

        def opt(name, res, *args):      # declared when the type has the entry point
            if hasattr(l, name):
                f(name, res, *args)
        LT = TP
        for name in ("add", "sub", "mul", "div", "pow", "cmaxValue", "cminValue", "fmod", "remainder",
                     "lshift", "rshift", "bitand", "bitor", "bitxor"):
            opt(T + "_" + name, None, P, TP, TP, creal)
        for name in ("cadd", "csub"):
            opt(T + "_" + name, None, P, TP, TP, creal, TP)
        for name in ("cmul", "cdiv", "cpow", "cmax", "cmin", "cfmod", "cremainder", "atan2", "clshift",
                     "crshift", "cbitand", "cbitor", "cbitxor"):
            opt(T + "_" + name, None, P, TP, TP, TP)
        for name in ("addcmul", "addcdiv"):
            opt(T + "_" + name, None, P, TP, TP, creal, TP, TP)
        for name in ("sigmoid", "log", "lgamma", "log1p", "exp", "cos", "acos", "cosh", "sin", "asin",
                     "sinh", "tan", "atan", "tanh", "sqrt", "rsqrt", "ceil", "floor", "round", "trunc",
                     "frac", "cinv", "neg", "abs", "sign"):
            opt(T + "_" + name, None, P, TP, TP)
        opt(T + "_clamp", None, P, TP, TP, creal, creal)
        opt(T + "_tpow", None, P, TP, creal, TP)
        opt(T + "_lerp", None, P, TP, TP, TP, creal)
        opt(T + "_equal", C.c_int, P, TP, TP)
        opt(T + "_fill", None, P, TP, creal)
        opt(T + "_zero", None, P, TP)
        acc = C.c_float if kind in _FLOAT_KINDS else (C.c_double if kind == "double" else C.c_long)
        for name in ("sum", "prod", "mean"):
            opt(T + "_" + name, None, P, TP, TP, C.c_long, C.c_int)
        opt(T + "_norm", None, P, TP, TP, creal, C.c_long, C.c_int)
        for name in ("max", "min"):
            opt(T + "_" + name, None, P, TP, LT, TP, C.c_long, C.c_int)
        for name in ("sumall", "prodall", "meanall"):
            opt(T + "_" + name, acc, P, TP)
        for name in ("cumsum", "cumprod"):
            opt(T + "_" + name, None, P, TP, TP, C.c_long)
        for name in ("var", "std"):
            opt(T + "_" + name, None, P, TP, TP, C.c_long, C.c_int, C.c_int)
        for name in ("varall", "stdall"):
            opt(T + "_" + name, acc, P, TP, C.c_int)
        opt(T + "_dist", acc, P, TP, TP, creal)
        opt(T + "_normall", acc, P, TP, creal)
        for name in ("minall", "maxall"):
            opt(T + "_" + name, creal, P, TP)
        opt(T + "_renorm", None, P, TP, TP, creal, C.c_long, creal)
    l.THCudaByteTensor_logicalall.argtypes = [P, TP]
    l.THCudaByteTensor_logicalany.argtypes = [P, TP]
    l.THCudaHalfTensor_copyCuda.argtypes = [P, TP, TP]
    l.THCudaTensor_sumallNoAlloc.argtypes = [P, TP, P]
    l.THCudaTensor_sumallNoAlloc.restype = None


def _longs(seq):
    return (C.c_long * max(1, len(seq)))(*seq)


def _half_bits(v):
    with np.errstate(over="ignore"):          # a scalar beyond half's range is +-inf, as in C
        return int(np.array(v, dtype=np.float16).view(np.uint16))


class Tensor(object):
    """A THCuda{,Half,Long}Tensor handle. `kind` is 'float', 'half' or 'long'."""

    def __init__(self, kind="float", handle=None):
        self.kind = kind
        self.T, self.S, self.creal, self.np_dtype = _TYPES[kind]
        self._st = state()
        self.h = handle if handle is not None else self._fn("new")(self._st)

    def _fn(self, name):
        return getattr(lib(), self.T + "_" + name)

    def _sfn(self, name):
        return getattr(lib(), self.S + "_" + name)

    def _real(self, v):
        return _half_bits(v) if self.kind == "half" else v

    def __del__(self):
        try:
            if self.h is not None and _lib is not None:
                self._fn("free")(self._st, self.h)
                self.h = None
        except Exception:
            pass

    # ----------------------------------------------------------- creation --
    @classmethod
    def from_numpy(cls, arr, kind=None):
        """Contiguous device tensor with the shape and values of `arr`."""
        arr = np.ascontiguousarray(arr)
        if kind is None:
            kind = {np.dtype(t[3]): k for k, t in _TYPES.items()}[arr.dtype]
        t = cls(kind)
        if arr.ndim > 0 and arr.size > 0:
            t.resize(arr.shape)
            t._fn("copyFromHost")(t._st, t.h, arr.ctypes.data_as(C.c_void_p))
            _check()
        return t

    @classmethod
    def from_storage(cls, storage, offset, size, stride, kind="float"):
        """Mirror a host storage array exactly (holes included) and view it
        through (offset, size, stride) -- cloneExactlyToGPU, test/test.lua:232-245."""
        t = cls(kind)
        storage = np.ascontiguousarray(storage, dtype=t.np_dtype)
        st = t._sfn("newWithSize")(t._st, storage.size)
        _check()
        t._sfn("copyFromHost")(t._st, st, storage.ctypes.data_as(C.c_void_p), storage.size)
        _check()
        t._fn("setStorageNd")(t._st, t.h, st, offset, len(size), _longs(size), _longs(stride))
        t._sfn("free")(t._st, st)
        _check()
        return t

    def resize(self, shape):
        self._fn("resizeNd")(self._st, self.h, len(shape), _longs(shape), None)
        _check()
        return self

    def _wrap(self, handle):
        _check()
        return Tensor(self.kind, handle)

    def t(self, d1=0, d2=1):
        return self._wrap(self._fn("newTranspose")(self._st, self.h, d1, d2))

    def narrow(self, dim, first, size):
        return self._wrap(self._fn("newNarrow")(self._st, self.h, dim, first, size))

    def select(self, dim, idx):
        return self._wrap(self._fn("newSelect")(self._st, self.h, dim, idx))

    def contiguous(self):
        return self._wrap(self._fn("newContiguous")(self._st, self.h))

    def clone(self):
        return self._wrap(self._fn("newClone")(self._st, self.h))

    def view_as_strided(self, offset, size, stride):
        """New tensor on the same storage with explicit geometry."""
        r = Tensor(self.kind)
        r._fn("setStorageNd")(self._st, r.h, self.h.contents.storage, offset, len(size),
                              _longs(size), _longs(stride))
        _check()
        return r

    # ---------------------------------------------------------- inspection --
    @property
    def shape(self):
        c = self.h.contents
        return tuple(c.size[i] for i in range(c.nDimension))

    @property
    def strides(self):
        c = self.h.contents
        return tuple(c.stride[i] for i in range(c.nDimension))

    @property
    def offset(self):
        return self.h.contents.storageOffset

    def numel(self):
        return self._fn("nElement")(self._st, self.h)

    def is_contiguous(self):
        return bool(self._fn("isContiguous")(self._st, self.h))

    def data_ptr(self):
        return self._fn("data")(self._st, self.h)

    def numpy(self):
        """Logical contents as a contiguous host array."""
        out = np.empty(self.shape, dtype=self.np_dtype)
        if out.size:
            self._fn("copyToHost")(self._st, out.ctypes.data_as(C.c_void_p), self.h)
            _check()
        return out

    def copy_async_from_host(self, host_ptr, n):
        """Queues host memory (n elements at host_ptr, ideally pinned) -> this contiguous tensor on the
        current stream; does not wait (copyAsyncCPU, generic/THCTensorCopy.c:104-132)."""
        self._fn("copyAsyncFromHost")(self._st, self.h, C.c_void_p(host_ptr), n)
        _check()
        return self

    def copy_async_to_host(self, host_ptr, n):
        """Queues this contiguous tensor -> host memory on the current stream; does not wait
        (copyAsyncCuda, generic/THCTensorCopy.c:134-164)."""
        self._fn("copyAsyncToHost")(self._st, C.c_void_p(host_ptr), n, self.h)
        _check()
        return self

    def storage_numpy(self):
        """The whole underlying storage (to check that holes stay untouched)."""
        st = self.h.contents.storage
        n = self._sfn("size")(self._st, st)
        out = np.empty(n, dtype=self.np_dtype)
        self._sfn("copyToHost")(self._st, out.ctypes.data_as(C.c_void_p), st, n)
        _check()
        return out

    # --------------------------------------------------------------- math --
    def _call(self, name, *args):
        self._fn(name)(self._st, *args)
        _check()
        return self

    def copy(self, src):
        return self._call("copy", self.h, src.h)

    def fill(self, v):
        return self._call("fill", self.h, self._real(v))

    def zero(self):
        return self._call("zero", self.h)

    def add(self, src, v):      # self = src + v
        return self._call("add", self.h, src.h, self._real(v))

    def sub(self, src, v):
        return self._call("sub", self.h, src.h, self._real(v))

    def mul(self, src, v):
        return self._call("mul", self.h, src.h, self._real(v))

    def div(self, src, v):
        return self._call("div", self.h, src.h, self._real(v))

    def cadd(self, src1, v, src2):  # self = src1 + v * src2
        return self._call("cadd", self.h, src1.h, self._real(v), src2.h)

    def csub(self, src1, v, src2):
        return self._call("csub", self.h, src1.h, self._real(v), src2.h)

    def cmul(self, src1, src2):
        return self._call("cmul", self.h, src1.h, src2.h)

    def cdiv(self, src1, src2):
        return self._call("cdiv", self.h, src1.h, src2.h)

    def addcmul(self, t, v, src1, src2):  # self = t + v * src1 * src2
        return self._call("addcmul", self.h, t.h, self._real(v), src1.h, src2.h)

    def addcdiv(self, t, v, src1, src2):
        return self._call("addcdiv", self.h, t.h, self._real(v), src1.h, src2.h)

    def unary(self, name, src):          # self = name(src): exp, log, abs, ...
        return self._call(name, self.h, src.h)

    def clamp(self, src, lo, hi):
        return self._call("clamp", self.h, src.h, self._real(lo), self._real(hi))

    def pow(self, src, v):
        return self._call("pow", self.h, src.h, self._real(v))

    def tpow(self, v, src):
        return self._call("tpow", self.h, self._real(v), src.h)

    def scalar2(self, name, src, v):     # cmaxValue, cminValue, fmod, remainder
        return self._call(name, self.h, src.h, self._real(v))

    def binary(self, name, src1, src2):  # cpow, cmax, cmin, cfmod, cremainder, atan2
        return self._call(name, self.h, src1.h, src2.h)

    def lerp(self, a, b, w):
        return self._call("lerp", self.h, a.h, b.h, self._real(w))

    def copy_from(self, src):            # type-converting copy, any kind to any kind
        return self._call("copyCuda" + _COPY_SUFFIX[src.kind], self.h, src.h)

    def compare_value(self, cmp, src, v, same_type=False):
        """self = src (cmp) v as 0/1; self is a Byte tensor unless same_type."""
        return getattr(lib(), "%s_%sValue%s" % (src.T, cmp, "T" if same_type else ""))(
            self._st, self.h, src.h, src._real(v)) or _check() or self

    def compare_tensor(self, cmp, a, b, same_type=False):
        return getattr(lib(), "%s_%sTensor%s" % (a.T, cmp, "T" if same_type else ""))(
            self._st, self.h, a.h, b.h) or _check() or self

    def equal(self, other):
        r = self._fn("equal")(self._st, self.h, other.h)
        _check()
        return bool(r)

    def sum(self, src, dim, keepdim=1):   # dim is 0-based, as at the C level
        return self._call("sum", self.h, src.h, dim, keepdim)

    def prod(self, src, dim, keepdim=1):
        return self._call("prod", self.h, src.h, dim, keepdim)

    def mean(self, src, dim, keepdim=1):
        return self._call("mean", self.h, src.h, dim, keepdim)

    def norm(self, src, p, dim, keepdim=1):
        return self._call("norm", self.h, src.h, self._real(p), dim, keepdim)

    def cumsum(self, src, dim):
        return self._call("cumsum", self.h, src.h, dim)

    def cumprod(self, src, dim):
        return self._call("cumprod", self.h, src.h, dim)

    def renorm(self, src, p, dim, maxnorm):
        return self._call("renorm", self.h, src.h, self._real(p), dim, self._real(maxnorm))

    def var(self, src, dim, biased=0, keepdim=1):
        return self._call("var", self.h, src.h, dim, biased, keepdim)

    def std(self, src, dim, biased=0, keepdim=1):
        return self._call("std", self.h, src.h, dim, biased, keepdim)

    def varall(self, biased=0):
        return self._scalar("varall", biased)

    def stdall(self, biased=0):
        return self._scalar("stdall", biased)

    def dist(self, other, p):
        r = self._fn("dist")(self._st, self.h, other.h, self._real(p))
        _check()
        return r

    def max(self, indices, src, dim, keepdim=1):  # self = values
        return self._call("max", self.h, indices.h, src.h, dim, keepdim)

    def min(self, indices, src, dim, keepdim=1):
        return self._call("min", self.h, indices.h, src.h, dim, keepdim)

    def _scalar(self, name, *args):
        r = self._fn(name)(self._st, self.h, *args)
        _check()
        return r

    def sumall(self):
        return self._scalar("sumall")

    def sumall_no_alloc(self, result):
        """Launches the sum of all elements into result[0] (a float device tensor);
        does not wait for the stream (THCudaTensor_sumallNoAlloc)."""
        lib().THCudaTensor_sumallNoAlloc(self._st, self.h, C.c_void_p(result.data_ptr()))
        _check()
        return result

    def prodall(self):
        return self._scalar("prodall")

    def meanall(self):
        return self._scalar("meanall")

    def normall(self, p):
        return self._scalar("normall", self._real(p))

    def _real_out(self, r):
        if self.kind == "half":
            return float(np.array(r, dtype=np.uint16).view(np.float16))
        return r

    def logicalall(self):
        r = lib().THCudaByteTensor_logicalall(self._st, self.h)
        _check()
        return r

    def logicalany(self):
        r = lib().THCudaByteTensor_logicalany(self._st, self.h)
        _check()
        return r

    def minall(self):
        return self._real_out(self._scalar("minall"))

    def maxall(self):
        return self._real_out(self._scalar("maxall"))


def cached_memory():
    """(free incl. parked blocks, total, largest block) from THCudaMemGetInfoCached."""
    f, t, b = C.c_size_t(0), C.c_size_t(0), C.c_size_t(0)
    err = lib().THCudaMemGetInfoCached(state(), C.byref(f), C.byref(t), C.byref(b))
    if err:
        raise THCError("THCudaMemGetInfoCached failed: %d" % err)
    return f.value, t.value, b.value


def last_kernel():
    return lib().THCAmd_lastKernel().decode()


def set_tuning(key, value):
    lib().THCAmd_setTuning(key.encode(), int(value))


def force_64bit_index(on):
    lib().THCAmd_setForce64BitIndex(1 if on else 0)


def synchronize():
    """Wait for the engine's current stream (hipStreamSynchronize)."""
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamSynchronize.argtypes = [C.c_void_p]
    err = hip.hipStreamSynchronize(lib().THCState_getCurrentStream(state()))
    if err:
        raise THCError("hipStreamSynchronize failed: %d" % err)
