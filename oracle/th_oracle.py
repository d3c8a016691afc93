"""ctypes loader for the CPU oracle (oracle/libth_oracle.so).

TEST INFRASTRUCTURE: only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import this module. Build the library with
`make -C oracle`.

A tensor is described the way a TH view is: a host storage array, a storage
offset, sizes and strides in elements. `View` keeps that description; results
are written into the storage array in place, so holes can be checked too.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libth_oracle.so")

OPS = {"copy": 0, "addc": 1, "subc": 2, "mulc": 3, "divc": 4, "add": 5, "sub": 6, "mul": 7,
       "div": 8, "cadd": 9, "addcmul": 10, "addcdiv": 11, "fill": 12, "pow": 13}
DTYPES = {"float": 0, "half": 1, "long": 2, "byte": 3, "char": 4, "short": 5, "int": 6, "double": 7}
NP_OF = {"float": np.float32, "half": np.float16, "long": np.int64, "byte": np.uint8, "char": np.int8,
         "short": np.int16, "int": np.int32, "double": np.float64}
KIND_OF = {np.dtype(v): k for k, v in NP_OF.items()}
CMPS = {"lt": 0, "gt": 1, "le": 2, "ge": 3, "eq": 4, "ne": 5}
FNS = ["sigmoid", "log", "lgamma", "log1p", "exp", "cos", "acos", "cosh", "sin", "asin", "sinh", "tan",
       "atan", "tanh", "sqrt", "rsqrt", "ceil", "floor", "round", "trunc", "frac", "cinv", "neg", "abs",
       "sign", "clamp", "sqdiffValue", "pow", "tpow", "cmaxValue", "cminValue", "fmod", "remainder",
       "cpow", "cmax", "cmin", "cfmod", "cremainder", "atan2", "equal", "sqdiff",
       "lshift", "rshift", "bitand", "bitor", "bitxor", "clshift", "crshift", "cbitand", "cbitor", "cbitxor"]
BINARY_FNS = {"cpow", "cmax", "cmin", "cfmod", "cremainder", "atan2", "equal", "sqdiff", "clshift", "crshift",
              "cbitand", "cbitor", "cbitxor"}
OPS["lerp"] = 14
for _i, _n in enumerate(FNS):
    OPS["fn:" + _n] = (200 if _n in BINARY_FNS else 100) + _i
KINDS = {"sum": 0, "prod": 1, "min": 2, "max": 3, "norm": 4, "mean": 5, "var_biased": 6, "var": 7,
         "std_biased": 8, "std": 9}


class _CView(C.Structure):
    _fields_ = [("data", C.c_void_p), ("nd", C.c_int), ("size", C.POINTER(C.c_long)),
                ("stride", C.POINTER(C.c_long))]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is missing: run `make -C oracle`" % LIB_PATH)
        l = C.CDLL(LIB_PATH)
        VP = C.POINTER(_CView)
        for suffix in ("float", "half"):
            f = getattr(l, "th_pointwise_" + suffix)
            f.argtypes = [C.c_int, C.c_float, VP, VP, VP, VP]
            f.restype = C.c_int
            f = getattr(l, "th_reduce_dim_" + suffix)
            f.argtypes = [C.c_int, C.c_double, VP, VP, C.c_int]
            f.restype = C.c_int
            for mm in ("max", "min"):
                f = getattr(l, "th_%s_dim_%s" % (mm, suffix))
                f.argtypes = [VP, VP, VP, C.c_int]
                f.restype = C.c_int
            f = getattr(l, "th_reduce_all_" + suffix)
            f.argtypes = [C.c_int, C.c_double, VP]
            f.restype = C.c_double
            f = getattr(l, "th_scan_dim_" + suffix)
            f.argtypes = [C.c_int, VP, VP, C.c_int]
            f.restype = C.c_int
            f = getattr(l, "th_var_all_" + suffix)
            f.argtypes = [VP, C.c_int]
            f.restype = C.c_double
        l.th_typed_pointwise.argtypes = [C.c_int, C.c_int, C.c_int, C.c_double, C.c_long, C.c_double, C.c_long,
                                         VP, VP, VP, VP]
        l.th_typed_compare.argtypes = [C.c_int, C.c_int, C.c_int, C.c_double, C.c_long, VP, VP, VP]
        l.th_typed_convert.argtypes = [C.c_int, VP, C.c_int, VP]
        l.th_typed_reduce_dim.argtypes = [C.c_int, C.c_int, VP, VP, C.c_int]
        l.th_typed_minmax_dim.argtypes = [C.c_int, C.c_int, VP, VP, VP, C.c_int]
        l.th_typed_reduce_all.argtypes = [C.c_int, C.c_int, VP, C.POINTER(C.c_long)]
        l.th_typed_reduce_all.restype = C.c_double
        l.th_typed_scan_dim.argtypes = [C.c_int, C.c_int, VP, VP, C.c_int]
        l.th_renorm.argtypes = [C.c_int, VP, VP, C.c_double, C.c_int, C.c_double]
        l.th_half2float.argtypes = [C.c_uint16]
        l.th_half2float.restype = C.c_float
        l.th_float2half.argtypes = [C.c_float]
        l.th_float2half.restype = C.c_uint16
        l.th_half2float_array.argtypes = [C.c_void_p, C.c_void_p, C.c_long]
        l.th_float2half_array.argtypes = [C.c_void_p, C.c_void_p, C.c_long]
        l.th_set_num_threads.argtypes = [C.c_int]
        l.th_set_second_scalar.argtypes = [C.c_float]
        _lib = l
    return _lib


class View(object):
    """A strided view on a host storage array (any of the eight element types)."""

    def __init__(self, storage, offset=0, size=None, stride=None):
        assert storage.flags["C_CONTIGUOUS"] and storage.ndim == 1
        self.storage = storage
        self.offset = int(offset)
        if size is None:
            size = (storage.size,) if storage.size else ()
        self.size = tuple(int(s) for s in size)
        if stride is None:
            stride, run = [], 1
            for s in reversed(self.size):
                stride.append(run)
                run *= s
            stride = tuple(reversed(stride))
        self.stride = tuple(int(s) for s in stride)
        n = max(1, len(self.size))
        self._size = (C.c_long * n)(*self.size)
        self._stride = (C.c_long * n)(*self.stride)
        self.c = _CView(storage.ctypes.data + self.offset * storage.itemsize, len(self.size),
                        self._size, self._stride)

    @classmethod
    def of(cls, arr):
        """Contiguous view holding a copy of `arr`."""
        arr = np.ascontiguousarray(arr)
        return cls(arr.reshape(-1).copy(), 0, arr.shape)

    @classmethod
    def empty(cls, shape, dtype=np.float32):
        n = int(np.prod(shape)) if len(shape) else 0
        return cls(np.zeros(n, dtype=dtype), 0, shape)

    @property
    def is_half(self):
        return self.storage.dtype == np.float16

    @property
    def kind(self):
        return KIND_OF[self.storage.dtype]

    def numpy(self):
        """Logical contents, gathered through numpy's own stride machinery."""
        if not self.size:
            return np.empty((0,), dtype=self.storage.dtype)
        item = self.storage.itemsize
        return np.lib.stride_tricks.as_strided(
            self.storage[self.offset:], shape=self.size,
            strides=tuple(s * item for s in self.stride)).copy()


def _ptr(v):
    return C.byref(v.c) if v is not None else None


def pointwise(op, out, a=None, b=None, c=None, value=0.0, value2=0.0):
    """op: a name from OPS; the math family is spelled "fn:<name>" (e.g.
    "fn:exp", "fn:clamp" with value = min and value2 = max, "fn:cmax")."""
    lib().th_set_second_scalar(value2)
    f = lib().th_pointwise_half if out.is_half else lib().th_pointwise_float
    rc = f(OPS[op], value, _ptr(out), _ptr(a), _ptr(b), _ptr(c))
    if rc:
        raise ValueError("sizes do not match")
    return out


def _int_scalar(kind, v):
    """The scalar as the element type holds it (wrapped), as a Python int."""
    if kind in ("float", "half", "double"):
        return 0
    return int(np.array(int(v)).astype(NP_OF[kind]))


def typed_pointwise(op, out, a=None, b=None, c=None, value=0, value2=0):
    """Pointwise op on byte/char/short/int/long/double views. `op` as for
    pointwise(): a name from OPS or "fn:<name>"."""
    kind = out.kind
    code = OPS[op]
    fn = 0
    if code >= 200:
        code, fn = 200, code - 200
    elif code >= 100:
        code, fn = 100, code - 100
    rc = lib().th_typed_pointwise(DTYPES[kind], code, fn, float(value), _int_scalar(kind, value),
                                  float(value2), _int_scalar(kind, value2), _ptr(out), _ptr(a), _ptr(b),
                                  _ptr(c))
    if rc:
        raise ValueError("sizes do not match")
    return out


def typed_compare(cmp, out, a, b=None, value=0):
    """out = a (cmp) (b or value) as 0/1; out is a byte view or one of a's kind."""
    kind = a.kind
    vf = float(np.float16(value)) if kind == "half" else (float(np.float32(value)) if kind == "float" else float(value))
    rc = lib().th_typed_compare(DTYPES[kind], DTYPES[out.kind], CMPS[cmp], vf, _int_scalar(kind, value),
                                _ptr(out), _ptr(a), _ptr(b))
    if rc:
        raise ValueError("sizes do not match")
    return out


def typed_convert(dst, src):
    if lib().th_typed_convert(DTYPES[dst.kind], _ptr(dst), DTYPES[src.kind], _ptr(src)):
        raise ValueError("sizes do not match")
    return dst


TYPED_KINDS = {"sum": 0, "prod": 1, "min": 2, "max": 3, "mean": 4}


def typed_reduce_dim(kind, src, dim, out=None):
    """sum / prod / min / max / mean along dim for byte..long and double views."""
    if out is None:
        out = View.empty(reduced_shape(src.size, dim), src.storage.dtype)
    if lib().th_typed_reduce_dim(DTYPES[src.kind], TYPED_KINDS[kind], _ptr(out), _ptr(src), dim):
        raise ValueError("shape mismatch")
    return out


def typed_minmax_dim(which, src, dim):
    shape = reduced_shape(src.size, dim)
    values, indices = View.empty(shape, src.storage.dtype), View.empty(shape, np.int64)
    if lib().th_typed_minmax_dim(DTYPES[src.kind], 1 if which == "max" else 0, _ptr(values), _ptr(indices),
                                 _ptr(src), dim):
        raise ValueError("shape mismatch")
    return values, indices


def typed_scan_dim(src, dim, product=False):
    out = View.empty(src.size, src.storage.dtype)
    if lib().th_typed_scan_dim(DTYPES[src.kind], 1 if product else 0, _ptr(out), _ptr(src), dim):
        raise ValueError("shape mismatch")
    return out


def renorm(src, p, dim, maxnorm, out=None):
    """float / half / double views."""
    if out is None:
        out = View.empty(src.size, src.storage.dtype)
    if lib().th_renorm(DTYPES[src.kind], _ptr(out), _ptr(src), float(p), dim, float(maxnorm)):
        raise ValueError("shape mismatch")
    return out


def typed_reduce_all(kind, src):
    """accreal result: a Python int for the integer kinds, a float for double."""
    ri = C.c_long(0)
    rf = lib().th_typed_reduce_all(DTYPES[src.kind], TYPED_KINDS[kind], _ptr(src), C.byref(ri))
    return rf if src.kind == "double" else ri.value


def reduced_shape(shape, dim):
    return tuple(1 if d == dim else s for d, s in enumerate(shape))


def reduce_dim(kind, src, dim, p=0.0, out=None):
    if out is None:
        out = View.empty(reduced_shape(src.size, dim), src.storage.dtype)
    f = lib().th_reduce_dim_half if src.is_half else lib().th_reduce_dim_float
    if f(KINDS[kind], p, _ptr(out), _ptr(src), dim):
        raise ValueError("shape mismatch")
    return out


def minmax_dim(which, src, dim, values=None, indices=None):
    shape = reduced_shape(src.size, dim)
    if values is None:
        values = View.empty(shape, src.storage.dtype)
    if indices is None:
        indices = View.empty(shape, np.int64)
    f = getattr(lib(), "th_%s_dim_%s" % (which, "half" if src.is_half else "float"))
    if f(_ptr(values), _ptr(indices), _ptr(src), dim):
        raise ValueError("shape mismatch")
    return values, indices


def reduce_all(kind, src, p=0.0):
    f = lib().th_reduce_all_half if src.is_half else lib().th_reduce_all_float
    return f(KINDS[kind], p, _ptr(src))


def scan_dim(src, dim, product=False, out=None):
    if out is None:
        out = View.empty(src.size, src.storage.dtype)
    f = lib().th_scan_dim_half if src.is_half else lib().th_scan_dim_float
    if f(1 if product else 0, _ptr(out), _ptr(src), dim):
        raise ValueError("shape mismatch")
    return out


def var_all(src, biased=False):
    f = lib().th_var_all_half if src.is_half else lib().th_var_all_float
    return f(_ptr(src), 1 if biased else 0)


def set_num_threads(n):
    lib().th_set_num_threads(int(n))
