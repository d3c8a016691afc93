"""Host-side logic of the engine, exercised without a GPU through the layout
hooks of the C ABI: collapse (lib/THC/THCTensorInfo.cuh:76-224), linear index
-> offset (:229-278), overlap test and index-width rule
(lib/THC/THCTensorTypeUtils.cu:164-245), the joint collapse used by the apply
planner, and the fp16 conversion used for host staging. Everything is checked
by brute force over tiny shapes or exhaustively."""
import ctypes as C
import itertools
import os
import re
import subprocess

import numpy as np
import pytest

import cutorch_amd
from tests.util import random_geometry

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def L(seq):
    return (C.c_long * max(1, len(seq)))(*seq)


def all_offsets(size, stride):
    """Offsets in logical row-major order by a plain nested loop."""
    return [sum(i * s for i, s in zip(idx, stride)) for idx in itertools.product(*[range(n) for n in size])]


def collapse(size, stride, exclude=-1):
    lib = cutorch_amd.lib()
    osz, ost, od = L([0] * 25), L([0] * 25), C.c_int(0)
    r = lib.THCAmd_collapseDims(len(size), L(size), L(stride), exclude, osz, ost, C.byref(od))
    return r, list(osz[:od.value]), list(ost[:od.value])


def test_worked_examples():
    assert collapse((4, 1, 3), (3, 3, 1))[1:] == ([12], [1])
    assert collapse((3, 4), (1, 3))[1:] == ([3, 4], [1, 3])            # transposed
    assert collapse((2, 3, 4), (24, 4, 1))[1:] == ([2, 12], [24, 1])   # hole in dim 0
    assert collapse((4, 3), (5, 1))[1:] == ([4, 3], [5, 1])            # narrowed last dim
    assert collapse((2, 3), (0, 1))[1:] == ([2, 3], [0, 1])            # expanded
    assert collapse((2, 3, 4), (12, 4, 1), 1) == (1, [2, 3, 4], [12, 4, 1])
    assert collapse((2, 3, 4), (12, 4, 1), 0) == (0, [2, 12], [12, 1])
    assert collapse((1, 1, 1), (7, 3, 9))[1:] == ([1], [1])
    assert collapse((2, 3, 4), (12, 4, 1))[1:] == ([24], [1])


@pytest.mark.parametrize("seed", range(40))
def test_collapse_preserves_offsets_brute_force(seed):
    rng = np.random.default_rng(seed)
    nd = int(rng.integers(1, 6))
    shape = tuple(int(x) for x in rng.integers(1, 5, nd))
    _, _, size, stride = random_geometry(rng, shape, holes=bool(seed % 2), permute=bool(seed % 3))
    want = all_offsets(size, stride)
    _, csz, cst = collapse(size, stride)
    assert all_offsets(csz, cst) == want
    assert len(csz) <= nd
    lib = cutorch_amd.lib()
    for lin in range(len(want)):
        assert lib.THCAmd_indexToOffset(nd, L(size), L(stride), lin) == want[lin]
    # with an excluded dim: that dim survives with its size/stride and the
    # remaining dims still enumerate the same offsets
    ex = int(rng.integers(0, nd))
    r, esz, est = collapse(size, stride, ex)
    assert all_offsets(esz, est) == want
    assert esz[r] == size[ex] and (est[r] == stride[ex] or size[ex] == 1)


def test_contiguous_collapses_to_one_dim():
    for shape in ((2, 3, 4), (5,), (1, 6, 1, 2), (3, 1)):
        stride = tuple(int(np.prod(shape[i + 1:])) for i in range(len(shape)))
        _, csz, cst = collapse(shape, stride)
        assert csz == [int(np.prod(shape))] and cst == [1]


@pytest.mark.parametrize("seed", range(30))
def test_overlap_brute_force(seed):
    rng = np.random.default_rng(100 + seed)
    nd = int(rng.integers(1, 4))
    size = tuple(int(x) for x in rng.integers(1, 5, nd))
    stride = tuple(int(x) for x in rng.integers(0, 7, nd))
    offs = all_offsets(size, stride)
    really = len(set(offs)) != len(offs)
    said = bool(cutorch_amd.lib().THCAmd_overlappingIndices(nd, L(size), L(stride)))
    # the test is conservative: it may call a non-overlapping exotic layout
    # overlapping (e.g. strides (2,3) sizes (2,2)), never the other way round
    assert said or not really
    if not said:
        assert not really


def test_overlap_known_cases():
    ov = lambda sz, st: bool(cutorch_amd.lib().THCAmd_overlappingIndices(len(sz), L(sz), L(st)))
    assert not ov((3, 4), (4, 1)) and not ov((3, 4), (1, 3)) and not ov((3, 4), (8, 2))
    assert ov((3, 4), (0, 1)) and ov((3, 4), (2, 1)) and ov((5,), (0,))
    assert not ov((1, 4), (0, 1)) and not ov((1,), (0,))


def test_index_width_rule():
    f = lambda sz, st: bool(cutorch_amd.lib().THCAmd_canUse32BitIndexMath(len(sz), L(sz), L(st)))
    assert f((1 << 24,), (1,))
    assert f((8192, 8192), (1, 8192))
    assert not f((2048, 2048, 520), (1, 2048, 4194304))      # 2.18e9 elements
    assert not f((2048, 2048, 520), (1064960, 520, 1))
    assert f(((1 << 31) - 1,), (1,)) and not f((1 << 31,), (1,))
    assert not f((2, 2), (1 << 31, 1))                       # small count, far offset
    assert f((65536, 1024), (1024, 1))


@pytest.mark.parametrize("seed", range(30))
def test_joint_collapse_brute_force(seed):
    rng = np.random.default_rng(500 + seed)
    nd = int(rng.integers(1, 5))
    nops = int(rng.integers(1, 5))
    shape = tuple(int(x) for x in rng.integers(1, 5, nd))
    strides = []
    for k in range(nops):
        contiguous = rng.random() < 0.4
        _, _, _, st = random_geometry(rng, shape, holes=not contiguous, permute=not contiguous)
        strides += list(st)
    osz, ost = L([0] * 25), L([0] * 100)
    m = cutorch_amd.lib().THCAmd_jointCollapse(nops, nd, L(shape), L(strides), osz, ost)
    assert 1 <= m <= max(nd, 1)
    csz = list(osz[:m])
    for k in range(nops):
        assert all_offsets(csz, list(ost[k * m:(k + 1) * m])) == all_offsets(shape, strides[k * nd:(k + 1) * nd])


def test_fp16_conversion_exhaustive():
    lib = cutorch_amd.lib()
    allbits = np.arange(65536, dtype=np.uint16)
    f = allbits.view(np.float16).astype(np.float32)
    for b in range(0, 65536, 7):
        got = np.float32(lib.THC_half2float(b))
        assert got.view(np.uint32) == f[b].view(np.uint32) or (np.isnan(got) and np.isnan(f[b]))
        if not np.isnan(f[b]):
            assert lib.THC_float2half(float(f[b])) == b
    fin = np.sort(f[np.isfinite(f)].astype(np.float64))
    mids = ((fin[:-1] + fin[1:]) / 2).astype(np.float32)[::5]
    probes = np.concatenate([mids, np.nextafter(mids, np.float32(np.inf)),
                             np.array([65504, 65520, 65519.99, 1e10, 2.9802322e-8, 2.9802326e-8],
                                      dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = probes.astype(np.float16).view(np.uint16)
    for x, w in zip(probes, want):
        assert lib.THC_float2half(float(x)) == int(w), x


def test_64bit_multiply_shift_division_is_exact():
    """The 64-bit index kernels divide by launch-invariant sizes with a 65-bit multiplier and a shift;
    against Python's integers for the divisors and dividends where such schemes break first: 1, powers
    of two and their neighbours, divisors just above and below 2^32 and 2^63, dividends that are
    multiples of the divisor and one less, and the largest values."""
    lib = cutorch_amd.lib()
    lib.THCAmd_divmod64.argtypes = [C.c_ulonglong, C.c_ulonglong, C.POINTER(C.c_ulonglong), C.POINTER(C.c_ulonglong)]
    lib.THCAmd_divmod64.restype = None
    rng = np.random.default_rng(11)
    top = (1 << 64) - 1
    divisors = {1, 2, 3, 5, 6, 7, 10, 520, 2048, 8191, 8193, 641, 6700417, 274177, 67280421310721, top, top - 1}
    for k in range(1, 64):
        divisors |= {1 << k, (1 << k) + 1, (1 << k) - 1}
    divisors |= {int(x) for x in rng.integers(1, 1 << 63, 200, dtype=np.uint64)}
    divisors |= {int(x) >> int(sh) for x, sh in zip(rng.integers(1 << 62, 1 << 63, 200, dtype=np.uint64),
                                                 rng.integers(0, 62, 200))}
    divisors.discard(0)
    q, r = C.c_ulonglong(), C.c_ulonglong()
    for d in sorted(divisors):
        ns = {0, 1, d - 1, d, d + 1, top, top - 1, top - d, (top // d) * d, (top // d) * d - 1, 1 << 63, (1 << 63) - 1,
              (1 << 32) - 1, 1 << 32}
        ns |= {int(x) for x in rng.integers(0, 1 << 63, 24, dtype=np.uint64)}
        ns |= {(int(x) * d) & top for x in rng.integers(0, 1 << 40, 8, dtype=np.uint64)}
        for n in ns:
            if not 0 <= n <= top:
                continue
            lib.THCAmd_divmod64(n, d, C.byref(q), C.byref(r))
            assert (q.value, r.value) == (n // d, n % d), (n, d)


def test_library_exports_every_declared_symbol():
    """Every function declared in include/THC.h is exported by libTHC.so."""
    header = os.path.join(ROOT, "include", "THC.h")
    pre = subprocess.run(["gcc", "-E", "-P", header], capture_output=True, text=True, check=True).stdout
    names = set(re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(", pre))
    names = {n for n in names if n.startswith(("TH", "__THC"))}
    names -= {"THErrorHandlerFunction", "THArgErrorHandlerFunction"}
    assert len(names) > 250
    nm = subprocess.run(["nm", "-D", "--defined-only", cutorch_amd.LIB_PATH], capture_output=True,
                        text=True, check=True).stdout
    exported = {line.split()[-1] for line in nm.splitlines() if line.strip()}
    missing = sorted(names - exported)
    assert not missing, missing
    lib = cutorch_amd.lib()
    for n in sorted(names):
        getattr(lib, n)


def test_struct_layout_matches_header():
    src = '#include <stdio.h>\n#include <stddef.h>\n#include "THC.h"\nint main(){printf("%zu %zu %zu %zu %zu %zu\\n",' \
          'sizeof(THCudaTensor),offsetof(THCudaTensor,storage),offsetof(THCudaTensor,storageOffset),' \
          'sizeof(THCudaStorage),offsetof(THCudaStorage,allocator),offsetof(THCudaStorage,device));return 0;}'
    exe = "/tmp/thc_layout_probe"
    subprocess.run(["gcc", "-x", "c", "-", "-I", os.path.join(ROOT, "include"), "-o", exe], input=src,
                   text=True, check=True)
    got = [int(x) for x in subprocess.run([exe], capture_output=True, text=True, check=True).stdout.split()]
    T, S = cutorch_amd._Tensor, cutorch_amd._Storage
    assert got == [C.sizeof(T), T.storage.offset, T.storageOffset.offset, C.sizeof(S),
                   S.allocator.offset, S.device.offset]
    assert got == [48, 24, 32, 56, 24, 48]   # LP64 layout of generic/THCTensor.h:7-19, THCStorage.h:9-19
