#!/usr/bin/env python3
"""Benchmark of the apply / reduce hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs all|primary] [--no-cpu]

A "step" is one pass of the hot path over one batch of synthetic input that is
already resident in HBM. The headline line is quoted on the largest
configuration that fits one GPU: c = a + b on 2048 x 2048 x 520 fp32 (26 GB),
a viewed through permute(3,2,1), 64-bit indices. Every other benchmark
configuration is measured in the same run and reported under
"roofline.configs" (fraction of peak, microseconds per launch, parity flag)
and, as flat scalars that survive a parser which keeps scalars only, as
"roofline.frac_<config>" / "roofline.parity_<config>", with a plain
1-read-1-write calibration stream ("CAL-copy") that tells a slow box from a
regression, and host-side call latencies of three small calls ("latency").
Prints ONE JSON line.

  value               algorithmic bytes * steps / wall time of the timed region
  roofline.achieved   algorithmic bytes / average launch duration, from two
                      HIP events that bracket the K launches of the timed
                      region on the stream the engine launches on
  roofline.configs    the same per configuration; "parity" is a check of the
                      configuration's own output, outside the timed region,
                      against a closed form computed with numpy on the host
                      copy of the inputs (bit-exact for add/mul/addcmul and
                      max+argmax, 1e-5 / 2e-3 relative for sums and norms)
  cpu_baseline        the CPU restatement (oracle/) timed on this box's host
                      cores: a 1/16 sample of the headline workload (the same
                      strides, 32 of the 520 planes) single-threaded is the
                      value; all-core figures, the strided apply3 (C2) and the
                      reduction path (row sums of 65536 x 1024, middle-dim sums
                      of 64 x 4096 x 512) are reported beside it under
                      "configs" and as flat "<config>_single_gbps" /
                      "<config>_all_cores_gbps" scalars
  --configs all       adds the neighbours of the hot path (N-* lines) and the
                      full per-configuration detail under "all_configs"
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_GBPS = 8000.0
METRIC = "achieved HBM GB/s (% of ~8 TB/s peak): pointwise apply + dim reduction, fp32"


class Hip(object):
    def __init__(self):
        self.l = C.CDLL("libamdhip64.so")
        self.l.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.l.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.l.hipEventSynchronize.argtypes = [C.c_void_p]
        self.l.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.l.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        self.l.hipDeviceSynchronize.argtypes = []

    def check(self, err, what):
        if err != 0:
            raise RuntimeError("%s failed with hip error %d" % (what, err))

    def event(self):
        e = C.c_void_p()
        self.check(self.l.hipEventCreate(C.byref(e)), "hipEventCreate")
        return e

    def record(self, e, stream):
        self.check(self.l.hipEventRecord(e, stream), "hipEventRecord")

    def elapsed_ms(self, a, b):
        self.check(self.l.hipEventSynchronize(b), "hipEventSynchronize")
        ms = C.c_float()
        self.check(self.l.hipEventElapsedTime(C.byref(ms), a, b), "hipEventElapsedTime")
        return ms.value

    def sync(self):
        self.check(self.l.hipDeviceSynchronize(), "hipDeviceSynchronize")

    def d2d(self, dst, src, nbytes):
        self.check(self.l.hipMemcpy(dst, src, nbytes, 3), "hipMemcpy d2d")


def device_fill_from_block(hip, thc, shape, block):
    """A device tensor of `shape` whose storage repeats `block` (host array):
    lets the 8.7 GB operands of the 64-bit-index configuration be set up in
    seconds; values stay normal(0,1)."""
    t = thc.Tensor("float").resize(shape)
    n = int(np.prod(shape))
    blk = thc.Tensor.from_numpy(block)
    base = t.data_ptr()
    done = 0
    while done < n:
        m = min(block.size, n - done)
        hip.d2d(base + 4 * done, blk.data_ptr(), 4 * m)
        done += m
    return t


class Config(object):
    """One benchmark configuration: `sets` rotating operand sets, a `run(i)`
    that launches the op on set i, its algorithmic byte count, and `check()`,
    which runs the op once more outside the timed region and compares its
    output with a closed form computed by numpy from the host inputs."""

    def __init__(self, name, desc, nbytes, elements, sets, run, check=None, kernel=None):
        self.name, self.desc, self.nbytes, self.elements = name, desc, nbytes, elements
        self.sets, self.run, self.check, self.kernel = sets, run, check, kernel
        self.note = None


def bit_equal(got, want):
    got, want = np.ascontiguousarray(got), np.ascontiguousarray(want)
    u = {2: np.uint16, 4: np.uint32, 8: np.uint64}[got.itemsize]
    return got.shape == want.shape and bool(np.array_equal(got.view(u), want.view(u)))


def sums_close(got, ref64, mass, rel):
    """|got - ref| <= rel * max(|ref|, mass / 64): the stated relative bound, with a
    floor of 1/64 of the summed magnitudes for results that cancel."""
    got = np.asarray(got, np.float64).reshape(-1)
    ref64 = np.asarray(ref64, np.float64).reshape(-1)
    mass = np.asarray(mass, np.float64).reshape(-1)
    return bool(np.all(np.abs(got - ref64) <= rel * np.maximum(np.abs(ref64), mass / 64.0)))


def build_configs(thc, hip, which, only=None, stagger=0):
    rng = np.random.default_rng(0xC0FFEE)
    cfgs = []
    T = thc.Tensor
    host = {}

    def want(*names):
        return not only or any(n in only for n in names)

    # C5 (the headline): 2048 x 2048 x 520 with a = permute(3,2,1) view, 64-bit index path. The 8.7 GB
    # operands repeat a 2^24-element block of normal(0,1) values (the element at storage offset o is
    # block[o % 2^24]).
    if want('C5', 'CEIL-2r1w-26GB'):
        nb5 = 1 << 24
        block = rng.standard_normal(nb5, dtype=np.float32)
        rblock = block[::-1].copy()
        a5 = device_fill_from_block(hip, thc, (520, 2048, 2048), block)
        b5 = device_fill_from_block(hip, thc, (2048, 2048, 520), rblock)
        c5 = T("float").resize((2048, 2048, 520))
        a5v = a5.view_as_strided(0, (2048, 2048, 520), (1, 2048, 2048 * 2048))
        n5 = 2048 * 2048 * 520
        planes = sorted(set(range(0, 2048, 31)) | {1, 1023, 1024, 2047})     # 70 of the 2048 [j][k] planes

        def c5_check():
            ok = True
            j, k = np.arange(2048, dtype=np.int64)[:, None], np.arange(520, dtype=np.int64)[None, :]
            for i in planes:
                got = c5.select(0, i).numpy()
                wa = block[(i + 2048 * j + 2048 * 2048 * k) % nb5]
                wb = rblock[((i * 2048 + j) * 520 + k) % nb5]
                ok = ok and bit_equal(got, wa + wb)
            return ok
        cfgs.append(Config("C5", "c = a + b, 2048x2048x520 fp32, a = permute(3,2,1) view, 64-bit indices",
                           12 * n5, n5, 1, lambda i: c5.cadd(a5v, 1.0, b5), c5_check))
        cfgs[-1].note = "parity on %d of the 2048 output planes, first to last" % len(planes)
        host["C5"] = (block, rblock)
        if which == "all" or (only and "CEIL-2r1w-26GB" in only):
            a5flat = a5.view_as_strided(0, (2048, 2048, 520), (2048 * 520, 520, 1))
            cfgs.append(Config("CEIL-2r1w-26GB", "c = a + b on the same 3 x 8.7 GB buffers, all contiguous (flat ceiling of C5)",
                               12 * n5, n5, 1, lambda i: c5.cadd(a5flat, 1.0, b5)))
        if which == "primary":
            return [c for c in cfgs if want(c.name)], host

    # C2: out = a:t() * b + d, out and d rotating over three buffer sets.
    n2 = 8192
    a2 = rng.standard_normal((n2, n2), dtype=np.float32)
    b2 = rng.standard_normal((n2, n2), dtype=np.float32)
    d2 = [rng.standard_normal((n2, n2), dtype=np.float32)]
    da, db = T.from_numpy(a2), T.from_numpy(b2)
    at = da.t()
    dd = [T.from_numpy(d2[0])]
    out2 = [T("float").resize((n2, n2))]
    for k in (1, 2):      # the other two d buffers are shifted copies of the first (set up on the host once)
        d2.append(np.roll(d2[0], k * 1237, axis=1))
        dd.append(T.from_numpy(d2[k]))
        out2.append(T("float").resize((n2, n2)))

    def c2_check(k):
        def check():
            out2[k].fill(0.0)
            out2[k].addcmul(dd[k], 1.0, at, db)
            want_ = a2.T * b2
            want_ += d2[k]
            return bit_equal(out2[k].numpy(), want_)
        return check
    desc2 = "out = a:t()*b + d, 8192x8192 fp32, a stride (1,8192) [addcmul]"
    cfgs.append(Config("C2", desc2 + ", out and d rotate over 3 buffer sets", 16 * n2 * n2, n2 * n2, 3,
                       lambda i: out2[i % 3].addcmul(dd[i % 3], 1.0, at, db), c2_check(2)))
    host["C2"] = (a2, b2, d2[0])
    cfgs.append(Config("C2-fixed", desc2 + ", one buffer set (the output is rewritten in place every step)",
                       16 * n2 * n2, n2 * n2, 1, lambda i: out2[0].addcmul(dd[0], 1.0, at, db), c2_check(0)))

    # C1: contiguous 2^24, three rotating buffer sets (working set < Infinity Cache)
    n1 = 1 << 24
    sets1, h1 = [], None
    for k in range(3 if want('C1-add', 'C1-mul') else 0):
        ha, hb = rng.uniform(-1, 1, n1).astype(np.float32), rng.uniform(-1, 1, n1).astype(np.float32)
        if k == 0:
            h1 = (ha, hb)
        if stagger:
            # operands inside larger allocations, b and c starting `stagger` and 2 x `stagger` elements in: shifts
            # the three streams against each other in the memory channels' interleave (a probe, see --stagger)
            pad = lambda h, k: T.from_numpy(np.concatenate([np.zeros(k * stagger, np.float32), h])).narrow(0, k * stagger, n1)
            sets1.append((pad(ha, 0), pad(hb, 1), T("float").resize((n1 + 2 * stagger,)).narrow(0, 2 * stagger, n1)))
        else:
            sets1.append((T.from_numpy(ha), T.from_numpy(hb), T("float").resize((n1,))))

    def c1_check(op):
        def check():
            a, b, c = sets1[0]
            c.fill(0.0)
            (c.cadd(a, 1.0, b) if op == "add" else c.cmul(a, b))
            return bit_equal(c.numpy(), h1[0] + h1[1] if op == "add" else h1[0] * h1[1])
        return check
    cfgs.append(Config("C1-add", "c = a + b, 2^24 fp32 contiguous [cadd]", 12 * n1, n1, 3,
                       lambda i: sets1[i % 3][2].cadd(sets1[i % 3][0], 1.0, sets1[i % 3][1]), c1_check("add")))
    cfgs.append(Config("C1-mul", "c = a * b, 2^24 fp32 contiguous [cmul]", 12 * n1, n1, 3,
                       lambda i: sets1[i % 3][2].cmul(sets1[i % 3][0], sets1[i % 3][1]), c1_check("mul")))

    # C3a/b: 65536 x 1024, last dim; ~1 % of every row are copies of other entries of the row,
    # one of them a copy of the row maximum (so that argmax has a tie to resolve)
    r3, n3 = 65536, 1024
    sets3, h3 = [], None
    for k in range(3 if want('C3a-sum', 'C3b-max') else 0):
        x = rng.standard_normal((r3, n3), dtype=np.float32)
        rows = np.arange(r3)
        dup = rng.integers(0, n3, (r3, 10))
        x[rows[:, None], dup] = x[rows[:, None], dup[:, ::-1]]
        x[rows, rng.integers(0, n3, r3)] = x.max(axis=1)
        if k == 0:
            h3 = x
        sets3.append((T.from_numpy(x), T("float").resize((r3, 1)), T("long").resize((r3, 1))))

    def c3a_check():
        x, o, _ = sets3[0]
        o.fill(0.0)
        o.sum(x, 1)
        return sums_close(o.numpy(), h3.sum(axis=1, dtype=np.float64), np.abs(h3).sum(axis=1, dtype=np.float64), 1e-5)

    def c3b_check():
        x, o, ix = sets3[0]
        o.fill(0.0)
        o.max(ix, x, 1)
        am = h3.argmax(axis=1)                   # numpy returns the first occurrence
        return (bit_equal(o.numpy().reshape(-1), h3[np.arange(r3), am])
                and bool(np.array_equal(ix.numpy().reshape(-1), am + 1)))
    cfgs.append(Config("C3a-sum", "sum over last dim of 65536x1024 fp32", 4 * r3 * n3 + 4 * r3, r3 * n3,
                       3, lambda i: sets3[i % 3][1].sum(sets3[i % 3][0], 1), c3a_check))
    cfgs.append(Config("C3b-max", "max+argmax over last dim of 65536x1024 fp32",
                       4 * r3 * n3 + 12 * r3, r3 * n3, 3,
                       lambda i: sets3[i % 3][1].max(sets3[i % 3][2], sets3[i % 3][0], 1), c3b_check))
    host["C3a-sum"] = h3

    # C3c: reduceAll over 2^28
    n3c = 1 << 28
    h3c = rng.random(n3c if want('C3c-sumall', 'N-fill') else 4, dtype=np.float32)
    xa = T.from_numpy(h3c)
    ref3c = float(h3c.sum(dtype=np.float64))

    def c3c_check():
        return sums_close([xa.sumall()], [ref3c], [ref3c], 1e-5)      # all summands are positive: mass = sum
    cfgs.append(Config("C3c-sumall", "sumall over 2^28 fp32 (blocks on a 4-byte D2H copy)",
                       4 * n3c + 4, n3c, 1, lambda i: xa.sumall(), c3c_check))

    # C4: 64 x 4096 x 512, middle dim; fp32 and fp16
    s4 = (64, 4096, 512) if want('C4-sum-f32', 'C4-norm-f32', 'C4-sum-f16', 'C4-norm-f16', 'N-std-cols', 'N-cumsum-cols') else (1, 4, 8)
    x4 = rng.uniform(-2, 2, s4).astype(np.float32)
    d4 = T.from_numpy(x4)
    o4 = T("float").resize((s4[0], 1, s4[2]))
    n4 = int(np.prod(s4))

    def c4_check(kind, half):
        def check():
            if half:
                x, o = sets4h[0]
                hx = h4h.astype(np.float32)
            else:
                x, o, hx = d4, o4, x4
            o.fill(0.0)
            (o.sum(x, 1) if kind == "sum" else o.norm(x, 2.0, 1))
            got = o.numpy().astype(np.float64)
            if kind == "sum":
                ref, mass = hx.sum(axis=1, dtype=np.float64), np.abs(hx).sum(axis=1, dtype=np.float64)
            else:
                ref = np.sqrt(np.square(hx.astype(np.float64)).sum(axis=1))
                mass = ref
            return sums_close(got, ref, mass, 2e-3 if half else 1e-5)
        return check
    cfgs.append(Config("C4-sum-f32", "sum over middle dim of 64x4096x512 fp32", 4 * n4 + 4 * s4[0] * s4[2],
                       n4, 1, lambda i: o4.sum(d4, 1), c4_check("sum", False)))
    cfgs.append(Config("C4-norm-f32", "L2 norm over middle dim of 64x4096x512 fp32",
                       4 * n4 + 4 * s4[0] * s4[2], n4, 1, lambda i: o4.norm(d4, 2.0, 1), c4_check("norm", False)))
    sets4h, h4h = [], None
    for k in range(3):
        hh = (x4 * np.float32(rng.uniform(0.5, 1.0))).astype(np.float16)
        if k == 0:
            h4h = hh
        sets4h.append((T.from_numpy(hh), T("half").resize((s4[0], 1, s4[2]))))
    cfgs.append(Config("C4-sum-f16", "sum over middle dim of 64x4096x512 fp16, fp32 accumulate",
                       2 * n4 + 2 * s4[0] * s4[2], n4, 3, lambda i: sets4h[i % 3][1].sum(sets4h[i % 3][0], 1),
                       c4_check("sum", True)))
    cfgs.append(Config("C4-norm-f16", "L2 norm over middle dim of 64x4096x512 fp16, fp32 accumulate",
                       2 * n4 + 2 * s4[0] * s4[2], n4, 3,
                       lambda i: sets4h[i % 3][1].norm(sets4h[i % 3][0], 2.0, 1), c4_check("norm", True)))
    host["C4-sum-f32"] = x4

    # A plain 1-read-1-write stream of known size: out = src + 0 on 2^26 contiguous fp32 (reads 256 MiB,
    # writes 256 MiB). About 0.88-0.90 of peak on a healthy box; a box that runs write-heavy kernels slowly
    # shows here first.
    nc = 1 << 26
    if want("CAL-copy"):
        hcal = rng.uniform(-1, 1, nc).astype(np.float32)
        csrc, cdst = T.from_numpy(hcal), T("float").resize((nc,))

        def cal_check():
            cdst.fill(1.0)
            cdst.add(csrc, 0.0)
            return bit_equal(cdst.numpy(), hcal + np.float32(0.0))
        cfgs.append(Config("CAL-copy", "out = src + 0, 2^26 fp32 contiguous (1 read + 1 write of 256 MiB each)",
                           8 * nc, nc, 1, lambda i: cdst.add(csrc, 0.0), cal_check))
    # Neighbours of the hot path on the same engines (same operands where possible).
    nx = [n for n in ("N-copy-t", "N-fill", "N-exp", "N-var-rows", "N-std-cols", "N-cumsum-rows",
                      "N-cumsum-cols", "N-dist", "N-varall", "N-int-add", "N-lt-byte", "N-cvt-half",
                      "N-double-sum", "N-renorm", "N-sum-rows33", "N-max-rows33", "N-sum-slab", "N-sum-tall",
                      "N-cumsum-rows10", "N-cumsum-tall", "N-add-t-odd", "N-bias-odd", "N-int-add-t", "N-lt-t", "N-add-2p25", "N-add-2p26", "CEIL-copy-rot", "CEIL-3r1w-rot",
                      "N-half-exp", "N-half-abs-t", "N-half-exp-t", "N-half-exp-t-odd", "N-short-add-t", "N-short-add-t-odd", "N-short-neg-t", "N-int-neg-t", "N-cvt-float-t", "N-cmax-t", "N-cmax-t-odd", "N-int-div-t", "N-int-lt-t",
                      "N-cvt-half-t", "N-equal", "N-copy-contig-64M", "N-copy-contig-256M", "N-copy-contig-1G",
                      "N-add-strided", "N-add-strided-u64", "N-var-tall", "N-cumsum-wide", "N-cumsum-1d", "N-copy-nhwc3", "N-copy-skinny16", "N-argmax-1d", "N-argmax-tall", "N-add-view-odd", "N-cvt-image", "N-transpose-16x16", "N-sumall-t", "N-std-rows8192")
          if (only and n in only) or (not only and which == "all")]
    if nx:
        ne = 1 << 26
        e_src = T.from_numpy(rng.uniform(-1, 1, ne).astype(np.float32))
        e_dst = T("float").resize((ne,))
        sq, sq_t, sq_out = da, at, out2[0]
        x3 = sets3[0][0] if sets3 else T.from_numpy(rng.standard_normal((r3, n3), dtype=np.float32))
        o3 = T("float").resize((r3, 1))
        s3 = T("float").resize((r3, n3))
        s4o = T("float").resize(s4)
        big = 1 << 28
        nodd_ = 8191 * 8193
        table = {
            "N-copy-t": ("out:copy(a:t()), 8192x8192 fp32", 8 * 8192 * 8192, 8192 * 8192, lambda i: sq_out.copy(sq_t)),
            "N-fill": ("fill of 2^28 fp32", 4 * big, big, lambda i: xa.fill(0.5) if xa.numel() == big else e_dst.fill(0.5)),
            "N-exp": ("out = exp(x), 2^26 fp32 contiguous", 8 * ne, ne, lambda i: e_dst.unary("exp", e_src)),
            "N-var-rows": ("var over last dim of 65536x1024 fp32 (input counted once)", 4 * r3 * n3 + 4 * r3,
                           r3 * n3, lambda i: o3.var(x3, 1)),
            "N-std-cols": ("std over middle dim of 64x4096x512 fp32 (input counted once)",
                           4 * n4 + 4 * s4[0] * s4[2], n4, lambda i: o4.std(d4, 1)),
            "N-cumsum-rows": ("cumsum over last dim of 65536x1024 fp32", 8 * r3 * n3, r3 * n3,
                              lambda i: s3.cumsum(x3, 1)),
            "N-cumsum-cols": ("cumsum over middle dim of 64x4096x512 fp32", 8 * n4, n4, lambda i: s4o.cumsum(d4, 1)),
            "N-dist": ("dist(a, b, 2) over 2^26 fp32", 8 * ne, ne, lambda i: e_src.dist(e_dst, 2.0)),
            "N-varall": ("varall over 2^26 fp32 (one read, blocks on the scalar)", 4 * ne, ne, lambda i: e_src.varall()),
        }
        if set(nx) & {"N-int-add", "N-lt-byte", "N-cvt-half", "N-double-sum", "N-renorm"}:
            ia = T.from_numpy(rng.integers(-1000, 1000, ne).astype(np.int32))
            ib = T.from_numpy(rng.integers(-1000, 1000, ne).astype(np.int32))
            ic = T("int").resize((ne,))
            mask = T("byte").resize((ne,))
            hdst = T("half").resize((ne,))
            dsrc = T.from_numpy(rng.uniform(-1, 1, (8192, 4096)))
            dout = T("double").resize((8192, 1))
            table.update({
                "N-int-add": ("c = a + b, 2^26 int32 contiguous", 12 * ne, ne, lambda i: ic.cadd(ia, 1, ib)),
                "N-lt-byte": ("mask = x < 0 into a Byte tensor, 2^26 fp32", 5 * ne, ne,
                              lambda i: mask.compare_value("lt", e_src, 0.0)),
                "N-cvt-half": ("half <- float converting copy, 2^26", 6 * ne, ne, lambda i: hdst.copy_from(e_src)),
                "N-double-sum": ("sum over last dim of 8192x4096 fp64", 8 * 8192 * 4096 + 8 * 8192, 8192 * 4096,
                                 lambda i: dout.sum(dsrc, 1)),
                "N-renorm": ("renorm(p=2, dim 0, maxnorm 1) of 8192x8192 fp32 (one read, one write)",
                             8 * 8192 * 8192, 8192 * 8192, lambda i: sq_out.renorm(sq, 2.0, 0, 1.0)),
            })
        if set(nx) & {"N-sum-rows33", "N-max-rows33", "N-sum-slab", "N-sum-tall", "N-cumsum-rows10",
                      "N-cumsum-tall", "N-add-t-odd", "N-bias-odd", "N-var-tall", "N-cumsum-wide", "N-cumsum-1d", "N-argmax-1d", "N-argmax-tall"}:
            # shapes off the aligned grid: short / misaligned rows, small slices, tall narrow matrices
            nr = 1 << 26
            flat = e_src
            v33 = flat.view_as_strided(0, ((nr // 33), 33), (33, 1))
            v10 = flat.view_as_strided(0, ((nr // 10), 10), (10, 1))
            vslab = flat.view_as_strided(0, (nr // 128, 8, 16), (128, 16, 1))
            o33, i33 = T("float").resize((nr // 33, 1)), T("long").resize((nr // 33, 1))
            otall, oslab = T("float").resize((1, 10)), T("float").resize((nr // 128, 1, 16))
            s10 = T("float").resize((nr // 10, 10))
            vwide = flat.view_as_strided(0, (65536, 1000), (1000, 1))
            swide = T("float").resize((65536, 1000))
            s1d = T("float").resize((nr,))
            omax1, imax1 = T("float").resize((1,)), T("long").resize((1,))
            omaxt, imaxt = T("float").resize((1, 10)), T("long").resize((1, 10))
            oddT = T.from_numpy(rng.standard_normal((8193, 8191), dtype=np.float32)).t()
            oddB = T.from_numpy(rng.standard_normal((8191, 8193), dtype=np.float32))
            oddO = T("float").resize((8191, 8193))
            n33, n10, nodd = (nr // 33) * 33, (nr // 10) * 10, 8191 * 8193
            bias = T.from_numpy(rng.standard_normal(8193, dtype=np.float32)).view_as_strided(0, (8191, 8193), (0, 1))
            table.update({
                "N-bias-odd": ("c = x + bias (stride-0 row bias), 8191x8193 fp32 (no 16-byte aligned rows)", 8 * nodd,
                               nodd, lambda i: oddO.cadd(oddB, 1.0, bias)),
                "N-sum-rows33": ("sum over last dim of 2033601x33 fp32 (misaligned short rows)", 4 * n33 + 4 * (nr // 33),
                                 n33, lambda i: o33.sum(v33, 1)),
                "N-max-rows33": ("max+argmax over last dim of 2033601x33 fp32", 4 * n33 + 12 * (nr // 33), n33,
                                 lambda i: o33.max(i33, v33, 1)),
                "N-sum-slab": ("sum over middle dim of 524288x8x16 fp32 (512-byte slices)", 4 * nr + 4 * (nr // 8), nr,
                               lambda i: oslab.sum(vslab, 1)),
                "N-sum-tall": ("sum over dim 0 of 6710886x10 fp32 (tall, 40-byte rows)", 4 * n10, n10,
                               lambda i: otall.sum(v10, 0)),
                "N-var-tall": ("var over dim 0 of 6710886x10 fp32 (one read)", 4 * n10, n10, lambda i: otall.var(v10, 0)),
                "N-cumsum-wide": ("cumsum over dim 0 of 65536x1000 fp32 (rows cut into parts, input read twice, "
                                  "counted once)", 8 * 65536 * 1000, 65536 * 1000,
                                  lambda i: swide.cumsum(vwide, 0)),
                "N-cumsum-1d": ("cumsum of a 2^26-element fp32 vector (a wave per piece, input read twice, counted once)",
                                8 * nr, nr, lambda i: s1d.cumsum(flat, 0)),
                "N-argmax-tall": ("max+argmax over dim 0 of 6710886x10 fp32", 4 * n10, n10, lambda i: omaxt.max(imaxt, v10, 0)),
                "N-argmax-1d": ("max+argmax of a 2^26-element fp32 vector", 4 * nr, nr, lambda i: omax1.max(imax1, flat, 0)),
                "N-cumsum-rows10": ("cumsum over last dim of 6710886x10 fp32", 8 * n10, n10, lambda i: s10.cumsum(v10, 1)),
                "N-cumsum-tall": ("cumsum over dim 0 of 6710886x10 fp32 (input read twice, counted once)", 8 * n10, n10,
                                  lambda i: s10.cumsum(v10, 0)),
                "N-add-t-odd": ("c = a:t() + b, 8191x8193 fp32 (no 16-byte aligned rows)", 12 * nodd, nodd,
                                lambda i: oddO.cadd(oddT, 1.0, oddB)),
            })
        if set(nx) & {"N-int-add-t", "N-lt-t"}:
            # transposed operands of ops that have no LDS-tiled kernel of their own (slab-wise densify)
            it_a = T.from_numpy(rng.integers(-1000, 1000, (8192, 8192)).astype(np.int32)).t()
            it_b = T.from_numpy(rng.integers(-1000, 1000, (8192, 8192)).astype(np.int32))
            it_c = T("int").resize((8192, 8192))
            lt_m = T("byte").resize((8192, 8192))
            table.update({
                "N-int-add-t": ("c = a:t() + b, 8192x8192 int32", 12 * 8192 * 8192, 8192 * 8192,
                                lambda i: it_c.cadd(it_a, 1, it_b)),
                "N-lt-t": ("mask = a:t() < b into a Byte tensor, 8192x8192 fp32", 9 * 8192 * 8192, 8192 * 8192,
                           lambda i: lt_m.compare_tensor("lt", sq_t, db)),
            })
        if set(nx) & {"N-half-exp", "N-half-abs-t", "N-half-exp-t", "N-half-exp-t-odd", "N-short-add-t", "N-short-add-t-odd", "N-short-neg-t", "N-int-neg-t", "N-cvt-float-t", "N-cmax-t", "N-cmax-t-odd",
                      "N-int-div-t", "N-int-lt-t", "N-cvt-half-t"}:
            # transposed operands of the op families beyond plain float arithmetic: one-input math on half,
            # narrow integer arithmetic, two-input float math, integer division, integer comparison into Byte,
            # type-converting copy
            m = 8192
            hx = T.from_numpy(rng.uniform(-2, 2, (m, m)).astype(np.float16)).t()
            ho = T("half").resize((m, m))
            hxo = T.from_numpy(rng.uniform(-2, 2, (8193, 8191)).astype(np.float16)).t()
            hoo = T("half").resize((8191, 8193))
            sa = T.from_numpy(rng.integers(-1000, 1000, (m, m)).astype(np.int16)).t()
            sb = T.from_numpy(rng.integers(-1000, 1000, (m, m)).astype(np.int16))
            sc = T("short").resize((m, m))
            ja = T.from_numpy(rng.integers(-100000, 100000, (m, m)).astype(np.int32)).t()
            jb = T.from_numpy(rng.integers(1, 1000, (m, m)).astype(np.int32))
            jc = T("int").resize((m, m))
            jm = T("byte").resize((m, m))
            fo = T("float").resize((m, m))
            hc = T("half").resize((m, m))
            sa_odd = T.from_numpy(rng.integers(-1000, 1000, (8193, 8191)).astype(np.int16)).t()
            sb_odd = T.from_numpy(rng.integers(-1000, 1000, (8191, 8193)).astype(np.int16))
            so_odd = T("short").resize((8191, 8193))
            fa_odd = T.from_numpy(rng.standard_normal((8193, 8191), dtype=np.float32)).t()
            fb_odd = T.from_numpy(rng.standard_normal((8191, 8193), dtype=np.float32))
            fo_odd = T("float").resize((8191, 8193))
            table.update({
                "N-half-exp": ("out = exp(a), 8192x8192 fp16 contiguous (the flat form of N-half-exp-t)", 4 * m * m, m * m,
                               lambda i: ho.unary("exp", hc)),
                "N-half-abs-t": ("out = abs(a:t()), 8192x8192 fp16", 4 * m * m, m * m, lambda i: ho.unary("abs", hx)),
                "N-half-exp-t": ("out = exp(a:t()), 8192x8192 fp16", 4 * m * m, m * m, lambda i: ho.unary("exp", hx)),
                "N-half-exp-t-odd": ("out = exp(a:t()), 8191x8193 fp16 (no 16-byte aligned rows)", 4 * nodd_,
                                     nodd_, lambda i: hoo.unary("exp", hxo)),
                "N-short-add-t": ("c = a:t() + b, 8192x8192 int16", 6 * m * m, m * m, lambda i: sc.cadd(sa, 1, sb)),
                "N-cmax-t": ("c = cmax(a:t(), b), 8192x8192 fp32", 12 * m * m, m * m,
                             lambda i: fo.binary("cmax", sq_t, db)),
                "N-short-neg-t": ("out = -a:t(), 8192x8192 int16", 4 * m * m, m * m, lambda i: sc.unary("neg", sa)),
                "N-int-neg-t": ("out = -a:t(), 8192x8192 int32", 8 * m * m, m * m, lambda i: jc.unary("neg", ja)),
                "N-cvt-float-t": ("float <- half converting copy of a:t(), 8192x8192", 6 * m * m, m * m,
                                  lambda i: fo.copy_from(hx)),
                "N-short-add-t-odd": ("c = a:t() + b, 8191x8193 int16 (no 16-byte aligned rows)", 6 * nodd_, nodd_,
                                      lambda i: so_odd.cadd(sa_odd, 1, sb_odd)),
                "N-cmax-t-odd": ("c = cmax(a:t(), b), 8191x8193 fp32 (no 16-byte aligned rows)", 12 * nodd_, nodd_,
                                 lambda i: fo_odd.binary("cmax", fa_odd, fb_odd)),
                "N-int-div-t": ("c = a:t() / b, 8192x8192 int32 (truncating division)", 12 * m * m, m * m,
                                lambda i: jc.cdiv(ja, jb)),
                "N-int-lt-t": ("mask = a:t() < b into a Byte tensor, 8192x8192 int32", 9 * m * m, m * m,
                               lambda i: jm.compare_tensor("lt", ja, jb)),
                "N-cvt-half-t": ("half <- float converting copy of a:t(), 8192x8192", 6 * m * m, m * m,
                                 lambda i: hc.copy_from(sq_t)),
            })
        if set(nx) & {"N-add-strided", "N-add-strided-u64"}:
            # an operand with no unit-stride dim (every second column of a 8192 x 16384 buffer): the indexed
            # kernel, one division chain per element; with 32-bit and with 64-bit index arithmetic (the latter
            # is what operands beyond 2^31 elements take when no tiled kernel fits them)
            m = 8192
            st_buf = T.from_numpy(rng.standard_normal((m, 2 * m), dtype=np.float32))
            st_a = st_buf.view_as_strided(0, (m, m), (2 * m, 2))
            st_o = T("float").resize((m, m))

            def strided_add(force):
                def run(i):
                    thc.force_64bit_index(force)
                    st_o.cadd(st_a, 1.0, db)
                    thc.force_64bit_index(False)
                return run
            table["N-add-strided"] = ("c = a + b, 8192x8192 fp32, a = every second column of a 8192x16384 buffer "
                                      "(32-bit offsets; a's lines are half used)", 12 * m * m, m * m, strided_add(False))
            table["N-add-strided-u64"] = ("the same with 64-bit index arithmetic forced", 12 * m * m, m * m,
                                          strided_add(True))
        if set(nx) & {"N-copy-nhwc3", "N-copy-skinny16", "N-cvt-image", "N-transpose-16x16"}:
            # tall-and-skinny transposes: a short dim of a few elements against a long one
            img = T.from_numpy(rng.standard_normal((64, 3, 512, 512), dtype=np.float32))
            nhwc_view = img.view_as_strided(0, (64, 512, 512, 3), (3 * 262144, 512, 1, 262144))
            nhwc = T("float").resize((64, 512, 512, 3))
            sk_src = T.from_numpy(rng.standard_normal((16, 1 << 22), dtype=np.float32)).t()
            sk_dst = T("float").resize((1 << 22, 16))
            table["N-copy-nhwc3"] = ("NCHW -> NHWC copy of 64x3x512x512 fp32", 8 * 64 * 3 * 262144, 64 * 3 * 262144,
                                     lambda i: nhwc.copy(nhwc_view))
            img8 = T.from_numpy(rng.integers(0, 256, (64, 512, 512, 3)).astype(np.uint8))          # NHWC bytes
            chw_view = img8.view_as_strided(0, (64, 3, 512, 512), (3 * 262144, 1, 1536, 3))
            chw = T("float").resize((64, 3, 512, 512))
            table["N-cvt-image"] = ("float NCHW <- byte NHWC converting copy of 64x512x512x3", 5 * 64 * 3 * 262144,
                                    64 * 3 * 262144, lambda i: chw.copy_from(chw_view))
            small = T.from_numpy(rng.standard_normal((1 << 18, 16, 16), dtype=np.float32))
            small_t = small.view_as_strided(0, (1 << 18, 16, 16), (256, 1, 16))
            small_o = T("float").resize((1 << 18, 16, 16))
            table["N-transpose-16x16"] = ("2^18 transposed 16 x 16 fp32 matrices copied", 8 * (1 << 26), 1 << 26,
                                          lambda i: small_o.copy(small_t))
            table["N-copy-skinny16"] = ("(2^22, 16) <- (16, 2^22):t() copy, fp32", 8 * (1 << 26), 1 << 26,
                                        lambda i: sk_dst.copy(sk_src))
        if "N-add-view-odd" in nx:
            # views whose rows start off the 16-byte grid and have an odd length: x[:, 3:8190] of wider matrices
            vw = [T.from_numpy(rng.standard_normal((8192, 8200), dtype=np.float32)) for _ in range(3)]
            va, vb, vc = (w.narrow(1, o, 8187) for w, o in zip(vw, (3, 1, 2)))
            table["N-add-view-odd"] = ("c = a + b on 8192x8187 fp32 views of 8192x8200 matrices at column offsets 2, 3, 1",
                                       12 * 8192 * 8187, 8192 * 8187, lambda i: vc.cadd(va, 1.0, vb))
        if "N-std-rows8192" in nx:
            std_o = T("float").resize((8192, 1))
            table["N-std-rows8192"] = ("std over last dim of 8192x8192 fp32 (rows beyond a lane group's registers, one read)",
                                       4 * 8192 * 8192 + 4 * 8192, 8192 * 8192, lambda i: std_o.std(sq, 1))
        if "N-sumall-t" in nx:
            table["N-sumall-t"] = ("sumall over the transposed view of 8192x8192 fp32 (blocks on the scalar)", 4 * 8192 * 8192,
                                   8192 * 8192, lambda i: sq_t.sumall())
        if "N-equal" in nx:
            eq_b = e_src.clone()
            table["N-equal"] = ("equal(a, b) over 2^26 fp32 (both equal: no early exit possible)", 8 * ne, ne,
                                lambda i: e_src.equal(eq_b))
        for tag, lg in (("64M", 24), ("256M", 26), ("1G", 28)):
            if "N-copy-contig-" + tag in nx:
                m = 1 << lg
                cc_src = T.from_numpy(rng.uniform(-1, 1, m).astype(np.float32))
                cc_dst = [T("float").resize((m,)) for _ in range(3)]
                table["N-copy-contig-" + tag] = (
                    "dst:copy(src), 2^%d fp32 contiguous, 3 rotating destinations" % lg, 8 * m, m,
                    (lambda q, src_: lambda i: q[i % 3].copy(src_))(cc_dst, cc_src))
        if set(nx) & {"N-add-2p25", "N-add-2p26"}:
            # c = a + b as in C1 at two and four times the size (rotating sets): kernel time against
            # bytes gives the fixed cost of a launch (t = t0 + bytes / BW)
            for lg, nset in ((25, 3), (26, 3)):
                m = 1 << lg
                ss = [(T.from_numpy(rng.uniform(-1, 1, m).astype(np.float32)),
                       T.from_numpy(rng.uniform(-1, 1, m).astype(np.float32)), T("float").resize((m,)))
                      for _ in range(nset)]
                table["N-add-2p%d" % lg] = ("c = a + b, 2^%d fp32 contiguous, %d rotating sets" % (lg, nset), 12 * m, m,
                                            (lambda q, k: lambda i: q[i % k][2].cadd(q[i % k][0], 1.0, q[i % k][1]))(ss, nset))
        if set(nx) & {"CEIL-copy-rot", "CEIL-3r1w-rot"}:
            # What flat kernels reach on the same stream shapes (the ceilings the strided configurations are
            # judged against): a 1-read-1-write stream and the 3-read-1-write stream of C2 without the
            # transposition, outputs rotating so that no write is absorbed by the memory-side cache.
            cr_out = [T("float").resize((ne,)) for _ in range(4)]
            table["CEIL-copy-rot"] = ("out = src + 0, 2^26 fp32 contiguous, 4 rotating outputs", 8 * ne, ne,
                                      lambda i: cr_out[i % 4].add(e_src, 0.0))
            table["CEIL-3r1w-rot"] = ("out = a*b + d, 8192x8192 fp32, all contiguous, out and d rotate over 3 sets",
                                      16 * n2 * n2, n2 * n2, lambda i: out2[i % 3].addcmul(dd[i % 3], 1.0, da, db))
        if "N-fill" in nx and xa.numel() != big:
            table["N-fill"] = ("fill of 2^26 fp32", 4 * ne, ne, lambda i: e_dst.fill(0.5))
        for n in nx:
            d, nb, el, fn = table[n]
            cfgs.append(Config(n, d, nb, el, 1, fn))

    return [c for c in cfgs if want(c.name)], host


def time_config(hip, thc, cfg, steps, warmup, stream):
    """Runs `steps` timed launches. Returns (wall seconds, event ms for the
    whole region, per-step event ms of a second, separately instrumented
    pass). The region-level events bracket the K launches on the engine's
    stream, so event_ms / K is the average launch duration including the gaps
    between back-to-back launches; the per-step pass gives min/median."""
    for i in range(warmup):
        cfg.run(i)
    hip.sync()
    cfg.kernel = thc.last_kernel()
    e0, e1 = hip.event(), hip.event()
    hip.sync()
    t0 = time.perf_counter()
    hip.record(e0, stream)
    for i in range(steps):
        cfg.run(warmup + i)
    hip.record(e1, stream)
    hip.sync()
    wall = time.perf_counter() - t0
    region_ms = hip.elapsed_ms(e0, e1)
    evs = [(hip.event(), hip.event()) for _ in range(steps)]
    for i in range(steps):
        hip.record(evs[i][0], stream)
        cfg.run(warmup + steps + i)
        hip.record(evs[i][1], stream)
    hip.sync()
    ms = np.array([hip.elapsed_ms(a, b) for a, b in evs])
    return wall, region_ms, ms


def cpu_baseline(host, cfg_bytes, budget_s=24.0):
    """Times the CPU restatement on this box's host cores, single thread and all
    cores: a 1/16 sample of the headline workload (c = a + b with a seen through
    permute(3,2,1): 2048 x 2048 x 32 of the 520 planes, the same strides), the
    strided apply3 out = a:t()*b + d on the full 8192x8192 operands
    (TH_TENSOR_APPLY path) and, for the reduction path, the row sums of
    65536x1024 and the middle-dim sums of 64x4096x512. Every figure is the
    median of the runs after the first, GB/s on the algorithmic bytes."""
    from oracle import th_oracle as oracle
    cores = len(os.sched_getaffinity(0))
    jobs = []
    nbytes = dict(cfg_bytes)
    if "C5" in host and "C5" in cfg_bytes:
        block, rblock = host["C5"]
        k5 = 32
        n5 = 2048 * 2048 * k5
        ha, hb = np.resize(block, n5), np.resize(rblock, n5)
        va = oracle.View(ha, 0, (2048, 2048, k5), (1, 2048, 2048 * 2048))
        vb, vc = oracle.View(hb, 0, (2048, 2048, k5)), oracle.View.empty((2048, 2048, k5))
        jobs.append(("C5", 0.3, lambda: oracle.pointwise("cadd", vc, va, vb, value=1.0)))
        nbytes["C5"] = 12 * n5
    if "C2" in host and "C2" in cfg_bytes:
        a, b, d = host["C2"]
        n = a.shape[0]
        va2 = oracle.View(a.reshape(-1), 0, (n, n), (1, n))
        vb2, vd2 = oracle.View(b.reshape(-1), 0, (n, n)), oracle.View(d.reshape(-1), 0, (n, n))
        out2 = oracle.View.empty((n, n))
        jobs.append(("C2", 0.3, lambda: oracle.pointwise("addcmul", out2, vd2, va2, vb2, value=1.0)))
    if host.get("C3a-sum") is not None and "C3a-sum" in cfg_bytes:
        x = host["C3a-sum"]
        vx, o3 = oracle.View(x.reshape(-1), 0, x.shape), oracle.View.empty((x.shape[0], 1))
        jobs.append(("C3a-sum", 0.15, lambda: oracle.reduce_dim("sum", vx, 1, out=o3)))
    if host.get("C4-sum-f32") is not None and host["C4-sum-f32"].size > 64 and "C4-sum-f32" in cfg_bytes:
        x4 = host["C4-sum-f32"]
        v4, o4 = oracle.View(x4.reshape(-1), 0, x4.shape), oracle.View.empty((x4.shape[0], 1, x4.shape[2]))
        jobs.append(("C4-sum-f32", 0.25, lambda: oracle.reduce_dim("sum", v4, 1, out=o4)))
    res = {}
    for name, share, fn in jobs:
        res[name] = {}
        for label, threads, part in (("single", 1, 0.7), ("all", cores, 0.3)):
            oracle.set_num_threads(threads)
            times, t_start = [], time.perf_counter()
            while len(times) < 26 and (len(times) < 3 or time.perf_counter() - t_start < budget_s * share * part):
                t0 = time.perf_counter()
                fn()
                times.append(time.perf_counter() - t0)
            res[name][label] = (nbytes[name] / float(np.median(times[1:])) / 1e9, threads, len(times) - 1)
    oracle.set_num_threads(1)
    return res


def call_latency(thc, hip, calls=2000):
    """Host-side cost of small calls (entry point, planning, launch): microseconds per call with the
    queue left to fill (calls back to back, one wait at the end) and with the stream drained after every
    call (launch + completion). "ctypes_us" is what the Python binding itself costs per call (an entry
    point that does nothing), to be subtracted."""
    T = thc.Tensor
    rng = np.random.default_rng(7)
    a = T.from_numpy(rng.standard_normal(1024).astype(np.float32))
    b = T.from_numpy(rng.standard_normal(1024).astype(np.float32))
    c = T("float").resize((1024,))
    m = T.from_numpy(rng.standard_normal((64, 64)).astype(np.float32))
    o, ix = T("float").resize((64, 1)), T("long").resize((64, 1))
    st = thc.state()
    noop = thc.lib().THCState_getCurrentStream
    cases = {"cadd_1k": lambda: c.cadd(a, 1.0, b), "sum_64x64": lambda: o.sum(m, 1), "max_64x64": lambda: o.max(ix, m, 1)}
    out = {}
    t0 = time.perf_counter()
    for _ in range(calls):
        noop(st)
    out["ctypes_us"] = round((time.perf_counter() - t0) / calls * 1e6, 2)
    for name, fn in cases.items():
        for _ in range(50):
            fn()
        hip.sync()
        t0 = time.perf_counter()
        for _ in range(calls):
            fn()
        t_issue = time.perf_counter() - t0
        hip.sync()
        t_all = time.perf_counter() - t0
        t1 = time.perf_counter()
        for _ in range(calls // 4):
            fn()
            hip.sync()
        t_drained = time.perf_counter() - t1
        out[name + "_queued_us"] = round(t_issue / calls * 1e6, 2)
        out[name + "_queued_incl_drain_us"] = round(t_all / calls * 1e6, 2)
        out[name + "_drained_us"] = round(t_drained / (calls // 4) * 1e6, 2)
    return out


def flat_key(name):
    return name.replace("-", "_")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--configs", default="bar", choices=["bar", "all", "primary"],
                    help="bar: the benchmark configurations + calibration stream (default); all: also the "
                         "neighbouring ops (N-*) and full detail; primary: the headline only")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-check", action="store_true", help="skip the per-configuration parity checks")
    ap.add_argument("--only", default="", help="comma-separated config names to measure (the first one "
                                               "built becomes the line's headline)")
    ap.add_argument("--tune", action="append", default=[], help="engine tuning knob key=value")
    ap.add_argument("--stagger", type=int, default=0, help="probe: C1's second input and its output start this many / twice "
                                                           "this many elements into their allocations (a multiple of 4)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this engine has no multi-GPU path (run with --gpus 1)")

    import cutorch_amd as thc
    thc.state()                      # raises if libTHC.so is missing or no GPU is visible
    hip = Hip()
    stream = thc.lib().THCState_getCurrentStream(thc.state())
    for kv in args.tune:
        k, v = kv.split("=")
        thc.set_tuning(k, int(v))
    only = set(args.only.split(",")) if args.only else None
    cfgs, host = build_configs(thc, hip, args.configs, only, args.stagger)
    if not cfgs:
        sys.exit("no configuration selected")
    results = []
    for cfg in cfgs:
        steps = args.steps
        wall, region_ms, ms = time_config(hip, thc, cfg, steps, args.warmup, stream)
        ok = None if (args.no_check or cfg.check is None) else bool(cfg.check())
        mean_ms = region_ms / steps
        results.append({
            "name": cfg.name, "desc": cfg.desc, "kernel": cfg.kernel, "steps": steps,
            "algorithmic_bytes": cfg.nbytes,
            "ms_mean": round(mean_ms, 5), "ms_min": round(float(ms.min()), 5),
            "ms_median": round(float(np.median(ms)), 5),
            "gbps_mean": round(cfg.nbytes / mean_ms / 1e6, 1),
            "gbps_best": round(cfg.nbytes / float(ms.min()) / 1e6, 1),
            "frac_of_peak": round(cfg.nbytes / mean_ms / 1e6 / PEAK_GBPS, 4),
            "gelem_per_s": round(cfg.elements / mean_ms / 1e6, 2),
            "wall_gbps": round(cfg.nbytes * steps / wall / 1e9, 1),
            "rotating_sets": cfg.sets, "parity_ok": ok, "note": cfg.note,
        })
    p = results[0]
    traffic, traffic_src = None, None   # HBM bytes per launch from the committed rocprofv3 --pmc summary
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            measured = json.load(f)
        traffic = measured.get(p["name"], {}).get("traffic_bytes")
        traffic_src = "profiles/traffic.json (committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary; not measured in this run)"
        for r in results:
            r["traffic_bytes"] = measured.get(r["name"], {}).get("traffic_bytes")
    except (OSError, ValueError):
        pass
    compact = {}
    for r in results:
        compact[r["name"]] = {"frac": r["frac_of_peak"], "us": round(1e3 * r["ms_mean"], 2),
                              "us_min": round(1e3 * r["ms_min"], 2), "gbps": r["gbps_mean"],
                              "gelem_s": r["gelem_per_s"], "parity": r["parity_ok"], "kernel": r["kernel"],
                              "sets": r["rotating_sets"]}
        if r["note"]:
            compact[r["name"]]["note"] = r["note"]
    roof = {"bound": "hbm", "achieved": p["gbps_mean"], "peak": PEAK_GBPS, "unit": "GB/s",
            "frac": p["frac_of_peak"], "traffic": traffic, "traffic_source": traffic_src}
    # the same per configuration as flat scalars (a parser that keeps scalars only still sees them)
    bar = [r for r in results if r["name"][0] == "C" and r["name"][1].isdigit() and r["name"] != "C2-fixed"]
    for r in results:
        roof["frac_" + flat_key(r["name"])] = r["frac_of_peak"]
        roof["us_" + flat_key(r["name"])] = round(1e3 * r["ms_mean"], 2)
        if r["parity_ok"] is not None:
            roof["parity_" + flat_key(r["name"])] = r["parity_ok"]
    if bar:
        worst = min(bar, key=lambda r: r["frac_of_peak"])
        roof["frac_min"] = worst["frac_of_peak"]
        roof["frac_min_config"] = worst["name"]
        checked = [r["parity_ok"] for r in bar if r["parity_ok"] is not None]
        roof["parity_all"] = bool(checked) and all(checked)
    roof["configs"] = compact
    line = {
        "metric": METRIC, "value": p["wall_gbps"], "unit": "GB/s", "n_gpus": 1,
        "steps": p["steps"], "warmup": args.warmup,
        "ms_per_step": round(1e3 * p["algorithmic_bytes"] / (p["wall_gbps"] * 1e9), 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (fixed-seed host generator, copied to HBM before timing)",
        "config": {"workload": p["desc"], "name": p["name"], "elements": cfgs[0].elements, "kernel": p["kernel"],
                   "parity_ok": p["parity_ok"], "note": p["note"]},
        "roofline": roof,
    }
    if args.configs != "primary" and not only:
        line["latency"] = call_latency(thc, hip)
    if not args.no_cpu:
        cb = cpu_baseline(host, {c.name: c.nbytes for c in cfgs})
        per = {}
        head = cb.get(p["name"])
        base = {"value": round(head["single"][0], 2) if head else None, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": ("1/16 of the headline workload: c = a + b on 2048x2048x32 fp32 with a seen through "
                           "permute(3,2,1) (the same strides, 32 of the 520 planes; 1.6 GB of traffic per run), "
                           "median of %d runs" % head["single"][2]) if head and p["name"] == "C5" else
                          ("the %s workload at full size, median of %d runs" % (p["name"], head["single"][2]) if head else None)}
        for name, r in cb.items():
            per[name] = {"single_gbps": round(r["single"][0], 2), "all_cores_gbps": round(r["all"][0], 2),
                         "cores": r["all"][1], "runs": [r["single"][2], r["all"][2]]}
            base[flat_key(name) + "_single_gbps"] = round(r["single"][0], 2)
            base[flat_key(name) + "_all_cores_gbps"] = round(r["all"][0], 2)
            base["all_cores"] = r["all"][1]
        base["configs"] = per
        line["cpu_baseline"] = base
    if args.configs == "all":
        line["all_configs"] = results
    print(json.dumps(line))


if __name__ == "__main__":
    main()
