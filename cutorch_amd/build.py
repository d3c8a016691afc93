"""Build libTHC.so (HIP, gfx950) in-tree: `python -m cutorch_amd.build`.

hipcc cross-compiles without a GPU. Objects go to cutorch_amd/build/, the
library to cutorch_amd/libTHC.so. Flags that matter for results:
  -ffp-contract=off   a*b+c stays two roundings, as on the CPU path
  -packed-fp32-ops    off (v_pk_*_f32 forms are not relied upon)
Correctly rounded fp32 divide/sqrt and denormal support are hipcc defaults
and are left on.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
BUILD = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libTHC.so")
SOURCES = ["general.cpp", "tensor.cpp", "math.cpp", "math_wide.cpp", "caching_allocator.cpp", "apply.hip", "apply_f32_0.hip", "apply_f32_1.hip",
           "apply_f32_2.hip", "apply_f16_0.hip", "apply_f16_1.hip", "apply_f16_2.hip", "apply_raw.hip",
           "reduce.hip", "reduce_f32.hip", "reduce_f16.hip", "reduce_w_u8.hip", "reduce_w_i8.hip",
           "reduce_w_i16.hip", "reduce_w_i32.hip", "reduce_w_i64.hip", "reduce_w_f64.hip", "scan.hip", "no_alloc.hip", "convert.hip", "apply_cmp_f.hip", "apply_w_u8.hip",
           "apply_rawmath_u32u64.hip", "apply_rawmath_f64.hip", "apply_w_i8.hip", "apply_w_i16.hip", "apply_w_i32.hip", "apply_w_i64.hip", "apply_w_f64.hip",
           "apply_cvt_u8.hip", "apply_cvt_i8.hip", "apply_cvt_i16.hip", "apply_cvt_i32.hip", "apply_cvt_i64.hip",
           "apply_cvt_f16.hip", "apply_cvt_f32.hip", "apply_cvt_f64.hip", "apply_policy.hip"]
HEADERS = ["common.hpp", "layout.hpp", "device_util.hpp", os.path.join("..", "..", "include", "THC.h")]   # every source
APPLY_HEADERS = ["apply_plan.hpp", "apply_impl.hpp", "apply_ldstile.hpp", "apply_wide.hpp"]   # apply*.hip, convert.hip
REDUCE_HEADERS = ["reduce_plan.hpp", "reduce_impl.hpp"]                                       # reduce*.hip, scan.hip, no_alloc.hip

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-pragmas", "-Wno-pass-failed",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


# headers only some sources include (touching one rebuilds only those)
EXTRA_DEPS = {"caching_allocator.cpp": ["caching_pool.hpp", "stream_guard.hpp"],
              "general.cpp": ["stream_guard.hpp"], "tensor.cpp": ["stream_guard.hpp"],
              "apply.hip": ["stream_guard.hpp", "apply_rawmath.hpp"],
              "apply_rawmath_u32u64.hip": ["apply_rawmath.hpp", "apply_rawmath_impl.hpp"],
              "apply_rawmath_f64.hip": ["apply_rawmath.hpp", "apply_rawmath_impl.hpp"], "reduce.hip": ["stream_guard.hpp"],
              "scan.hip": ["stream_guard.hpp"], "no_alloc.hip": ["stream_guard.hpp"], "convert.hip": ["stream_guard.hpp"]}
EXTRA_DEPS.update({"apply_cvt_%s.hip" % t: ["apply_convert_impl.hpp", "apply_skinny.hpp"]
                   for t in ("u8", "i8", "i16", "i32", "i64", "f16", "f32", "f64")})
EXTRA_DEPS["apply_raw.hip"] = ["apply_skinny.hpp"]


def _compile(src, force):
    obj = os.path.join(BUILD, src + ".o")
    group = APPLY_HEADERS if src.startswith(("apply", "convert")) else (
        REDUCE_HEADERS if src.startswith(("reduce", "scan", "no_alloc")) else [])
    deps = [os.path.join(CSRC, src)] + [os.path.join(CSRC, h) for h in HEADERS + group + EXTRA_DEPS.get(src, [])]
    only = os.environ.get("THC_BUILD_ONLY")   # development aid: rebuild just these sources, reuse every other object as it is
    if only and os.path.exists(obj) and src not in only.split(","):
        return obj
    if not force and not _stale(obj, deps):
        return obj
    cmd = [_hipcc(), "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj] + FLAGS
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass does not know the packed-fp32 feature name; harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, res.stderr))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force=False, verbose=True):
    os.makedirs(BUILD, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 4)) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), SOURCES))
    if force or _stale(LIB, objs):
        cmd = [_hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("link failed:\n" + res.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
