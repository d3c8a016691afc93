"""Block bookkeeping of the caching allocator (cutorch_amd/csrc/caching_pool.hpp)
on the host: best fit per stream, split and merge, event-guarded reuse after
cross-stream use, release on out-of-memory (lib/THC/THCCachingAllocator.cpp:108-330
is the role). The pool is compiled against a fake device, with the host
sanitizers on, and driven by tests/allocator_host_test.cpp."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_caching_pool_on_a_fake_device(tmp_path):
    exe = str(tmp_path / "allocator_host_test")
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined",
                    "-fno-sanitize-recover=all", "-I", os.path.join(ROOT, "cutorch_amd", "csrc"),
                    os.path.join(ROOT, "tests", "allocator_host_test.cpp"), "-o", exe], check=True)
    res = subprocess.run([exe], capture_output=True, text=True)
    assert res.returncode == 0 and res.stdout.strip() == "ok", res.stdout + res.stderr
