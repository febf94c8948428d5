"""The scratch-buffer cache of the device library (leases, growth, eviction,
release) as pure policy, compiled for the CPU with a counting allocator: no
GPU involved."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_scratch_cache_policy(tmp_path):
    exe = str(tmp_path / "scratch_cache_check")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-g", "-pthread", "-fsanitize=address,undefined",
                           "-I", os.path.join(ROOT, "iree_amd", "csrc"),
                           os.path.join(ROOT, "tests", "cpp", "scratch_cache_check.cc"), "-o", exe])
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    sys.stderr.write(out.stderr)
    assert out.returncode == 0 and out.stdout.strip() == "ok"
