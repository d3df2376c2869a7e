"""Helper-level unit tests (the reference's UT tier, tests/train/flash_attention/ut/): the integer index
arithmetic of the kernels -- workgroup map, LDS swizzles, head-dim classes, the dK/dV query split -- lives in
a header without HIP in it, so a host compiler builds the checks and they run without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_index_math_host_build(tmp_path):
    src = os.path.join(ROOT, "tests", "host", "index_math_test.cpp")
    exe = str(tmp_path / "index_math_test")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-o", exe, src], check=True)
    res = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    sys.stdout.write(res.stdout)
    assert res.returncode == 0, res.stdout[-2000:]
    assert "all checks passed" in res.stdout
