"""The host side of the library (packer, layouts) under AddressSanitizer and UndefinedBehaviorSanitizer:
a small C++ driver is compiled together with eet_amd/csrc/packer.cc and run.  Host code only."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CLANG = os.environ.get("EET_HOST_CLANG", "/opt/rocm/llvm/bin/clang++")


@pytest.mark.skipif(not os.path.exists(CLANG), reason="ROCm's clang++ (with the sanitizer runtimes) is not installed")
def test_packer_under_asan_ubsan(tmp_path):
    exe = str(tmp_path / "host_sanitize")
    cmd = [CLANG, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-pthread",
           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "eet_amd", "csrc"),
           os.path.join(HERE, "host_sanitize_driver.cc"), os.path.join(ROOT, "eet_amd", "csrc", "packer.cc"),
           "-o", exe]
    build = subprocess.run(cmd, capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-2000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    run = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=300)
    assert run.returncode == 0, (run.stdout + run.stderr)[-3000:]
    assert "host sanitizer run ok" in run.stdout
