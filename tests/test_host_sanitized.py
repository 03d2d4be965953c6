"""The host library (csrc/host_core.cpp, csrc/step_program.cpp) under AddressSanitizer and UBSan on the CPU: see
tests/native/host_sanitized.cpp."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "infernum_amd", "csrc")


def test_host_library_under_the_sanitizers(tmp_path):
    cxx = shutil.which("g++") or shutil.which("clang++")
    if cxx is None:
        pytest.skip("no C++ compiler")
    exe = str(tmp_path / "host_sanitized")
    cmd = [cxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
           "-fno-omit-frame-pointer", os.path.join(ROOT, "tests", "native", "host_sanitized.cpp"),
           os.path.join(CSRC, "host_core.cpp"), os.path.join(CSRC, "step_program.cpp"), "-o", exe]
    build = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    if build.returncode != 0 and "sanitize" in build.stderr and "cannot find" in build.stderr:
        pytest.skip("the sanitizers' runtime libraries are not installed")
    assert build.returncode == 0, build.stderr[-4000:]
    env = dict(os.environ)
    # the sanitizer's runtime wants to be the first library of the process; where the environment preloads another
    # one, it is told not to insist
    env["ASAN_OPTIONS"] = "detect_leaks=1:verify_asan_link_order=0"
    run = subprocess.run([exe], capture_output=True, text=True, timeout=600, env=env)
    assert run.returncode == 0, (run.stdout + run.stderr)[-6000:]
    assert "host library: ok" in run.stdout
