"""Builds the mini-executor's sources with AddressSanitizer and
UndefinedBehaviorSanitizer (host code only) and runs a scenario on the CPU
mock device."""
import os
import subprocess

from polarai_framework_amd import PACKAGE_DIR, REPO_ROOT


def test_harness_under_asan_ubsan(tmp_path):
    src = os.path.join(PACKAGE_DIR, "harness")
    exe = str(tmp_path / "harness_sanitized")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fno-omit-frame-pointer",
           "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-I" + os.path.join(REPO_ROOT, "include"), "-I" + src, "-I" + os.path.join(PACKAGE_DIR, "host"),
           os.path.join(REPO_ROOT, "tests", "native", "harness_sanitized.cpp"),
           os.path.join(src, "coherent_allocator.cpp"), os.path.join(src, "support_routines.cpp"),
           os.path.join(src, "mini_executor.cpp"), os.path.join(src, "support_factory.cpp"), "-ldl", "-lpthread", "-o", exe]
    subprocess.run(cmd, check=True, capture_output=True, text=True, timeout=300)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:verify_asan_link_order=0")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120, env=env)
    assert r.returncode == 0, r.stderr[-3000:]
    assert r.stdout.strip() == "ok"
