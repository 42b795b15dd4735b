"""The host core under AddressSanitizer and UndefinedBehaviorSanitizer (host code only, on the
CPU): tests/native/host_core_stress.cpp drives allocator, managers, prefix cache, scheduler and
batch builder with random workloads under page pressure."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("g++") is None, reason="no host compiler")
def test_host_core_stress_under_sanitizers(tmp_path):
    exe = str(tmp_path / "host_core_stress")
    src = [os.path.join(ROOT, "tests", "native", "host_core_stress.cpp"),
           os.path.join(ROOT, "kv-cache-manager_amd", "csrc", "host", "capi.cpp")]
    build = subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                            "-fno-omit-frame-pointer", *src, "-o", exe], capture_output=True, text=True, timeout=300)
    assert build.returncode == 0, build.stderr[-3000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    assert run.returncode == 0, (run.stdout[-2000:], run.stderr[-4000:])
    assert "host core stress: ok" in run.stdout
