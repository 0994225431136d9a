"""The host library's load-time code under AddressSanitizer and UndefinedBehaviorSanitizer:
tests/host_sanitize_driver.cpp is compiled together with the host sources and run as a child
process (host code only; no GPU call is made)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "reinstinct_amd", "csrc", "host")


def test_load_time_code_is_clean_under_asan_and_ubsan(tmp_path):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no g++")
    exe = str(tmp_path / "host_sanitize_driver")
    srcs = [os.path.join(ROOT, "tests", "host_sanitize_driver.cpp")] + \
           [os.path.join(HOST, f) for f in sorted(os.listdir(HOST)) if f.endswith(".cpp")]
    build = subprocess.run([gxx, "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                            "-pthread", *srcs, "-ldl", "-o", exe], capture_output=True, text=True, timeout=300)
    if build.returncode != 0 and ("asan" in build.stderr or "ubsan" in build.stderr):
        pytest.skip("sanitizer runtimes are not installed")
    assert build.returncode == 0, build.stderr[-2000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0")
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    if "ASan runtime does not come first" in run.stderr:
        pytest.skip("another preloaded library keeps the ASan runtime from coming first in this environment")
    assert run.returncode == 0, (run.stdout + run.stderr)[-3000:]
    assert run.stdout.strip().startswith("ok ")
