"""The host library under the address and undefined-behaviour sanitizers (no GPU): a driver in
C++ runs random allocations, steps and releases against a model of plain containers."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BOOKS = os.path.join(os.path.dirname(HERE), "torchless_rs_amd", "csrc", "host", "books.cpp")


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_books_and_packer_under_sanitizers(tmp_path):
    exe = str(tmp_path / "driver")
    build = subprocess.run(["g++", "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined",
                            "-fno-sanitize-recover=all", "-static-libasan", BOOKS,
                            os.path.join(HERE, "host_books_driver.cpp"), "-o", exe],
                           capture_output=True, text=True, timeout=300)
    if build.returncode != 0 and "sanitize" in build.stderr:
        pytest.skip("this compiler has no sanitizer runtime: " + build.stderr[-200:])
    assert build.returncode == 0, build.stderr[-2000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0")
    for seed in ("1", "2", "3", "4"):
        r = subprocess.run([exe, seed], capture_output=True, text=True, timeout=120, env=env)
        assert r.returncode == 0 and r.stdout.strip() == "ok", (seed, r.stdout[-500:], r.stderr[-2000:])
