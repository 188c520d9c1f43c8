"""The library's integer logic (kernel choice, tile numbering, row-block lookup, workspace layout, arrival-counter
bookkeeping, placement tables) built for the host with g++ and run under the address and undefined-behaviour
sanitizers.  The checks themselves are in tests/host/host_logic_test.cpp."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "host", "host_logic_test.cpp")


@pytest.mark.skipif(shutil.which("g++") is None, reason="g++ not available")
def test_host_logic_under_sanitizers(tmp_path):
    exe = str(tmp_path / "host_logic_test")
    build = subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                            "-static-libasan", "-static-libubsan", "-pthread", SRC, "-o", exe], capture_output=True, text=True, cwd=ROOT)
    assert build.returncode == 0, build.stderr
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=1", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "all checks passed" in run.stdout
