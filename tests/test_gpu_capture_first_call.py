"""A process whose first layer call is recorded into a HIP graph: the once-per-process look-ups of the library happen
inside the capture.  Each case runs tests/capture_first_call.py in a process of its own (one at a time)."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("entry", ["layer", "routed"])
def test_first_call_of_a_process_under_capture(entry):
    res = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "capture_first_call.py"), entry], capture_output=True,
                         text=True, timeout=280, cwd=ROOT)
    assert res.returncode == 0, f"stdout:\n{res.stdout[-2000:]}\nstderr:\n{res.stderr[-3000:]}"
    assert f"capture-first-call {entry} OK" in res.stdout
