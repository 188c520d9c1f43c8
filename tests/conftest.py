import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _announce(request):
    # name the case before it touches the GPU, flushed, so a dead box still tells which one ran
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield


@pytest.fixture
def tuning(monkeypatch):
    """Sets OMNI_MOE_* tuning variables for one test.  The library reads them once per process, so every
    change is followed by omni_moe_reload_tuning(), and the defaults are restored the same way afterwards."""
    from omni_infer_amd import _lib as L

    def set_vars(**kv):
        for k, v in kv.items():
            if v is None:
                monkeypatch.delenv(k, raising=False)
            else:
                monkeypatch.setenv(k, str(v))
        L.lib().omni_moe_reload_tuning()

    yield set_vars
    monkeypatch.undo()
    L.lib().omni_moe_reload_tuning()
