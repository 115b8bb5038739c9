import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    import json
    with open(os.path.join(ROOT, "tests", "golden", "wiring_golden.json")) as f:
        return json.load(f)


@pytest.fixture(autouse=True)
def _knobs_follow_the_environment():
    """The library reads its CLG_* environment knobs once per process; tests that force a code path set them through
    gpu_util.set_knobs (setenv + reload), and this re-reads them after monkeypatch has restored the environment."""
    yield
    from convlogic_amd.hip import _lib
    if _lib.available():
        _lib.reload_knobs()
