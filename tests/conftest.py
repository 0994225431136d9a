import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _release_device_uploads(request):
    """GPU tests: wait for the test's launches, then free what helpers.dev() uploaded."""
    yield
    if request.node.get_closest_marker("gpu") is None:
        return
    import helpers
    if helpers._uploads:
        from reinstinct_amd import hip
        hip.synchronize()
        helpers.release_uploads()


@pytest.fixture
def options():
    """Library options (rein_set_option) for one test: what the test sets goes back to its former
    state afterwards."""
    from reinstinct_amd import _lib

    class Options:
        def __init__(self):
            self.before = {}

        def set(self, name, value):
            self.before.setdefault(name, _lib.get_option(name))
            _lib.set_option(name, value)

        def unset(self, name):
            self.set(name, None)

    o = Options()
    yield o
    for name, value in o.before.items():
        _lib.set_option(name, value)
