import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """The libraries are built in-tree beforehand and loaded as they are; only a tree with nothing built (a fresh clone)
    builds them here, once."""
    import importlib
    pkg = importlib.import_module("m40-llm_amd")
    if not (os.path.exists(pkg.NATIVE_LIB) and os.path.exists(pkg.HOST_LIB)):
        pkg.build()


def _has_gpu() -> bool:
    # /dev/kfd is the ROCm compute device node; probing it does not initialise HIP.
    return os.path.exists("/dev/kfd")


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def orc():
    from oracle import pyoracle
    pyoracle.build()
    pyoracle.lib()
    return pyoracle


@pytest.fixture
def heartbeat(request):
    """A long test's sign of life: writes to the real terminal while output is captured, so that a run whose output is
    watched for activity does not look hung during minutes of CPU-side checking."""
    capman = request.config.pluginmanager.getplugin("capturemanager")

    def beat(text="."):
        if capman is None:
            sys.stdout.write(text); sys.stdout.flush()
            return
        with capman.global_and_fixture_disabled():
            sys.stdout.write(text); sys.stdout.flush()
    return beat
