import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


@pytest.fixture(autouse=True, scope="session")
def _isolated_plan_cache(tmp_path_factory):
    """Kernels requested with a zero schedule consult the plan cache; point it at an empty directory so that a plan
    left by an earlier search cannot change which kernel variant a test exercises (tests of the cache set their own)."""
    old = os.environ.get("KSEARCH_BEAM_CACHE")
    os.environ["KSEARCH_BEAM_CACHE"] = str(tmp_path_factory.mktemp("plans"))
    yield
    if old is None:
        os.environ.pop("KSEARCH_BEAM_CACHE", None)
    else:
        os.environ["KSEARCH_BEAM_CACHE"] = old


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _have_gpu() -> bool:
    return os.path.exists("/dev/kfd") and os.access("/dev/kfd", os.R_OK | os.W_OK)


def pytest_collection_modifyitems(config, items):
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU device node in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
