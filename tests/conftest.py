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
    old = {k: os.environ.get(k) for k in ("KSEARCH_BEAM_CACHE", "KSEARCH_SKIP_BEAM")}
    os.environ["KSEARCH_BEAM_CACHE"] = str(tmp_path_factory.mktemp("plans"))
    # models search their schedules when they are loaded and keep the winners as plans: timing decides between
    # near-equal candidates, so the kernel variants (and with them the f32 summation order) would change from run to
    # run and leak from one test's model to the next.  The tests of the search and of the warm-up switch it on.
    os.environ["KSEARCH_SKIP_BEAM"] = "1"
    yield
    for k, v in old.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v


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
