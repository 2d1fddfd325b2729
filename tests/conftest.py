import os
import sys

import pytest

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for _p in (os.path.join(_ROOT, "ops-rec_amd"), _ROOT):
    if _p not in sys.path:
        sys.path.insert(0, _p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box with -m gpu)")


def pytest_collection_modifyitems(config, items):
    # GPU tests are only meaningful on a box with a GPU; on a CPU-only host they are skipped
    # (the driver selects them with -m gpu / -m "not gpu" anyway).
    try:
        import torch

        has_gpu = torch.cuda.is_available()
    except Exception:  # noqa: BLE001
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _switches_follow_the_environment():
    """A test that changes one of the library's ``HSTU_MI355_*`` switches (``helpers.set_switch``) leaves the library
    holding that value; once the test's environment has been put back (this fixture is set up first, so it is torn
    down last) the library reads its switches again."""
    yield
    from ops_rec import _native

    if _native._lib is not None:
        _native.reload_switches()
