import pathlib
import sys

import pytest
import torch

ROOT = pathlib.Path(__file__).resolve().parent.parent
for p in (ROOT / "cutile-python_amd", ROOT):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def ct():
    import cutile_amd
    return cutile_amd


@pytest.fixture(scope="session")
def dev():
    assert torch.cuda.is_available()
    import cutile_amd
    rc = cutile_amd.lib().mx_device_check()
    assert rc == 0, cutile_amd._lib.last_error()
    return torch.device("cuda:0")
