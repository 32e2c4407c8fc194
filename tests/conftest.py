import os
import sys

os.environ["TORCH_MOJO_BACKEND_TESTING"] = "1"

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (_ROOT, os.path.join(_ROOT, "torch-max-backend_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

import pytest  # noqa: E402
import torch  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no HIP device in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def reset_compiler():
    torch.compiler.reset()
    yield


@pytest.fixture()
def call_checker():
    from torch_mojo_backend.testing import CallChecker

    checker = CallChecker()
    yield checker
    checker.check_was_called()


def pytest_make_parametrize_id(val):
    if isinstance(val, torch.dtype):
        return str(val).split(".")[-1]
    return None
