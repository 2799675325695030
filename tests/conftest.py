import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


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
def dev():
    return torch.device("cuda:0")


def pytest_sessionfinish(session, exitstatus):
    """After a GPU session: the worst element-wise error per quantity, in units of its bound."""
    from tests import helpers
    if not helpers.elementwise_record:
        return
    import json
    out = os.path.join(ROOT, "gpurun_out")
    try:
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, "elementwise_errors.json"), "w") as f:
            json.dump({k: round(v, 4) for k, v in sorted(helpers.elementwise_record.items())}, f, indent=1)
    except OSError:
        pass
