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
    """After a GPU session: the worst element-wise error per quantity, in units of its bound, written
    to $CF_REPORT_DIR/elementwise_errors.json when that variable names a directory."""
    from tests import helpers
    out = os.environ.get("CF_REPORT_DIR")
    if not helpers.elementwise_record or not out:
        return
    import json
    try:
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, "elementwise_errors.json"), "w") as f:
            json.dump({k: round(v, 4) for k, v in sorted(helpers.elementwise_record.items())}, f, indent=1)
    except OSError:
        pass
