import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _seed_every_test():
    """Tests that draw from torch's global generator see the same numbers whatever ran before them."""
    import torch
    torch.manual_seed(1234)
    yield


def pytest_sessionfinish(session, exitstatus):
    """LLSA_PARITY_REPORT=<file>: write the errors the parity checks measured (rel-L2, max-abs per tensor and the
    fractions of rows whose selection equals the oracle's) as JSON."""
    path = os.environ.get("LLSA_PARITY_REPORT")
    if not path:
        return
    import json
    mod = sys.modules.get("parity_cases")
    if mod is not None and mod.MEASURED:
        with open(path, "w") as f:
            json.dump(mod.MEASURED, f, indent=1)
