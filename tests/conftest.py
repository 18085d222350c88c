import json
import os
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN_DIR = Path(__file__).resolve().parent / "golden"


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
def known_answers():
    with open(GOLDEN_DIR / "reference_known_answers.json") as fh:
        return json.load(fh)


@pytest.fixture(scope="session")
def dev():
    return torch.device("cuda")


def pytest_runtest_logstart(nodeid, location):
    # name the case before any GPU work starts, so a lost box still tells which test ran
    if os.environ.get("MALTOS_TEST_TRACE", "1" if torch.cuda.is_available() else "0") == "1":
        print(f"\n[test] {nodeid}", flush=True)
