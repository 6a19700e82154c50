import os
import sys

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO not in sys.path:
    sys.path.insert(0, REPO)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu() -> bool:
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_sessionfinish(session, exitstatus):
    """Writes the float-parity statistics of the session (how many compared elements passed only through the
    summation-order term of the tolerance) to the file COOPVEC_PARITY_STATS_FILE names, if it is set."""
    path = os.environ.get("COOPVEC_PARITY_STATS_FILE")
    if not path:
        return
    try:
        import json
        import oracle_binding as ob
        if ob.PARITY_STATS["elements"]:
            with open(path, "w") as f:
                json.dump(ob.PARITY_STATS, f)
    except Exception:
        pass
