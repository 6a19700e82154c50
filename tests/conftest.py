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


def pytest_terminal_summary(terminalreporter, exitstatus, config):
    """Prints the float-parity statistics of the session: elements compared against the oracle under the bar
    max(2 ulp, 1e-3 relative, 2^-18 sum|terms|), how many of them passed only through the third (summation-order)
    term, and per test the outputs of multi-layer networks that lay outside the bar (each one checked to be a
    rounding-boundary case of a hidden unit).  COOPVEC_PARITY_STATS_FILE, if set, also receives them as JSON."""
    try:
        import json
        import oracle_binding as ob
    except Exception:
        return
    st = ob.PARITY_STATS
    if not st["elements"]:
        return
    tr = terminalreporter
    tr.write_sep("-", "float parity statistics")
    tr.write_line("elements compared with the oracle: %d; inside the bar only through the 2^-18 sum|terms| term: %d"
                  % (st["elements"], st["passed_only_by_floor_term"]))
    e2e = st["end_to_end"]
    if e2e:
        tr.write_line("multi-layer outputs outside the bar (every one a checked rounding-boundary case), per test:")
        for name in sorted(e2e):
            o, t = e2e[name]
            if o:
                tr.write_line("  %s: %d of %d" % (name, o, t))
        tr.write_line("  total: %d of %d" % (sum(o for o, _ in e2e.values()), sum(t for _, t in e2e.values())))
    path = os.environ.get("COOPVEC_PARITY_STATS_FILE")
    if path:
        try:
            with open(path, "w") as f:
                json.dump(st, f)
        except OSError:
            pass
