import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_terminal_summary(terminalreporter):
    """The largest differences the comparisons with the plain implementation met (their bounds are stated in helpers.py)."""
    try:
        import helpers
    except Exception:
        return
    if any(helpers.MEASURED.values()):
        terminalreporter.write_line("measured against the plain implementation: " + ", ".join(f"{k} {v:.3e}" for k, v in helpers.MEASURED.items()))
