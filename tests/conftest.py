import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


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
    """The worst row-wise error the comparisons with the plain implementation have met, for the record."""
    try:
        import gpu_common
    except Exception:
        return
    seen = {k: v for k, v in gpu_common.worst_row_seen.items() if v}
    if seen:
        terminalreporter.write_line("worst row of any comparison with the plain implementation, relative to the row's "
                                    "largest logit: " + ", ".join(f"{k} {v:.2e}" for k, v in seen.items()))
