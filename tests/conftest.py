import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _has_gpu():
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


def pytest_terminal_summary(terminalreporter):
    """The measured share of elements beyond two BF16 steps behind every rare-outlier bar of the run, largest first."""
    try:
        import helpers
    except Exception:
        return
    stats = sorted(helpers.OUTLIER_STATS, key=lambda t: -t[3])[:12]
    if stats:
        terminalreporter.write_line("rare-outlier bars, largest measured share beyond 2 steps:")
        for what, r, worst, frac, rare, loose in stats:
            terminalreporter.write_line("  %-70s rel L2 %.2e  worst %.1f / %d steps  share %.2e / %.1e" % (what[:70], r, worst, loose, frac, rare))
