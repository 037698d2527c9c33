import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped (not failed) when no device is present."""
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_terminal_summary(terminalreporter):
    """After a GPU run: how much of every stated tolerance the worst element used."""
    mod = sys.modules.get("tests.test_lfw_gpu")
    use = getattr(mod, "TOLERANCE_USE", None)
    if not use:
        return
    terminalreporter.write_sep("-", "largest |err| / bound per (rtol, afrac, tensor)")
    for (rtol, afrac, what), v in sorted(use.items()):
        terminalreporter.write_line("rtol %-8g afrac %-8g %-12s %.3f" % (rtol, afrac, what, v))
