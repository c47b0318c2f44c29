import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_terminal_summary(terminalreporter):
    """The distances the full-size configuration tests measured (they are
    captured output otherwise)."""
    mod = sys.modules.get("tests.test_gpu_parity") or sys.modules.get("test_gpu_parity")
    lines = getattr(mod, "FULL_SIZE_REPORT", None) if mod else None
    if lines:
        terminalreporter.write_sep("-", "full-size configurations: measured rel-L2")
        for line in lines:
            terminalreporter.write_line(line)
