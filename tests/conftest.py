import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; run with -m gpu on the GPU box")


def pytest_collection_modifyitems(config, items):
    try:
        import torch

        has_gpu = torch.cuda.is_available()
    except Exception:  # pragma: no cover
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_terminal_summary(terminalreporter):
    from tests import helpers

    for label, (ratio, abs_err) in sorted(helpers.ERROR_STATS.items()):
        terminalreporter.write_line(
            f"[numerics] {label}: worst error {abs_err:.3e}, {ratio:.2f} of its bound")
