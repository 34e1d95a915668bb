"""Shared pytest configuration: the ``gpu`` marker and repo-root imports."""

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


def pytest_terminal_summary(terminalreporter):
    from tests import helpers

    if helpers.PARITY_NOTES:
        terminalreporter.section("routing parity and load figures")
        for line in helpers.PARITY_NOTES:
            terminalreporter.write_line(line)
