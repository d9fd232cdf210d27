"""Shared test configuration.

Markers:  gpu -- needs an MI355X (run with `-m gpu`); everything else runs on a CPU-only box.
"""
import json
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a GPU (MI355X); deselect with -m 'not gpu'")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def golden():
    return json.loads((ROOT / "tests" / "golden" / "golden_vectors.json").read_text())


@pytest.fixture(scope="session")
def oracle():
    import oracle as _oracle

    _oracle.build()
    return _oracle


def pytest_terminal_summary(terminalreporter):
    """How many elements the parity tests let through the cancellation floor (oracle/compare.py)."""
    try:
        from oracle import compare
    except ImportError:
        return
    lines = compare.stats_lines()
    if lines:
        terminalreporter.section("cancellation-floor accounting")
        for ln in lines:
            terminalreporter.write_line(ln)
