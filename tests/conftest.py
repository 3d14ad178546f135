"""Shared pytest configuration: the ``gpu`` marker and fixture loading."""
from __future__ import annotations

import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN = Path(__file__).resolve().parent / "golden"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """Tests load the library that is built; only when there is none do they build it."""
    from triattention_amd import build as tri_build
    tri_build.ensure_built()


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def load_golden(name: str):
    """Fixtures are plain tensor dicts this repo wrote; nothing in them executes."""
    return torch.load(GOLDEN / name, map_location="cpu", weights_only=True)


def pytest_terminal_summary(terminalreporter):
    """One line for the whole run: how many kept indices differed from the oracle's (or the other
    path's) at near-ties, over how many compared."""
    import helpers
    if not helpers.SWAPS:
        return
    swapped = sum(s for s, _ in helpers.SWAPS.values())
    compared = sum(c for _, c in helpers.SWAPS.values())
    cases = sorted(f"{name} {s}/{c}" for name, (s, c) in helpers.SWAPS.items() if s)
    terminalreporter.write_line(
        f"near-tie swaps: {swapped} of {compared} kept indices in {len(helpers.SWAPS)} comparisons"
        + (f" (cases: {', '.join(cases)})" if cases else ""))
