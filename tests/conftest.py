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
    """Tests load the library that is built; it is built here only when there is none or when it was
    built from other sources than the ones next to it.  A build that fails (no hipcc on this machine)
    is reported and the session goes on: tests that need the library then fail through its loader's
    own error, the others still run."""
    from triattention_amd import build as tri_build
    try:
        tri_build.ensure_built()
    except Exception as exc:      # noqa: BLE001 - reported, not swallowed
        print(f"\nconftest: could not build libtriattention_hip.so: {exc}", file=sys.stderr, flush=True)


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _library_defaults():
    """Every test starts from and leaves behind the library's default settings (helpers.tune changes
    them for the rest of a test)."""
    yield
    import helpers
    from triattention_amd import _lib
    if _lib._lib is not None:
        helpers.reset_tuning()


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
