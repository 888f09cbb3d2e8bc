import os
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu() -> bool:
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def lib():
    """The HIP library; GPU tests must never run without it."""
    from lighthouse_amd import _lib

    return _lib.load()


PARITY_LOG: list[tuple[str, float, float, float]] = []


def assert_close(got, ref, rtol, what="", report=False, floor=1.0):
    """|got - ref| <= rtol * (|ref| + floor * max|ref|): the relative tolerance of the benchmark
    definition with an absolute floor tied to the magnitude of the reference, because sums
    that cancel to ~0 carry the rounding error of their largest terms.  ``floor`` < 1 tightens
    that absolute part (benchmark-size checks, where max|ref| is far above a typical element).
    ``report``: the achieved max|err| / max|ref| and max|err| / (|ref| + max|ref|) go into the
    summary printed at the end of the test run."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite values in result"
    scale = np.abs(ref).max() if ref.size else 0.0
    err = np.abs(got - ref)
    bound = rtol * (np.abs(ref) + floor * scale)
    if report and ref.size and scale > 0:
        PARITY_LOG.append((what, rtol, float(err.max() / scale), float((err / (np.abs(ref) + scale)).max())))
    bad = err > bound
    if bad.any():
        idx = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(
            f"{what}: {bad.sum()} of {bad.size} elements out of tolerance rtol={rtol}; worst at {idx}: "
            f"got {got[idx]!r} ref {ref[idx]!r} (max|ref|={scale})"
        )


def pytest_terminal_summary(terminalreporter):
    if not PARITY_LOG:
        return
    terminalreporter.section("achieved parity error (benchmark configurations)")
    for what, rtol, norm, rel in PARITY_LOG:
        terminalreporter.write_line(
            f"{what}: max|err|/max|ref| = {norm:.3e}, max|err|/(|ref|+max|ref|) = {rel:.3e} (tolerance {rtol:g})")
