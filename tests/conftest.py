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


def assert_close(got, ref, rtol, what=""):
    """|got - ref| <= rtol * (|ref| + max|ref|): the relative tolerance of the benchmark
    definition with an absolute floor tied to the magnitude of the reference, because sums
    that cancel to ~0 carry the rounding error of their largest terms."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite values in result"
    scale = np.abs(ref).max() if ref.size else 0.0
    err = np.abs(got - ref)
    bound = rtol * (np.abs(ref) + scale)
    bad = err > bound
    if bad.any():
        idx = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(
            f"{what}: {bad.sum()} of {bad.size} elements out of tolerance rtol={rtol}; worst at {idx}: "
            f"got {got[idx]!r} ref {ref[idx]!r} (max|ref|={scale})"
        )
