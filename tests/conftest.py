import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle_lib():
    """The CPU oracle; compiled on first use when oracle/liboracle.so is absent."""
    import oracle
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def hip_lib():
    """The HIP C-ABI library; built on first use when it is absent (never silently skipped)."""
    from swin3d_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH):
        build.build(force=True)
    return _lib.lib()


def random_scene(rng, n, extent=(12, 12, 6), batches=1, stride=1, duplicates=False):
    """n distinct voxels (batch,x,y,z) int32 inside a small box, unsorted."""
    capacity = batches * 8 * extent[0] * extent[1] * extent[2]
    assert duplicates or n <= 0.8 * capacity, f"{n} distinct voxels do not fit a box of {capacity} cells"
    rows = set()
    out = []
    while len(out) < n:
        b = int(rng.integers(0, batches))
        c = tuple(int(rng.integers(-extent[a], extent[a])) * stride for a in range(3))
        if (b,) + c in rows and not duplicates:
            continue
        rows.add((b,) + c)
        out.append((b,) + c)
    arr = np.asarray(out, np.int32)
    # batches must be contiguous and ascending
    return arr[np.argsort(arr[:, 0], kind="stable")]
