import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _have_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    O.lib()
    return O


@pytest.fixture(scope="session")
def golden():
    path = os.path.join(ROOT, "tests", "golden", "encoder_fixtures.npz")
    data = np.load(path, allow_pickle=False)
    cases = {}
    for name in data["names"]:
        name = str(name)
        cases[name] = {k: data[f"{name}/{k}"] for k in
                       ("W", "values", "offsets", "median", "bitmaps", "tile_counts", "scalars")}
    return cases


# Tolerance of the SpMM contract: fp32 accumulate, fp16 out.
MAX_ABS_FRAC = 1e-2   # max|C - C_ref| <= 1e-2 * max|C_ref|
REL_L2 = 1e-3         # ||C - C_ref||_2 <= 1e-3 * ||C_ref||_2


def assert_spmm_close(C, C_ref, what=""):
    C = np.asarray(C, dtype=np.float64)
    R = np.asarray(C_ref, dtype=np.float64)
    assert C.shape == R.shape, what
    assert np.isfinite(C).all(), f"{what}: non-finite output"
    scale = np.abs(R).max()
    if scale == 0:
        assert np.abs(C).max() == 0, f"{what}: expected all zeros"
        return
    max_abs = np.abs(C - R).max()
    rel_l2 = np.linalg.norm(C - R) / np.linalg.norm(R)
    assert max_abs <= MAX_ABS_FRAC * scale, f"{what}: max|d|={max_abs:.3e} > {MAX_ABS_FRAC}*{scale:.3e}"
    assert rel_l2 <= REL_L2, f"{what}: rel-L2={rel_l2:.3e} > {REL_L2}"
