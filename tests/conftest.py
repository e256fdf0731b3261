import os
import sys

import numpy as np
import pytest

# the library's test hooks (planner knobs, dump builds, calibration kernels) are refused unless the process asks for them
os.environ.setdefault("LLMOPS_TEST_HOOKS", "1")

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))
for p in (ROOT, os.path.join(ROOT, "llama.cl_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    # GPU tests are skipped outright when no device is visible, so a plain `pytest tests/` works anywhere
    try:
        import torch
        have = torch.cuda.is_available()
    except Exception:
        have = False
    if have:
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for it in items:
        if "gpu" in it.keywords:
            it.add_marker(skip)


def load_golden(name):
    with np.load(os.path.join(GOLDEN, name), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


@pytest.fixture(scope="session")
def orc():
    import oracle
    return oracle.Oracle()


def max_rel_err(got, ref):
    """max|got-ref| / max|ref| : the 1e-3 float gate of the FC and attention outputs."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    den = np.abs(ref).max()
    return np.abs(got - ref).max() / (den if den > 0 else 1.0)
