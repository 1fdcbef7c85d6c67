import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped (not failed) when no device is visible and the
    run did not ask for them with -m gpu."""
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# ------------------------------------------------------------ small graphs
def random_csc(rng, num_cols, num_rows, max_deg, empty_frac=0.2, hub_deg=0):
    """Ragged random CSC with empty columns and (optionally) one hub column."""
    deg = rng.integers(0, max_deg + 1, size=num_cols)
    deg[rng.random(num_cols) < empty_frac] = 0
    if hub_deg and num_cols > 0:
        deg[rng.integers(0, num_cols)] = hub_deg
    indptr = np.zeros(num_cols + 1, dtype=np.int64)
    np.cumsum(deg, out=indptr[1:])
    indices = rng.integers(0, num_rows, size=int(indptr[-1])).astype(np.int64)
    return indptr, indices


@pytest.fixture
def rng():
    return np.random.default_rng(12345)


def golden() -> dict:
    """Known answers of the reference's own tests (tests/golden/)."""
    import json
    import os
    path = os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")
    with open(path) as f:
        return json.load(f)
