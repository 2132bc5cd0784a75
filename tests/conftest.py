import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run through the C-ABI HIP library)")


@pytest.fixture(scope="session")
def lut_fixtures():
    """Golden LUTs written by tests/golden/make_lut_fixtures.py from the
    reference's own host code (data only)."""
    import json
    path = os.path.join(ROOT, "tests", "golden", "lut_fixtures.npz")
    z = np.load(path, allow_pickle=False)
    meta = json.loads(bytes(z["meta_json"]).decode())
    return z, meta


def mask_kwargs(meta_kw):
    kw = dict(meta_kw)
    if isinstance(kw.get("local_blocks"), list):
        kw["local_blocks"] = tuple(kw["local_blocks"])
    return kw
