import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def fixtures_small():
    """name -> dict(x, w, y, L, pad) from tests/golden/fixtures_small.npz (outputs of the
    reference's compiled CPU kernel)."""
    import numpy as np

    path = os.path.join(ROOT, "tests", "golden", "fixtures_small.npz")
    z = np.load(path, allow_pickle=False)
    out = {}
    for key in z.files:
        name, field = key.split("/")
        out.setdefault(name, {})[field] = z[key]
    for name, d in out.items():
        d["L"], d["pad"] = int(d["meta"][0]), int(d["meta"][1])
    return out


@pytest.fixture(scope="session")
def checksums():
    import json

    with open(os.path.join(ROOT, "tests", "golden", "checksums.json")) as f:
        return json.load(f)
