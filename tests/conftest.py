import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _decode(entry):
    a = np.array([float.fromhex(x) for x in entry["data_colmajor"]], dtype=np.float64)
    return a.reshape(entry["shape"], order="F")


@pytest.fixture(scope="session")
def golden():
    """The reference's own golden vectors (tests/golden/nnv_reference_vectors.json)."""
    with open(os.path.join(ROOT, "tests", "golden", "nnv_reference_vectors.json")) as f:
        raw = json.load(f)
    out = {}
    for grp, items in raw.items():
        out[grp] = {k: (_decode(v) if isinstance(v, dict) and "data_colmajor" in v else v)
                    for k, v in items.items()}
    return out
