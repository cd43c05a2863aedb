import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
sys.path.insert(0, os.path.join(ROOT, "tetris-artifact-evalution_amd"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

GOLDEN = os.path.join(ROOT, "tests", "golden")
REFERENCE = "/root/reference"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle_py

    if not oracle_py.available():
        pytest.skip("oracle/libtetris_oracle.so not built (make -C oracle)")
    return oracle_py


def golden_weights(name):
    z = np.load(os.path.join(GOLDEN, "weights_%s.npz" % name))
    hdr = dict(zip(("H", "W", "IC", "OC", "KS", "PAD", "STRIDE", "GROUPS"), [int(v) for v in z["header"]]))
    return hdr, np.ascontiguousarray(z["filter"], np.float32), str(z["source"])
