import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.pyoracle import Oracle

    return Oracle()


@pytest.fixture(scope="session")
def reflib():
    from oracle.pyoracle import RefLib

    if not RefLib.available():
        pytest.skip("oracle/_ref not built (needs the reference checkout: make -C oracle ref)")
    return RefLib()


@pytest.fixture(scope="session")
def ref_goldens():
    return dict(np.load(os.path.join(GOLDEN_DIR, "reference_goldens.npz"), allow_pickle=False))


@pytest.fixture(scope="session")
def ref_gaussian():
    return dict(np.load(os.path.join(GOLDEN_DIR, "ref_gaussian.npz"), allow_pickle=False))
