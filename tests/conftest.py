import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

import cases  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def model_dir(tmp_path_factory):
    """directory holding the synthetic models of tests/cases.py as kokkos.npz files"""
    d = str(tmp_path_factory.mktemp("models"))
    for name in cases.MODELS:
        cases.write_model(name, d)
    return d


@pytest.fixture(scope="session")
def gold():
    with np.load(os.path.join(cases.GOLDEN, "reference_outputs.npz")) as z:
        return {k: z[k] for k in z.files}


@pytest.fixture(scope="session")
def tf_gold():
    with np.load(os.path.join(cases.REF_FIXTURES, "order3_tf.npz")) as z:
        return {k: z[k] for k in z.files}


def fixture_cell(name):
    """reference fixture cell -> (types for species (Mo, W), offset, j, rij, volume)"""
    with np.load(os.path.join(cases.REF_FIXTURES, name + ".npz")) as c:
        types = np.array([2 if z == 74 else 1 for z in c["numbers"]], dtype=np.int32)
        return types, c["offset"], c["j"], c["rij"], abs(np.linalg.det(c["cell"]))
