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
def model_dir():
    """Directory of the synthetic models of tests/cases.py as kokkos.npz files.  A model is written when a test first asks
    for it (cases.model_file); the directory is shared by the workers of a run and by later runs as long as the
    generators do not change (its name carries a digest of their sources)."""
    import hashlib
    import tempfile
    h = hashlib.sha256()
    for f in (os.path.join(ROOT, "grace_runtime_amd", "synth.py"), os.path.join(ROOT, "grace_runtime_amd", "workloads.py"),
              os.path.join(ROOT, "tests", "cases.py")):
        with open(f, "rb") as fh:
            h.update(fh.read())
    d = os.path.join(tempfile.gettempdir(), "grace_hip_test_models_" + h.hexdigest()[:16])
    os.makedirs(d, exist_ok=True)
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
