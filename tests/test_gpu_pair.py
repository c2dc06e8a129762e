"""The two reverse pair kernels of the GRACE-2L / 3L engines (bond forces of the message layers and the adjoints of the
neighbours' messages; bond_yi_bwd_g, bond_scatter_bwd_t, bond_force: libgrace/include/grace/fused_cpu.h:836-942,1027-1050):
the one on the matrix cores (the default where it is the faster one) against the vector kernels (GRACE_HIP_PAIR_MFMA=0)
and both against the oracle, for block shapes with whole and partial slot groups, chunks of bonds that are not a
multiple of 16, per-atom virials and atoms in chunks."""
import numpy as np
import pytest

import cases
from grace_runtime_amd import kk

pytestmark = pytest.mark.gpu

_oracle = {}


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("model,struct,species", [("l2mix", "alloy54", ["Mo", "W"]), ("config3", "fcc108", ["Al", "Co", "Ni", "Ti"]),
                                                  ("l3mix", "alloy54", ["Mo", "W"]), ("l3wide", "fcc108", ["Al", "Co", "Ni", "Ti"]),
                                                  ("l3el", "alloy54", ["Mo", "W"]), ("l3mix", "molecule", ["Mo", "W"])])
@pytest.mark.parametrize("waves", [8, 4, 2])
def test_matrix_core_kernel_equals_the_vector_kernel_and_the_oracle(model_dir, monkeypatch, model, struct, species, precision, waves):
    path = cases.model_file(model_dir, model)
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    types = np.minimum(types, len(species)).astype(np.int32)
    n = len(pos)
    out = {}
    for mfma in ("1", "0"):
        monkeypatch.setenv("GRACE_HIP_PAIR_MFMA", mfma)
        monkeypatch.setenv("GRACE_HIP_PAIR_WAVES", str(waves))
        s = kk.System(kk.Model(path), species, skin=0.0, precision=precision, chunksize=0 if waves != 4 else 17)
        out[mfma] = s.compute(types, pos, cell, pbc, energies=True, virials=True)
    if (model, struct) not in _oracle:
        _oracle[(model, struct)] = cases.oracle_reference(model_dir, model, pos, cell, pbc, types)
    ref = _oracle[(model, struct)]
    fs = max(1.0, np.abs(ref["forces"]).max())
    vs = max(1.0, np.abs(ref["virials"]).max())
    tol = 1e-10 if precision == 64 else 2e-6
    for key in ("1", "0"):
        assert abs(out[key]["energy"] - ref["energy"]) / n < tol * fs
        assert np.abs(out[key]["forces"] - ref["forces"]).max() < 10 * tol * fs
        assert np.abs(out[key]["virial"] - ref["virial"]).max() < 100 * tol * fs
        assert np.abs(out[key]["virials"] - ref["virials"]).max() < 10 * tol * vs
    assert np.abs(out["1"]["forces"] - out["0"]["forces"]).max() < tol * fs
    assert np.abs(out["1"]["virials"] - out["0"]["virials"]).max() < 10 * tol * vs
