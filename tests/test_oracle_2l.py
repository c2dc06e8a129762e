"""Pins of the GRACE-2L CPU oracle (oracle/grace_oracle_2l.py).  No GPU.

* end to end against the reference's TensorFlow fp64 goldens (tests/golden/ref_fixtures/order3_tf.npz; recipe
  python/tests/test_ref_tf.py:43-55 of the reference): every stage of a max_order-3 GRACE-2L model at fp64 level, current
  and legacy layout;
* end to end against outputs of the compiled reference (fp32 + spline tables; tests/golden/reference_outputs.npz) on
  its own fixture models with the AAAA / BBBB stages and lmax 3, and on the synthetic lmax-4 and unequal-width models,
  at the reference's fp32-vs-fp64 tolerances (python/tests/test_ref_tf.py:22-23);
* forces = -dE/dx and virial = strain derivative by central differences, rotation invariance.
"""
import os

import numpy as np
import pytest

import cases
from conftest import fixture_cell
from oracle import grace_oracle as go
from oracle import grace_oracle_2l as g2

TOL = {"energy": 1e-6, "forces": 2e-5, "energies": 1e-5, "stress": 1e-5}    # eV/atom, eV/A, eV, relative


@pytest.mark.parametrize("cell", ["W54", "WMo54", "W2tri"])
@pytest.mark.parametrize("name", ["grace_2l_order3", "legacy_2l_order3"])
def test_oracle_matches_tf_fp64(tf_gold, name, cell):
    m = g2.Model2L(os.path.join(cases.REF_FIXTURES, name + ".npz"))
    types, offset, j, rij, vol = fixture_cell(cell)
    mu = np.array([m.names.index("Mo"), m.names.index("W")])[types - 1]
    out = g2.compute_2l(m, mu, offset, j, rij)
    k = f"{name}/{cell}"
    n = len(types)
    assert abs(out["energy"] - tf_gold[k + "/energy"]) / n < 1e-10
    assert np.abs(out["forces"] - tf_gold[k + "/forces"]).max() < 1e-9
    assert np.abs(out["energies"] - tf_gold[k + "/energies"]).max() < 1e-10
    assert np.abs(go.virial_to_stress(out["virial"], vol) - tf_gold[k + "/stress"]).max() < 1e-10
    assert np.abs(tf_gold[k + "/forces"]).max() > 1e-2


def _close(out, gold, tag, n):
    fmax = max(1.0, np.abs(gold[tag + "/forces"]).max())
    assert abs(out["energy"] - gold[tag + "/energy"]) / n < TOL["energy"] * fmax
    assert np.abs(out["forces"] - gold[tag + "/forces"]).max() < TOL["forces"] * fmax
    assert np.abs(out["energies"] - gold[tag + "/energies"]).max() < TOL["energies"] * fmax
    assert np.abs(out["virial"] - gold[tag + "/virial"]).max() < TOL["stress"] * max(1.0, np.abs(gold[tag + "/virial"]).max())


@pytest.mark.parametrize("model,cell", cases.FIXTURE_CASES_2L)
def test_oracle_matches_compiled_reference_on_fixture_models(gold, model, cell):
    m = g2.Model2L(os.path.join(cases.REF_FIXTURES, model + ".npz"))
    types, offset, j, rij, _ = fixture_cell(cell)
    mu = np.array([m.names.index("Mo"), m.names.index("W")])[types - 1]
    out = g2.compute_2l(m, mu, offset, j, rij)
    _close(out, gold, f"fixture/{model}/{cell}", len(types))


@pytest.mark.parametrize("model,struct,rc", cases.E2E_CASES_2L)
def test_oracle_matches_compiled_reference(model_dir, gold, model, struct, rc):
    m = g2.Model2L(cases.model_file(model_dir, model))
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    types = np.minimum(types, m.n_elements)
    tag = f"e2e/{model}/{struct}"
    key = f"nl/{struct}@{float(gold[tag + '/rc_list']):g}"
    perm, offset, j, image, shifts = (gold[f"{key}/{k}"] for k in ("perm", "offset", "j", "image", "shifts"))
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    out = g2.compute_2l(m, types[perm] - 1, offset, j, rij)
    _close(out, gold, tag, len(types))
    assert np.abs(gold[tag + "/forces"]).max() > 1e-2


def _tiny_system(seed=2):
    """12 atoms in a small triclinic cell, bonds by brute force over images"""
    rng = np.random.default_rng(seed)
    cell = np.array([[6.0, 0.0, 0.0], [0.7, 5.6, 0.0], [-0.5, 0.9, 6.3]])
    pos = rng.uniform(0, 1, (12, 3)) @ cell
    types = rng.integers(0, 2, 12)
    return pos, cell, types


def _bonds(pos, cell, rc):
    n = len(pos)
    off, jj, rij = [0], [], []
    rng3 = range(-2, 3)
    for i in range(n):
        for a in rng3:
            for b in rng3:
                for c in rng3:
                    S = a * cell[0] + b * cell[1] + c * cell[2]
                    for k in range(n):
                        d = pos[k] + S - pos[i]
                        if (a or b or c or k != i) and d @ d < rc * rc:
                            jj.append(k)
                            rij.append(d)
        off.append(len(jj))
    return np.array(off), np.array(jj), np.array(rij)


def test_forces_and_virial_are_derivatives_of_the_energy():
    m = g2.Model2L(os.path.join(cases.REF_FIXTURES, "grace_2l_small.npz"))
    pos, cell, mu = _tiny_system()

    def energy(p, c):
        off, jj, rij = _bonds(p, c, 5.0)
        return g2.compute_2l(m, mu, off, jj, rij, want_forces=False)["energy"]

    off, jj, rij = _bonds(pos, cell, 5.0)
    out = g2.compute_2l(m, mu, off, jj, rij)
    assert np.abs(out["forces"].sum(0)).max() < 1e-12
    h = 1e-5
    for i, d in [(0, 0), (5, 1), (11, 2)]:
        p1, p2 = pos.copy(), pos.copy()
        p1[i, d] += h
        p2[i, d] -= h
        assert abs(-(energy(p1, cell) - energy(p2, cell)) / (2 * h) - out["forces"][i, d]) < 1e-7
    # virial (xx yy zz xy xz yz) = -dE/d(strain): x -> (1 + eps) x
    for k, (a, b) in enumerate([(0, 0), (1, 1), (2, 2), (0, 1), (0, 2), (1, 2)]):
        eps = np.zeros((3, 3))
        eps[a, b] = h
        dE = (energy(pos @ (np.eye(3) + eps).T, cell @ (np.eye(3) + eps).T) -
              energy(pos @ (np.eye(3) - eps).T, cell @ (np.eye(3) - eps).T)) / (2 * h)
        assert abs(-dE - out["virial"][k]) < 1e-6


def test_rotation_invariance_of_a_generated_model(model_dir):
    """the structure generator's couplings (also the odd-parity ones) make an invariant energy and covariant forces"""
    m = g2.Model2L(cases.model_file(model_dir, "l2mix"))
    pos, cell, mu = _tiny_system(4)
    off, jj, rij = _bonds(pos, cell, 5.0)
    out = g2.compute_2l(m, mu, off, jj, rij)
    q, _ = np.linalg.qr(np.random.default_rng(0).standard_normal((3, 3)))
    if np.linalg.det(q) < 0:
        q[:, 0] = -q[:, 0]
    rot = g2.compute_2l(m, mu, off, jj, rij @ q.T)
    assert abs(rot["energy"] - out["energy"]) < 1e-9 * max(1.0, abs(out["energy"]))
    assert np.abs(rot["forces"] - out["forces"] @ q.T).max() < 1e-9 * max(1.0, np.abs(out["forces"]).max())
    # improper rotation: the energy is a scalar (the pseudo-tensor channels only enter in even products)
    inv = g2.compute_2l(m, mu, off, jj, -rij)
    assert abs(inv["energy"] - out["energy"]) < 1e-9 * max(1.0, abs(out["energy"]))


def test_isolated_atom_and_zero_bond():
    m = g2.Model2L(os.path.join(cases.REF_FIXTURES, "grace_2l_order3.npz"))
    out = g2.compute_2l(m, [1], [0, 0], np.zeros(0, int), np.zeros((0, 3)))
    assert np.abs(out["forces"]).max() == 0.0 and np.isfinite(out["energy"])
    with pytest.raises(go.ZeroBondError):
        g2.compute_2l(m, [0, 0], [0, 1, 2], [1, 0], np.zeros((2, 3)))
