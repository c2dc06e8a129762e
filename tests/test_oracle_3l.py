"""Pins of the GRACE-3L CPU oracle (oracle/grace_oracle_3l.py).  No GPU.

The reference checkout holds no GRACE-3L model file and no 3L golden vector (its 3L tests load a registry model that is
downloaded), so the pins are:

* end to end against outputs of the compiled reference CPU driver Grace3LFused (fp32 + spline tables;
  tests/golden/reference_outputs.npz, written by tests/golden/make_golden.py) on generated models: natural-parity and
  both-parity messages, pair-specific cutoffs, lmax 2 and 3, periodic / slab / molecule cells, at the reference's
  fp32-vs-fp64 tolerances (python/tests/test_ref_tf.py:22-23);
* forces = -dE/dx and virial = strain derivative by central differences of the oracle's energy;
* invariance under proper and improper rotations, translation and relabelling of the atoms;
* closed forms: an isolated atom gives the readout of the zero density; per-atom energies sum to the energy.
"""
import os

import numpy as np
import pytest

import cases
from oracle import grace_oracle as go
from oracle import grace_oracle_3l as g3
from test_oracle_2l import _bonds, _tiny_system

TOL = {"energy": 1e-6, "forces": 2e-5, "energies": 1e-5, "stress": 1e-5}    # eV/atom, eV/A, eV, relative


@pytest.mark.parametrize("model,struct,rc", cases.E2E_CASES_3L)
def test_oracle_matches_compiled_reference(model_dir, gold, model, struct, rc):
    m = g3.Model3L(cases.model_file(model_dir, model))
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    types = np.minimum(types, m.n_elements)
    tag = f"e2e/{model}/{struct}"
    key = f"nl/{struct}@{float(gold[tag + '/rc_list']):g}"
    perm, offset, j, image, shifts = (gold[f"{key}/{k}"] for k in ("perm", "offset", "j", "image", "shifts"))
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    out = g3.compute_3l(m, types[perm] - 1, offset, j, rij)
    n = len(types)
    fmax = max(1.0, np.abs(gold[tag + "/forces"]).max())
    assert abs(out["energy"] - gold[tag + "/energy"]) / n < TOL["energy"] * fmax
    assert np.abs(out["forces"] - gold[tag + "/forces"]).max() < TOL["forces"] * fmax
    assert np.abs(out["energies"] - gold[tag + "/energies"]).max() < TOL["energies"] * fmax
    assert np.abs(out["virial"] - gold[tag + "/virial"]).max() < TOL["stress"] * max(1.0, np.abs(gold[tag + "/virial"]).max())
    assert np.abs(gold[tag + "/forces"]).max() > 1e-2
    assert abs(out["energies"].sum() - out["energy"]) < 1e-10 * max(1.0, abs(out["energy"]))


@pytest.mark.parametrize("model", ["l3mix", "l3pad"])
def test_forces_and_virial_are_derivatives_of_the_energy(model_dir, model):
    m = g3.Model3L(cases.model_file(model_dir, model))
    pos, cell, mu = _tiny_system()

    def energy(p, c):
        off, jj, rij = _bonds(p, c, 5.0)
        return g3.compute_3l(m, mu, off, jj, rij, want_forces=False)["energy"]

    off, jj, rij = _bonds(pos, cell, 5.0)
    out = g3.compute_3l(m, mu, off, jj, rij)
    assert np.abs(out["forces"].sum(0)).max() < 1e-11
    h = 1e-5
    for i, d in [(0, 0), (5, 1), (11, 2)]:
        p1, p2 = pos.copy(), pos.copy()
        p1[i, d] += h
        p2[i, d] -= h
        assert abs(-(energy(p1, cell) - energy(p2, cell)) / (2 * h) - out["forces"][i, d]) < 1e-7 * max(1.0, np.abs(out["forces"]).max())
    for k, (a, b) in enumerate([(0, 0), (1, 1), (2, 2), (0, 1), (0, 2), (1, 2)]):
        eps = np.zeros((3, 3))
        eps[a, b] = h
        dE = (energy(pos @ (np.eye(3) + eps).T, cell @ (np.eye(3) + eps).T) -
              energy(pos @ (np.eye(3) - eps).T, cell @ (np.eye(3) - eps).T)) / (2 * h)
        assert abs(-dE - out["virial"][k]) < 1e-6 * max(1.0, np.abs(out["virial"]).max())


@pytest.mark.parametrize("model", ["l3mix", "l3wide"])
def test_invariances_of_a_generated_model(model_dir, model):
    """the generator's couplings (pseudo-tensor paths included) give an invariant energy and covariant forces"""
    m = g3.Model3L(cases.model_file(model_dir, model))
    pos, cell, mu = _tiny_system(4)
    off, jj, rij = _bonds(pos, cell, 5.0)
    out = g3.compute_3l(m, mu, off, jj, rij)
    escale, fscale = max(1.0, abs(out["energy"])), max(1.0, np.abs(out["forces"]).max())
    q, _ = np.linalg.qr(np.random.default_rng(0).standard_normal((3, 3)))
    if np.linalg.det(q) < 0:
        q[:, 0] = -q[:, 0]
    rot = g3.compute_3l(m, mu, off, jj, rij @ q.T)
    assert abs(rot["energy"] - out["energy"]) < 1e-9 * escale
    assert np.abs(rot["forces"] - out["forces"] @ q.T).max() < 1e-9 * fscale
    inv = g3.compute_3l(m, mu, off, jj, -rij)                       # improper rotation: the energy is a scalar
    assert abs(inv["energy"] - out["energy"]) < 1e-9 * escale
    assert np.abs(inv["forces"] + out["forces"]).max() < 1e-9 * fscale
    # relabelling the atoms permutes the per-atom results
    n = len(mu)
    p = np.random.default_rng(1).permutation(n)                     # new atom a is old atom p[a]
    inv_p = np.argsort(p)
    off2 = np.concatenate([[0], np.cumsum(np.diff(off)[p])])
    rows = [np.arange(off[a], off[a + 1]) for a in p]
    sel = np.concatenate(rows)
    per = g3.compute_3l(m, mu[p], off2, inv_p[jj[sel]], rij[sel])
    assert abs(per["energy"] - out["energy"]) < 1e-10 * escale
    assert np.abs(per["forces"] - out["forces"][p]).max() < 1e-10 * fscale
    assert np.abs(per["energies"] - out["energies"][p]).max() < 1e-10 * escale


def test_isolated_atoms_and_zero_bond(model_dir):
    m = g3.Model3L(cases.model_file(model_dir, "l3mix"))
    mu = np.array([0, 1, 1])
    out = g3.compute_3l(m, mu, np.zeros(4, np.int64), np.zeros(0, np.int64), np.zeros((0, 3)))
    # no neighbours: every density is zero, rho_norm = 0, E_i = MLP(0) + 0 = 0 (no biases) plus the shift
    assert np.abs(out["energies"] - m.shift.numpy()[mu]).max() < 1e-14
    assert np.abs(out["forces"]).max() == 0.0
    with pytest.raises(go.ZeroBondError):
        g3.compute_3l(m, np.array([0, 0]), np.array([0, 1, 2]), np.array([1, 0]), np.zeros((2, 3)))
    # a bond outside the pair cutoff is dropped: Mo-W cutoff 4.5, W-W 4.25
    far = g3.compute_3l(m, np.array([1, 1]), np.array([0, 1, 2]), np.array([1, 0]), np.array([[4.3, 0, 0], [-4.3, 0, 0]]))
    assert np.abs(far["forces"]).max() == 0.0
