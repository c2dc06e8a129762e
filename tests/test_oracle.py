"""Pins of the CPU oracle (oracle/grace_oracle.py).  No GPU.

* end to end against the reference's own TensorFlow fp64 goldens (tests/golden/ref_fixtures/order3_tf.npz;
  recipe python/tests/test_ref_tf.py:43-55 of the reference): all stages of GRACE-1L at fp64 level;
* end to end against outputs of the compiled reference (fp32 + spline tables) on synthetic models with the AAAA
  stage, A width != FC width, pair cutoffs (tests/golden/reference_outputs.npz), at the reference's fp32-vs-fp64
  tolerances (python/tests/test_ref_tf.py:22-23);
* closed forms and invariants for the pieces: spherical harmonics, radial basis, MLP tangent, forces = -dE/dx,
  virial = strain derivative, rotation invariance.
"""
import os

import numpy as np
import pytest

import cases
from conftest import fixture_cell
from oracle import grace_oracle as go

TOL = {"energy": 1e-6, "forces": 2e-5, "energies": 1e-5, "stress": 1e-5}    # eV/atom, eV/A, eV, relative


@pytest.mark.parametrize("cell", ["W54", "WMo54", "W2tri"])
@pytest.mark.parametrize("name", ["grace_1l_order3", "legacy_1l_order3"])
def test_oracle_matches_tf_fp64(tf_gold, name, cell):
    m = go.Model1L(os.path.join(cases.REF_FIXTURES, name + ".npz"))
    types, offset, j, rij, vol = fixture_cell(cell)
    mu = np.array([m.names.index("Mo"), m.names.index("W")])[types - 1]
    out = go.compute_1l(m, mu, offset, j, rij)
    k = f"{name}/{cell}"
    n = len(types)
    assert abs(out["energy"] - tf_gold[k + "/energy"]) / n < 1e-10
    assert np.abs(out["forces"] - tf_gold[k + "/forces"]).max() < 1e-9
    assert np.abs(out["energies"] - tf_gold[k + "/energies"]).max() < 1e-10
    assert np.abs(go.virial_to_stress(out["virial"], vol) - tf_gold[k + "/stress"]).max() < 1e-10
    assert np.abs(tf_gold[k + "/forces"]).max() > 1e-2


@pytest.mark.parametrize("model,struct,rc", cases.E2E_CASES)
def test_oracle_matches_compiled_reference(model_dir, gold, model, struct, rc):
    m = go.Model1L(cases.model_file(model_dir, model))
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    types = np.minimum(types, m.n_elements)
    tag = f"e2e/{model}/{struct}"
    key = f"nl/{struct}@{float(gold[tag + '/rc_list']):g}"
    perm, offset, j, image, shifts = (gold[f"{key}/{k}"] for k in ("perm", "offset", "j", "image", "shifts"))
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    out = go.compute_1l(m, types[perm] - 1, offset, j, rij)
    n = len(types)
    assert abs(out["energy"] - gold[tag + "/energy"]) / n < TOL["energy"]
    assert np.abs(out["forces"] - gold[tag + "/forces"]).max() < TOL["forces"]
    assert np.abs(out["energies"] - gold[tag + "/energies"]).max() < TOL["energies"]
    assert np.abs(out["virial"] - gold[tag + "/virial"]).max() < TOL["stress"] * max(1.0, np.abs(gold[tag + "/virial"]).max())
    assert np.abs(gold[tag + "/forces"]).max() > 1e-2


def _unit(n, seed=0):
    u = np.random.default_rng(seed).standard_normal((n, 3))
    return u / np.linalg.norm(u, axis=1)[:, None]


def test_sh_closed_forms():
    u = _unit(40)
    Y, G = go.real_sh(u, 6)
    assert np.allclose(Y[:, 0], 1.0)
    s3 = np.sqrt(3.0)
    assert np.allclose(Y[:, 1], s3 * u[:, 1]) and np.allclose(Y[:, 2], s3 * u[:, 2]) and np.allclose(Y[:, 3], s3 * u[:, 0])
    # l = 2: sqrt(15) xy, sqrt(15) yz, sqrt(5)/2 (3z^2 - 1), sqrt(15) xz, sqrt(15)/2 (x^2 - y^2)
    x, y, z = u.T
    s15, s5 = np.sqrt(15.0), np.sqrt(5.0)
    assert np.allclose(Y[:, 4:9], np.stack([s15 * x * y, s15 * y * z, 0.5 * s5 * (3 * z * z - 1), s15 * x * z,
                                            0.5 * s15 * (x * x - y * y)], 1))
    for l in range(7):      # addition theorem
        assert np.allclose((Y[:, l * l:(l + 1) ** 2] ** 2).sum(1), 2 * l + 1)


def test_sh_gradient_is_derivative_of_polynomial_extension():
    rng = np.random.default_rng(1)
    v = rng.standard_normal((10, 3)) * 0.8
    _, G = go.real_sh(v, 5)
    h = 1e-6
    for d in range(3):
        e = np.zeros(3)
        e[d] = h
        fd = (go.real_sh(v + e, 5)[0] - go.real_sh(v - e, 5)[0]) / (2 * h)
        assert np.abs(fd - G[:, :, d]).max() < 1e-7


def test_sh_orthonormal_on_sphere():
    from grace_runtime_amd.synth import _sphere_quadrature
    u, w = _sphere_quadrature(14)
    Y, _ = go.real_sh(u, 6)
    assert np.abs(np.einsum("n,na,nb->ab", w, Y, Y) - np.eye(49)).max() < 1e-12


@pytest.mark.parametrize("p,nrb", [(16, 8), (5, 8), (16, 10), (1, 3)])
def test_radial_basis_closed_forms(p, nrb):
    x = np.linspace(0.0, 1.0, 41)
    g, dg = go.radial_basis(x, p, nrb)
    t = 2 * x - 1
    fc = 1 - 0.5 * (p + 1) * (p + 2) * x ** p + p * (p + 2) * x ** (p + 1) - 0.5 * p * (p + 1) * x ** (p + 2)
    for k in range(nrb):
        assert np.allclose(g[:, k], np.cos((k + 1) * np.arccos(np.clip(t, -1, 1))) * fc, atol=1e-12)
    assert np.abs(g[-1]).max() < 1e-12 and np.abs(dg[-1]).max() < 1e-9      # value and slope vanish at the cutoff
    assert np.allclose(g[0], [(-1) ** (k + 1) for k in range(nrb)])            # fc(0) = 1, T_k(-1) = (-1)^k
    h = 1e-6
    xm = x[1:-1]
    fd = (go.radial_basis(xm + h, p, nrb)[0] - go.radial_basis(xm - h, p, nrb)[0]) / (2 * h)
    assert np.abs(fd - dg[1:-1]).max() < 1e-6


@pytest.mark.parametrize("act", [0, 1])
def test_mlp_tangent(act):
    rng = np.random.default_rng(2)
    layers = [(rng.standard_normal((8, 16)), 0.35), (rng.standard_normal((16, 16)), 0.25), (rng.standard_normal((16, 6)), 0.25)]
    x = np.linspace(0.1, 0.9, 9)
    f = lambda xx: go.mlp_value_tangent(layers, *go.radial_basis(xx, 16, 8), act)
    out, dout = f(x)
    h = 1e-6
    fd = (f(x + h)[0] - f(x - h)[0]) / (2 * h)
    assert np.abs(fd - dout).max() < 1e-7
    # one layer, linear: plain matrix product
    o1, _ = go.mlp_value_tangent(layers[2:], np.ones((1, 16)), np.zeros((1, 16)), act)
    assert np.allclose(o1, layers[2][0].sum(0) * 0.25)


def _w2tri_energy(m, mu, pos, cell, rc):
    from grace_runtime_amd.kk import neighbor_search
    perm, offset, j, image, shifts = neighbor_search(pos, cell, [1, 1, 1], rc)
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    out = go.compute_1l(m, mu[perm], offset, j, rij)
    f = np.empty_like(out["forces"])
    f[perm] = out["forces"]
    return out["energy"], f, out["virial"]


def test_forces_and_virial_are_energy_derivatives(model_dir):
    m = go.Model1L(cases.model_file(model_dir, "mix2"))
    pos, cell, pbc, types = cases.structure_triclinic()
    mu = types - 1
    E0, F, W = _w2tri_energy(m, mu, pos, cell, m.rcut)
    assert np.abs(F.sum(0)).max() < 1e-12
    h = 1e-5
    for (a, d) in [(0, 0), (3, 1), (7, 2), (11, 0)]:
        p1, p2 = pos.copy(), pos.copy()
        p1[a, d] += h
        p2[a, d] -= h
        fd = -(_w2tri_energy(m, mu, p1, cell, m.rcut)[0] - _w2tri_energy(m, mu, p2, cell, m.rcut)[0]) / (2 * h)
        assert abs(fd - F[a, d]) < 1e-7
    # virial = -dE/d(strain): W_ab = - sum_bonds ... ; check with a symmetric strain
    for (a, b, k) in [(0, 0, 0), (1, 1, 1), (0, 1, 3), (1, 2, 5)]:
        def e_of(eps):
            S = np.eye(3)
            S[a, b] += eps
            if a != b:
                S[b, a] += eps
            return _w2tri_energy(m, mu, pos @ S.T, cell @ S.T, m.rcut)[0]
        dE = (e_of(h) - e_of(-h)) / (2 * h)
        want = -W[k] * (1.0 if a == b else 2.0)
        assert abs(dE - want) < 1e-6, (a, b, dE, want)


def test_rotation_and_permutation_invariance(model_dir):
    m = go.Model1L(cases.model_file(model_dir, "mix2"))
    pos, cell, pbc, types = cases.structure_triclinic()
    mu = types - 1
    E0, F0, _ = _w2tri_energy(m, mu, pos, cell, m.rcut)
    Q, _ = np.linalg.qr(np.random.default_rng(4).standard_normal((3, 3)))
    E1, F1, _ = _w2tri_energy(m, mu, pos @ Q.T, cell @ Q.T, m.rcut)
    assert abs(E0 - E1) < 1e-10 and np.abs(F0 @ Q.T - F1).max() < 1e-10
    p = np.random.default_rng(5).permutation(len(pos))
    E2, F2, _ = _w2tri_energy(m, mu[p], pos[p], cell, m.rcut)
    assert abs(E0 - E2) < 1e-10 and np.abs(F0[p] - F2).max() < 1e-10


def test_isolated_atom_and_zero_bond(model_dir):
    m = go.Model1L(cases.model_file(model_dir, "mix2"))
    out = go.compute_1l(m, np.array([1]), np.array([0, 0]), np.zeros(0, int), np.zeros((0, 3)))
    # no bonds: A = 0, rho = 0, E = MLP(0) * scale + shift = shift (tests/test_driver.cpp:432-440 of the reference)
    assert abs(out["energy"] - m.shift[1]) < 1e-14 and np.all(out["forces"] == 0)
    with pytest.raises(go.ZeroBondError):
        go.compute_1l(m, np.array([0, 0]), np.array([0, 1, 2]), np.array([1, 0]), np.zeros((2, 3)))
