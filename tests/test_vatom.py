"""Per-atom virials of the CPU oracles (Outputs::vatom of the reference, libgrace/include/grace/system.h:71; add_vatom,
fused_cpu.h:1075-1087: half of every bond's (x_i - x_j) (x) f_i to each of its two atoms).  No GPU.  Pinned by the
compiled reference's vatom on a 1L, a 2L and a 3L model (tests/golden/reference_outputs.npz, at its fp32 gate), by the sum
rule (the rows add up to the total virial) and by a brute-force restatement from bond forces obtained by differences."""
import numpy as np
import pytest

import cases
from oracle import grace_oracle as g1
from oracle import grace_oracle_2l as g2
from oracle import grace_oracle_3l as g3


def _oracle(model_dir, model):
    path = cases.model_file(model_dir, model)
    layers = cases.LAYERS[model]
    if layers == 1:
        return g1.Model1L(path), g1.compute_1l
    if layers == 2:
        return g2.Model2L(path), g2.compute_2l
    return g3.Model3L(path), g3.compute_3l


@pytest.mark.parametrize("model,struct,rc", cases.VATOM_CASES)
def test_oracle_virials_match_the_compiled_reference(model_dir, gold, model, struct, rc):
    m, compute = _oracle(model_dir, model)
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    types = np.minimum(types, m.n_elements)
    tag = f"e2e/{model}/{struct}"
    key = f"nl/{struct}@{float(gold[tag + '/rc_list']):g}"
    perm, offset, j, image, shifts = (gold[f"{key}/{k}"] for k in ("perm", "offset", "j", "image", "shifts"))
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    out = compute(m, types[perm] - 1, offset, j, rij)
    ref = gold[tag + "/virials"]
    scale = max(1.0, np.abs(ref).max())
    assert np.abs(ref).max() > 1e-3
    assert np.abs(out["virials"] - ref).max() < 2e-5 * scale                       # the reference runs fp32 + spline tables
    assert np.abs(out["virials"].sum(0) - out["virial"]).max() < 1e-11 * max(1.0, np.abs(out["virial"]).max())


def test_virials_from_bond_forces_by_differences(model_dir):
    """a restatement that does not use the oracle's virial code: the force of bond b on its central atom is dE/d r_ij[b] of
    an energy that takes the bond vectors as independent variables (central differences on a sample; for all bonds read off
    the oracle's atom forces by re-targeting the bond at a fictitious atom, which then receives minus the bond force); half
    of (x_i - x_j) (x) f goes to each atom of the bond"""
    from test_oracle_2l import _bonds, _tiny_system
    m = g1.Model1L(cases.model_file(model_dir, "mix2"))
    pos, cell, mu = _tiny_system()
    offset, j, rij = _bonds(pos, cell, 5.0)
    n = len(mu)
    out = g1.compute_1l(m, mu, offset, j, rij)
    bi = np.repeat(np.arange(n), np.diff(offset))
    mu2 = np.concatenate([mu, [0]])
    off2 = np.concatenate([offset, [offset[-1]]])
    fb = np.zeros((len(j), 3))
    for b in range(len(j)):
        j2 = j.copy()
        mu2[-1] = mu[j[b]]              # the element of the neighbour decides the radial functions
        j2[b] = n
        fb[b] = -g1.compute_1l(m, mu2, off2, j2, rij)["forces"][n]
    h = 1e-5
    for b in range(0, len(j), 17):
        for d in range(3):
            rp, rm = rij.copy(), rij.copy()
            rp[b, d] += h
            rm[b, d] -= h
            fd = (g1.compute_1l(m, mu, offset, j, rp, want_forces=False)["energy"] -
                  g1.compute_1l(m, mu, offset, j, rm, want_forces=False)["energy"]) / (2 * h)
            assert abs(fd - fb[b, d]) < 1e-7 * max(1.0, np.abs(fb).max())
    dl = -rij
    v6 = 0.5 * np.stack([dl[:, 0] * fb[:, 0], dl[:, 1] * fb[:, 1], dl[:, 2] * fb[:, 2], dl[:, 0] * fb[:, 1], dl[:, 0] * fb[:, 2],
                         dl[:, 1] * fb[:, 2]], axis=1)
    rows = np.zeros((n, 6))
    np.add.at(rows, bi, v6)
    np.add.at(rows, j, v6)
    assert np.abs(rows).max() > 1e-3
    assert np.abs(rows - out["virials"]).max() < 1e-12 * max(1.0, np.abs(rows).max())


# index of component (a, b) in the centroid form xx yy zz xy xz yz yx zx zy (cvatom, kk/grace_1l_kk_impl.h:1344-1362)
CENTROID = {(0, 0): 0, (1, 1): 1, (2, 2): 2, (0, 1): 3, (0, 2): 4, (1, 2): 5, (1, 0): 6, (2, 0): 7, (2, 1): 8}


def permuted_centroid(cv, p):
    """the centroid rows of the structure with axes x'_a = x_p[a]: W'_ab = W_p[a]p[b]"""
    out = np.empty_like(cv)
    for (a, b), k in CENTROID.items():
        out[:, k] = cv[:, CENTROID[(p[a], p[b])]]
    return out


def test_centroid_form_of_the_1l_oracle(model_dir, gold):
    """the three components below the diagonal: equal to those above it of the structure with its axes exchanged (the model
    is invariant under any permutation of the axes), and the nine columns add up to the full tensor sum dl (x) f"""
    model, struct = "mix2", "alloy54"
    m, compute = _oracle(model_dir, model)
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    tag = f"e2e/{model}/{struct}"
    key = f"nl/{struct}@{float(gold[tag + '/rc_list']):g}"
    perm, offset, j, image, shifts = (gold[f"{key}/{k}"] for k in ("perm", "offset", "j", "image", "shifts"))
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    out = compute(m, types[perm] - 1, offset, j, rij)
    cv = out["centroid_virials"]
    assert cv.shape == (len(pos), 9) and np.array_equal(cv[:, :6], out["virials"])
    assert np.abs(cv[:, 6:] - cv[:, 3:6]).max() > 1e-6          # a bond's tensor is not symmetric: the lower half says something
    scale = max(1.0, np.abs(cv).max())
    for p in ([1, 0, 2], [1, 2, 0], [2, 1, 0]):
        outp = compute(m, types[perm] - 1, offset, j, rij[:, p])
        assert abs(outp["energy"] - out["energy"]) < 1e-10 * max(1.0, abs(out["energy"]))
        assert np.abs(outp["centroid_virials"] - permuted_centroid(cv, p)).max() < 1e-10 * scale
    # the total tensor is symmetric (rotational invariance of the energy) although the rows are not
    tot = cv.sum(0)
    assert np.abs(tot[6:] - tot[3:6]).max() < 1e-9 * max(1.0, np.abs(tot).max())
