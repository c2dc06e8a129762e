"""Atoms with few and uneven numbers of bonds through the GRACE-2L and GRACE-3L engines against the CPU oracle.  The
neighbour gather and its reverse walk an atom's bonds in chunks of 4 or 8 that are copied to LDS one chunk ahead: a
dilute, non-periodic cloud gives atoms with 0, 1, 2 ... bonds, so every length of a last chunk, the single-chunk atoms
and the atoms without any bond occur in one structure (reference behaviour: atom_yi / bond_yi_bwd of
libgrace/include/grace/fused_cpu.h:836-1025 loop over whatever bonds an atom has).  Needs an MI355X: run with -m gpu."""
import numpy as np
import pytest

import cases
from grace_runtime_amd import kk
from oracle import grace_oracle_2l as g2
from oracle import grace_oracle_3l as g3

pytestmark = pytest.mark.gpu

F64 = {"energy": 1e-10, "forces": 1e-9, "energies": 1e-10, "virial": 1e-9}
F32 = {"energy": 1e-6, "forces": 2e-5, "energies": 1e-5, "virial": 1e-5}


def dilute_cloud(n=110, box=20.0, dmin=1.7, seed=13):
    """n atoms of two types at random in a box of `box` A, no two closer than dmin, no periodicity"""
    rng = np.random.default_rng(seed)
    pos = []
    while len(pos) < n:
        p = rng.uniform(0, box, 3)
        if all(np.linalg.norm(p - q) >= dmin for q in pos):
            pos.append(p)
    return np.array(pos), np.zeros((3, 3)), np.array([False, False, False]), rng.integers(1, 3, size=n).astype(np.int32)


def _check(out, ref, n, tol):
    fs = max(1.0, np.abs(ref["forces"]).max())
    assert abs(out["energy"] - ref["energy"]) / n < tol["energy"] * fs
    assert np.abs(out["forces"] - ref["forces"]).max() < tol["forces"] * fs
    assert np.abs(out["energies"] - ref["energies"]).max() < tol["energies"] * fs
    assert np.abs(out["virial"] - ref["virial"]).max() < tol["virial"] * max(1.0, np.abs(ref["virial"]).max())


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("model,layers", [("l2mix", 2), ("l3mix", 3)])
def test_atoms_with_zero_to_many_bonds(model_dir, model, layers, precision):
    path = cases.model_file(model_dir, model)
    if layers == 2:
        om = g2.Model2L(path)
        names, oracle = om.names, g2.compute_2l
    else:
        om = g3.Model3L(path)
        names, oracle = [x.decode() for x in om.d["element_names"]], g3.compute_3l
    eng = kk.Engine(kk.Model(path), names, precision)
    pos, cell, pbc, types = dilute_cloud()
    rc = eng.cutoff(1, 2)
    pcell, shift = kk._padded_cell_arrays(cell, pos, rc, pbc)
    perm, offset, j, image, shifts = kk.neighbor_search(pos + shift, pcell, pbc, rc)
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    r = np.linalg.norm(rij, axis=1)
    keep_deg = np.bincount(np.repeat(np.arange(len(pos)), np.diff(offset))[r < rc], minlength=len(pos))
    # the cloud is dilute enough for the short ends: atoms without a bond, with one, and every remainder of a chunk of 4
    assert keep_deg.min() == 0 and 1 in keep_deg and {d % 4 for d in keep_deg} == {0, 1, 2, 3} and keep_deg.max() >= 9
    n = len(types)
    out = eng.compute(types[perm], offset, j, rij, energies=True)
    _check(out, oracle(om, types[perm] - 1, offset, j, rij), n, F64 if precision == 64 else F32)
    assert np.abs(out["forces"].sum(0)).max() < 1e-9 * max(1.0, np.abs(out["forces"]).max())
