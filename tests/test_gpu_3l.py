"""Parity of the HIP GRACE-3L path (through the C ABI, grace_runtime_amd.kk -> libgrace_hip.so) with the CPU oracle
and the outputs of the compiled reference.  Needs an MI355X: run with -m gpu.

Tolerances.  The fp64 engine (precision 64): against the fp64 oracle the north-star bounds are 1e-6 eV/atom, 1e-5 eV/A,
1e-6 eV/A^3, the tests hold it to 1e-10 eV/atom, 1e-9 eV/A (scaled by the largest force of the case where that exceeds
1 eV/A), 1e-10 eV per atom energy: summation order only (the message adjoints of the neighbours and the bond forces are
summed with atomic adds, so the last bits vary from run to run).  Against the compiled reference (fp32 + spline tables):
its own fp32-vs-fp64 gate, 1e-6 eV/atom, 2e-5 eV/A, 1e-5 eV, 1e-5 relative (python/tests/test_ref_tf.py:22-23).  The
fp32 engine (precision 32: network arithmetic in fp32, geometry, norms, readout, forces and sums in fp64) is held to
that same fp32 gate against the fp64 oracle.  The
reference checkout holds no GRACE-3L model, so all models here are generated (grace_runtime_amd/synth.py)."""
import os

import numpy as np
import pytest

import cases
from grace_runtime_amd import kk
from oracle import grace_oracle_3l as g3

pytestmark = pytest.mark.gpu

F64 = {"energy": 1e-10, "forces": 1e-9, "energies": 1e-10, "virial": 1e-9}
F32 = {"energy": 1e-6, "forces": 2e-5, "energies": 1e-5, "virial": 1e-5}


def _check(out, ref, n, tol):
    fs = max(1.0, np.abs(ref["forces"]).max())
    assert abs(out["energy"] - ref["energy"]) / n < tol["energy"] * fs
    assert np.abs(out["forces"] - ref["forces"]).max() < tol["forces"] * fs
    if "energies" in out and "energies" in ref:
        assert np.abs(out["energies"] - ref["energies"]).max() < tol["energies"] * fs
    assert np.abs(out["virial"] - ref["virial"]).max() < tol["virial"] * max(1.0, np.abs(ref["virial"]).max())


def _names(om):
    return [x.decode() for x in om.d["element_names"]]


@pytest.fixture(scope="module")
def engines(model_dir):
    cache = {}

    def get(name, precision=64):
        if (name, precision) not in cache:
            path = cases.model_file(model_dir, name)
            om = g3.Model3L(path)
            cache[(name, precision)] = (kk.Engine(kk.Model(path), _names(om), precision), om)
        return cache[(name, precision)]
    return get


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("model,struct,rc", cases.E2E_CASES_3L)
def test_matches_oracle_and_compiled_reference(engines, gold, model, struct, rc, precision):
    eng, om = engines(model, precision)
    assert eng.model.layers == 3
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    types = np.minimum(types, om.n_elements).astype(np.int32)
    tag = f"e2e/{model}/{struct}"
    rcl = float(gold[tag + "/rc_list"])
    pcell, shift = kk._padded_cell_arrays(cell, pos, rcl, pbc)
    perm, offset, j, image, shifts = kk.neighbor_search(pos + shift, pcell, pbc, rcl)
    n = len(types)
    out = eng.compute(types[perm], offset, j, energies=True, positions=pos[perm], image=image, shifts=shifts)
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    out2 = eng.compute(types[perm], offset, j, rij, energies=True)
    same = 1e-9 if precision == 64 else 1e-5      # the two geometry inputs differ in the last bits of the bond vectors
    assert abs(out["energy"] - out2["energy"]) < same * n and np.abs(out["forces"] - out2["forces"]).max() < same
    _check(out, g3.compute_3l(om, types[perm] - 1, offset, j, rij), n, F64 if precision == 64 else F32)
    _check(out, {k: gold[f"{tag}/{k}"] for k in ("energy", "energies", "forces", "virial")}, n, F32)
    assert np.abs(out["forces"].sum(0)).max() < 1e-9 * max(1.0, np.abs(out["forces"]).max())
    eo = eng.compute(types[perm], offset, j, rij, energy_only=True)
    assert abs(eo["energy"] - out["energy"]) < (1e-10 if precision == 64 else 1e-6) * max(1.0, abs(out["energy"])) and "forces" not in eo


@pytest.mark.parametrize("precision", [64, 32])
def test_padded_channel_widths(engines, precision):
    """20 radial channels in 32-wide tensors, 24 hidden units in 64-wide MFMA tiles, messages up to l = 1"""
    eng, om = engines("l3pad", precision)
    pos, cell, pbc, types = cases.structure_alloy54()
    perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, 5.0)
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    out = eng.compute(types[perm], offset, j, rij, energies=True)
    _check(out, g3.compute_3l(om, types[perm] - 1, offset, j, rij), len(types), F64 if precision == 64 else F32)


def test_properties_at_benchmark_shape(engines):
    """the benchmark model (lmax 5, 64 channels, 8 of 89 species) on 1500 atoms of the amorphous cube: against the oracle
    on a sample is too slow on the CPU, so size-independent properties: Newton's third law, checksum of the per-atom
    energies, translation, relabelling of the atoms, and a 2 x 1 x 1 replica has twice the energy and the same forces"""
    eng, om = engines("config4")
    pos, cell, pbc, types = cases.structure_config4(natoms=1500)

    def run(p, c, t, **kw):
        perm, offset, j, image, shifts = kk.neighbor_search(p, c, pbc, 6.0)
        out = eng.compute(t[perm], offset, j, positions=p[perm], image=image, shifts=shifts, **kw)
        f = np.empty_like(p)
        f[perm] = out["forces"]
        return out, f, len(j)

    o1, f1, nb1 = run(pos, cell, types, energies=True)
    fs, es = max(1.0, np.abs(f1).max()), max(1.0, abs(o1["energy"]))
    assert np.abs(f1).max() > 1e-2
    assert np.abs(f1.sum(0)).max() < 1e-8 * fs
    assert abs(o1["energies"].sum() - o1["energy"]) < 1e-9 * es
    o2, f2, _ = run(pos + np.array([0.4, -1.3, 2.2]), cell, types)
    assert abs(o2["energy"] - o1["energy"]) < 1e-9 * es and np.abs(f2 - f1).max() < 1e-8 * fs
    p = np.random.default_rng(0).permutation(len(pos))
    o3, f3, _ = run(pos[p], cell, types[p])
    assert abs(o3["energy"] - o1["energy"]) < 1e-9 * es and np.abs(f3 - f1[p]).max() < 1e-8 * fs
    c2 = cell * np.array([[2.0], [1.0], [1.0]])
    o4, f4, nb4 = run(np.concatenate([pos, pos + cell[0]]), c2, np.tile(types, 2))
    assert nb4 == 2 * nb1
    assert abs(o4["energy"] - 2 * o1["energy"]) < 1e-9 * es and np.abs(f4 - np.tile(f1, (2, 1))).max() < 1e-8 * fs
    assert np.abs(o4["virial"] - 2 * o1["virial"]).max() < 1e-8 * max(1.0, np.abs(o1["virial"]).max())


@pytest.mark.parametrize("precision", [64, 32])
def test_benchmark_model_against_oracle_on_a_small_cell(engines, precision):
    """the full-size model against the oracle on 40 atoms (the oracle needs a few seconds for it)"""
    eng, om = engines("config4", precision)
    pos, cell, pbc, types = cases.structure_config4(natoms=40, seed=11)
    perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, 6.0)
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    out = eng.compute(types[perm], offset, j, rij, energies=True)
    _check(out, g3.compute_3l(om, types[perm] - 1, offset, j, rij), len(types), F64 if precision == 64 else F32)


def test_finite_differences_on_gpu(engines):
    eng, om = engines("l3mix")
    pos, cell, pbc, types = cases.structure_triclinic()
    sysm = kk.System(eng.model, ["Mo", "W"], skin=0.0)

    def energy(p):
        return sysm.compute(types, p, cell, pbc, energy_only=True)["energy"]
    r = sysm.compute(types, pos, cell, pbc)
    h = 1e-5
    for a, d in [(0, 0), (5, 1), (9, 2)]:
        p1, p2 = pos.copy(), pos.copy()
        p1[a, d] += h
        p2[a, d] -= h
        assert abs(-(energy(p1) - energy(p2)) / (2 * h) - r["forces"][a, d]) < 1e-6 * max(1.0, np.abs(r["forces"]).max())


def test_edge_cases(engines):
    eng, om = engines("l3mix")
    out = eng.compute(np.zeros(0, np.int32), np.zeros(1, np.int64), np.zeros(0, np.int32), np.zeros((0, 3)))
    assert out["energy"] == 0.0 and out["forces"].shape == (0, 3)
    t2 = np.array([1, 2], np.int32)
    out = eng.compute(t2, np.zeros(3, np.int64), np.zeros(0, np.int32), np.zeros((0, 3)), energies=True)
    ref = g3.compute_3l(om, t2 - 1, np.zeros(3, np.int64), np.zeros(0, np.int64), np.zeros((0, 3)))
    assert abs(out["energy"] - ref["energy"]) < 1e-12 and np.all(out["forces"] == 0) and np.all(out["virial"] == 0)
    # ragged rows: atom 1 has no bonds of its own but is a neighbour (it receives message adjoints and a reaction force);
    # a bond beyond the cutoff is dropped; atom 3 is isolated
    types = np.array([1, 2, 1, 2], np.int32)
    offset = np.array([0, 3, 3, 4, 4], np.int64)
    j = np.array([2, 1, 3, 0], np.int32)
    rij = np.array([[1.5, 0.3, -0.2], [0.4, 2.0, 0.9], [9.0, 0, 0], [-1.5, -0.3, 0.2]])
    out = eng.compute(types, offset, j, rij, energies=True)
    assert eng.edge_count() == 3
    _check(out, g3.compute_3l(om, types - 1, offset, j, rij), 4, F64)
    assert np.abs(out["forces"][1]).max() > 1e-3 and out["forces"][3].tolist() == [0, 0, 0]
    with pytest.raises(RuntimeError, match="two atoms at the same position"):
        eng.compute(np.array([1, 1], np.int32), np.array([0, 1, 2], np.int64), np.array([1, 0], np.int32), np.zeros((2, 3)))
    again = eng.compute(types, offset, j, rij)
    assert abs(again["energy"] - out["energy"]) < 1e-12
    with pytest.raises(ValueError, match="precision must be 64 or 32"):
        kk.Engine(eng.model, ["Mo", "W"], 16)


def test_system_and_batch(engines):
    eng, om = engines("l3mix")
    pos, cell, pbc, types = cases.structure_alloy54()
    s = kk.System(eng.model, ["Mo", "W"], skin=0.5)
    s.compute(types, pos, cell, pbc)
    p1 = pos + np.random.default_rng(0).uniform(-0.1, 0.1, pos.shape)
    r1 = s.compute(types, p1, cell, pbc)
    assert s.rebuilds == 1
    r1x = kk.System(eng.model, ["Mo", "W"], skin=0.0).compute(types, p1, cell, pbc)
    fs = np.abs(r1x["forces"]).max()
    assert abs(r1["energy"] - r1x["energy"]) < 1e-9 and np.abs(r1["forces"] - r1x["forces"]).max() < 1e-9 * fs
    structs = [cases.structure_alloy54(), cases.structure_triclinic(), cases.structure_slab(), cases.structure_molecule()]
    b = kk.Batch(eng.model, ["Mo", "W"])
    out = b.compute([len(x[0]) for x in structs], np.concatenate([x[3] for x in structs]), np.concatenate([x[0] for x in structs]),
                    np.stack([x[1] for x in structs]), np.stack([x[2] for x in structs]), energies=True)
    assert b.passes == 1
    lo = 0
    for k, (p, c, pb, t) in enumerate(structs):
        one = kk.System(eng.model, ["Mo", "W"], skin=0.0).compute(t, p, c, pb)
        assert abs(out["energy"][k] - one["energy"]) < 1e-9
        assert np.abs(out["forces"][lo:lo + len(p)] - one["forces"]).max() < 1e-9 * max(1.0, np.abs(one["forces"]).max())
        assert np.abs(out["virial"][k] - one["virial"]).max() < 1e-9 * max(1.0, np.abs(one["virial"]).max())
        assert abs(out["energies"][lo:lo + len(p)].sum() - out["energy"][k]) < 1e-9
        lo += len(p)
