"""Parity of the HIP GRACE-2L path (through the C ABI, grace_runtime_amd.kk -> libgrace_hip.so) with the CPU oracle
and the golden vectors.  Needs an MI355X: run with -m gpu.

Tolerances.  The fp64 engine (precision 64): against the fp64 oracle and the TF fp64 goldens the north-star bounds are
1e-6 eV/atom, 1e-5 eV/A, 1e-6 eV/A^3, the tests hold it to 1e-10 eV/atom, 1e-9 eV/A (scaled by the largest force of
the case where that exceeds 1 eV/A), 1e-10 eV per atom energy: summation order only (the dE/dI rows of the neighbours
are summed with atomic adds, so the last bits vary from run to run).  Against the compiled reference (fp32 + spline
tables): its own fp32-vs-fp64 gate, 1e-6 eV/atom, 2e-5 eV/A, 1e-5 eV, 1e-5 relative (python/tests/test_ref_tf.py:22-23).
The fp32 engine (precision 32: network arithmetic in fp32, geometry, readout, forces and sums in fp64) is held to that
same fp32 gate against the fp64 oracle and the TF fp64 goldens."""
import os

import numpy as np
import pytest

import cases
from conftest import fixture_cell
from grace_runtime_amd import kk
from oracle import grace_oracle as go
from oracle import grace_oracle_2l as g2

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


@pytest.fixture(scope="module")
def engines(model_dir):
    cache = {}

    def get(name, species, fixture=False, precision=64):
        key = (name, tuple(species), precision)
        if key not in cache:
            path = (os.path.join(cases.REF_FIXTURES, name + ".npz") if fixture else cases.model_file(model_dir, name))
            cache[key] = kk.Engine(kk.Model(path), species, precision)
        return cache[key]
    return get


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("cell", ["W54", "WMo54", "W2tri"])
@pytest.mark.parametrize("name", ["grace_2l_order3", "legacy_2l_order3"])
def test_matches_tf_fp64_goldens(engines, tf_gold, name, cell, precision):
    eng = engines(name, ["Mo", "W"], True, precision)
    assert eng.model.layers == 2
    types, offset, j, rij, vol = fixture_cell(cell)
    out = eng.compute(types, offset, j, rij, energies=True)
    k = f"{name}/{cell}"
    n = len(types)
    tol = F64 if precision == 64 else F32
    assert abs(out["energy"] - tf_gold[k + "/energy"]) / n < tol["energy"]
    assert np.abs(out["forces"] - tf_gold[k + "/forces"]).max() < tol["forces"]
    assert np.abs(out["energies"] - tf_gold[k + "/energies"]).max() < tol["energies"]
    # eV/A^3 (north star 1e-6)
    assert np.abs(go.virial_to_stress(out["virial"], vol) - tf_gold[k + "/stress"]).max() < (1e-10 if precision == 64 else 1e-7)


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("model,cell", cases.FIXTURE_CASES_2L)
def test_fixture_models_match_oracle_and_compiled_reference(engines, gold, model, cell, precision):
    """the reference's 2L fixture models with the AAAA / BBBB stages, lmax 1 .. 3, widths 8 .. 40"""
    eng = engines(model, ["Mo", "W"], True, precision)
    om = g2.Model2L(os.path.join(cases.REF_FIXTURES, model + ".npz"))
    types, offset, j, rij, _ = fixture_cell(cell)
    out = eng.compute(types, offset, j, rij, energies=True)
    mu = np.array([om.names.index("Mo"), om.names.index("W")])[types - 1]
    _check(out, g2.compute_2l(om, mu, offset, j, rij), len(types), F64 if precision == 64 else F32)
    tag = f"fixture/{model}/{cell}"
    _check(out, {k: gold[f"{tag}/{k}"] for k in ("energy", "energies", "forces", "virial")}, len(types), F32)


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("model,struct,rc", cases.E2E_CASES_2L)
def test_matches_oracle_and_compiled_reference(engines, model_dir, gold, model, struct, rc, precision):
    om = g2.Model2L(cases.model_file(model_dir, model))
    eng = engines(model, om.names, False, precision)
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
    _check(out, g2.compute_2l(om, types[perm] - 1, offset, j, rij), n, F64 if precision == 64 else F32)
    _check(out, {k: gold[f"{tag}/{k}"] for k in ("energy", "energies", "forces", "virial")}, n, F32)
    assert np.abs(out["forces"].sum(0)).max() < 1e-9 * max(1.0, np.abs(out["forces"]).max())


def test_supercell_properties_at_benchmark_shape(engines):
    """the benchmark model on 4000 atoms (312 k edges): a 2 x 2 x 2 replica of a periodic cell has 8 x its energy and
    the same forces; Newton's third law; translation; checksum of the per-atom energies"""
    eng = engines("config3", ["Al", "Co", "Ni", "Ti"])
    from grace_runtime_amd import synth
    p0, c0 = synth.fcc_supercell(3.6, 5)
    p0 = synth.jitter(p0, 0.08, 9)
    t0 = np.random.default_rng(9).integers(1, 5, len(p0)).astype(np.int32)
    pbc = np.array([True, True, True])

    def run(pos, cell, types, **kw):
        perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, 6.0)
        out = eng.compute(types[perm], offset, j, positions=pos[perm], image=image, shifts=shifts, **kw)
        f = np.empty_like(pos)
        f[perm] = out["forces"]
        return out, f, len(j)

    o1, f1, nb1 = run(p0, c0, t0, energies=True)
    reps = [(a, b, c) for a in range(2) for b in range(2) for c in range(2)]
    p8 = np.concatenate([p0 + np.array(r) @ c0 for r in reps])
    o8, f8, nb8 = run(p8, 2 * c0, np.tile(t0, 8))
    assert nb8 == 8 * nb1 and eng.edge_count() == nb8
    fs = max(1.0, np.abs(f1).max())
    assert abs(o8["energy"] - 8 * o1["energy"]) < 1e-9 * abs(o1["energy"])
    assert np.abs(f8 - np.tile(f1, (8, 1))).max() < 1e-9 * fs
    assert np.abs(o8["virial"] - 8 * o1["virial"]).max() < 1e-9 * np.abs(o1["virial"]).max() * 8
    assert np.abs(f8.sum(0)).max() < 1e-8 * fs
    assert abs(o1["energies"].sum() - o1["energy"]) < 1e-9 * abs(o1["energy"])
    o2, f2, _ = run(p0 + np.array([0.4, -1.3, 2.2]), c0, t0)
    assert abs(o2["energy"] - o1["energy"]) < 1e-9 * abs(o1["energy"]) and np.abs(f2 - f1).max() < 1e-9 * fs


def test_finite_differences_on_gpu(engines):
    eng = engines("l2mix", ["Mo", "W"])
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
    eng = engines("l2mix", ["Mo", "W"])
    om = g2.Model2L(eng.model.path)
    out = eng.compute(np.zeros(0, np.int32), np.zeros(1, np.int64), np.zeros(0, np.int32), np.zeros((0, 3)))
    assert out["energy"] == 0.0 and out["forces"].shape == (0, 3)
    # isolated atoms: no bonds, no forces; the energy is the readout of zero densities
    t2 = np.array([1, 2], np.int32)
    out = eng.compute(t2, np.zeros(3, np.int64), np.zeros(0, np.int32), np.zeros((0, 3)), energies=True)
    ref = g2.compute_2l(om, t2 - 1, np.zeros(3, np.int64), np.zeros(0, np.int64), np.zeros((0, 3)))
    assert abs(out["energy"] - ref["energy"]) < 1e-12 and np.all(out["forces"] == 0) and np.all(out["virial"] == 0)
    # ragged rows: atoms without bonds between atoms with bonds; a bond beyond the cutoff is dropped.  Atom 1 has no
    # bonds of its own but is a neighbour: it receives dE/dI and a reaction force
    types = np.array([1, 2, 1, 2], np.int32)
    offset = np.array([0, 3, 3, 4, 4], np.int64)
    j = np.array([2, 1, 3, 0], np.int32)
    rij = np.array([[1.5, 0.3, -0.2], [0.4, 2.0, 0.9], [9.0, 0, 0], [-1.5, -0.3, 0.2]])
    out = eng.compute(types, offset, j, rij, energies=True)
    assert eng.edge_count() == 3
    _check(out, g2.compute_2l(om, types - 1, offset, j, rij), 4, F64)
    assert np.abs(out["forces"][1]).max() > 1e-3 and out["forces"][3].tolist() == [0, 0, 0]
    eo = eng.compute(types, offset, j, rij, energy_only=True)
    assert abs(eo["energy"] - out["energy"]) < 1e-12 and "forces" not in eo
    with pytest.raises(RuntimeError, match="two atoms at the same position"):
        eng.compute(np.array([1, 1], np.int32), np.array([0, 1, 2], np.int64), np.array([1, 0], np.int32), np.zeros((2, 3)))
    again = eng.compute(types, offset, j, rij)
    assert abs(again["energy"] - out["energy"]) < 1e-12
    with pytest.raises(ValueError, match="precision must be 64 or 32"):
        kk.Engine(eng.model, ["Mo", "W"], 16)


@pytest.mark.parametrize("precision", [64, 32])
def test_system_and_batch(engines, precision):
    eng = engines("l2mix", ["Mo", "W"])
    pos, cell, pbc, types = cases.structure_alloy54()
    tol = 1e-9 if precision == 64 else 2e-5      # fp32: the skin list and the batch change the summation order of fp32 sums
    s = kk.System(eng.model, ["Mo", "W"], skin=0.5, precision=precision)
    s.compute(types, pos, cell, pbc)
    p1 = pos + np.random.default_rng(0).uniform(-0.1, 0.1, pos.shape)
    r1 = s.compute(types, p1, cell, pbc)
    assert s.rebuilds == 1
    r1x = kk.System(eng.model, ["Mo", "W"], skin=0.0, precision=precision).compute(types, p1, cell, pbc)
    fs = np.abs(r1x["forces"]).max()
    assert abs(r1["energy"] - r1x["energy"]) < tol * len(pos) and np.abs(r1["forces"] - r1x["forces"]).max() < tol * fs
    structs = [cases.structure_alloy54(), cases.structure_triclinic(), cases.structure_slab()]
    b = kk.Batch(eng.model, ["Mo", "W"], precision=precision)
    out = b.compute([len(x[0]) for x in structs], np.concatenate([x[3] for x in structs]), np.concatenate([x[0] for x in structs]),
                    np.stack([x[1] for x in structs]), np.stack([x[2] for x in structs]))
    lo = 0
    for k, (p, c, pb, t) in enumerate(structs):
        one = kk.System(eng.model, ["Mo", "W"], skin=0.0, precision=precision).compute(t, p, c, pb)
        assert abs(out["energy"][k] - one["energy"]) < tol * len(p)
        assert np.abs(out["forces"][lo:lo + len(p)] - one["forces"]).max() < tol * max(1.0, np.abs(one["forces"]).max())
        lo += len(p)


def test_batched_small_structures(engines):
    """48 cells of the batched benchmark workload (32 .. 128 atoms, bcc / fcc / hcp, strained, 3 species): one engine pass
    over all of them = the structures one by one; per-structure energies are the sums of their atoms' energies"""
    eng = engines("config5", ["Al", "Ni", "Ti"])
    structs = cases.structures_config5(48)
    natoms = [len(x[0]) for x in structs]
    assert min(natoms) >= 32 and max(natoms) <= 128 and len(set(natoms)) > 20
    b = kk.Batch(eng.model, ["Al", "Ni", "Ti"])
    pbc = np.ones((len(structs), 3), bool)
    out = b.compute(natoms, np.concatenate([x[2] for x in structs]), np.concatenate([x[0] for x in structs]),
                    np.stack([x[1] for x in structs]), pbc, energies=True)
    assert b.passes == 1
    one = kk.System(eng.model, ["Al", "Ni", "Ti"], skin=0.0)
    lo = 0
    for k, (p, c, t) in enumerate(structs):
        r = one.compute(t, p, c, [True, True, True], energies=True)
        fs = max(1.0, np.abs(r["forces"]).max())
        assert abs(out["energy"][k] - r["energy"]) < 1e-9 * max(1.0, abs(r["energy"]))
        assert np.abs(out["forces"][lo:lo + len(p)] - r["forces"]).max() < 1e-9 * fs
        assert np.abs(out["virial"][k] - r["virial"]).max() < 1e-9 * max(1.0, np.abs(r["virial"]).max())
        assert abs(out["energies"][lo:lo + len(p)].sum() - out["energy"][k]) < 1e-9 * max(1.0, abs(r["energy"]))
        lo += len(p)
    eo = b.compute(natoms, np.concatenate([x[2] for x in structs]), np.concatenate([x[0] for x in structs]),
                   np.stack([x[1] for x in structs]), pbc, energy_only=True)
    assert np.abs(eo["energy"] - out["energy"]).max() < 1e-9 * np.abs(out["energy"]).max() and "forces" not in eo
    with pytest.raises(ValueError, match="do not describe"):
        b.compute(natoms[:-1], np.concatenate([x[2] for x in structs]), np.concatenate([x[0] for x in structs]),
                  np.stack([x[1] for x in structs]), pbc)
