"""Deterministic synthetic test cases (models and structures) shared by the golden-vector generator
(tests/golden/make_golden.py) and the tests.  Everything derives from fixed numpy Generator seeds."""
from __future__ import annotations

import os

import numpy as np

from grace_runtime_amd import synth
from grace_runtime_amd.workloads import (CONFIG4_SPECIES, model_config1, model_config3, model_config4, model_config5,  # noqa: F401
                                         structure_config1, structure_config2, structure_config3, structure_config4,
                                         structures_config5)

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")
REF_FIXTURES = os.path.join(GOLDEN, "ref_fixtures")


def model_mix2():
    """two elements, lmax 3, A width 20 != FC width 40, 10 radial basis functions, with the AAAA stage"""
    return synth.random_model_1l(lmax=3, n_elements=2, element_names=("Mo", "W"), embedding_size=16, nradbase=10,
                                 nradmax=20, fc_width=40, hidden=64, rho_n_out=9, energy_hidden=32, rcut=5.0,
                                 inv_avg_n_neigh=1.0 / 26.0, seed=7)


def model_cut2():
    """two elements with pair-specific cutoffs, lmax 2, max_order 3"""
    d = synth.random_model_1l(lmax=2, n_elements=2, element_names=("Al", "Ni"), embedding_size=8, nradbase=8,
                              nradmax=16, hidden=32, rho_n_out=5, energy_hidden=16, rcut=5.5, order4=False,
                              inv_avg_n_neigh=1.0 / 30.0, seed=11)
    d["has_bond_specific_cutoff"] = np.array([1], dtype=np.int64)
    d["bond_cutoff_map"] = np.array([[5.5, 4.75], [4.75, 4.0]])
    return d


def model_ch20():
    """two elements, lmax 3, 20 channels in every stage (padded to 32 on the device: the widths the fused dense chain
    covers), with the AAAA stage"""
    return synth.random_model_1l(lmax=3, n_elements=2, element_names=("Mo", "W"), embedding_size=12, nradbase=8,
                                 nradmax=20, hidden=32, rho_n_out=9, energy_hidden=16, rcut=5.0,
                                 inv_avg_n_neigh=1.0 / 26.0, seed=31)


def model_ch3():
    """two elements, lmax 2, 32 channels, max_order 3 (no AA2 / AAAA stage)"""
    return synth.random_model_1l(lmax=2, n_elements=2, element_names=("Mo", "W"), embedding_size=8, nradbase=8,
                                 nradmax=32, hidden=32, rho_n_out=7, energy_hidden=16, rcut=5.0, order4=False,
                                 inv_avg_n_neigh=1.0 / 26.0, seed=32)


def model_chleg():
    """two elements, lmax 2, 24 channels, the legacy product AAA = AA1 x A (right operand A instead of A1)"""
    d = synth.random_model_1l(lmax=2, n_elements=2, element_names=("Mo", "W"), embedding_size=8, nradbase=8,
                              nradmax=24, hidden=32, rho_n_out=7, energy_hidden=16, rcut=5.0,
                              inv_avg_n_neigh=1.0 / 26.0, seed=33)
    d["AAA_right_A"] = np.array([1], dtype=np.int64)
    return d


def model_l2mix():
    """GRACE-2L, two elements with pair-specific cutoffs, lmax 2, different (unpadded) widths in every stage"""
    d = synth.random_model_2l(lmax=2, n_elements=2, element_names=("Mo", "W"), embedding_size=8, nradbase=10, c1=20, cr=12,
                              c2=24, i1_width=10, hidden=32, rho_n_out=9, energy_hidden=16, rcut=5.0,
                              inv_avg_n_neigh=1.0 / 26.0, seed=13)
    d["has_bond_specific_cutoff"] = np.array([1], dtype=np.int64)
    d["bond_cutoff_map"] = np.array([[5.0, 4.5], [4.5, 4.25]])
    return d


def model_l3mix():
    """GRACE-3L, two elements with pair-specific cutoffs, lmax 2, messages with both parities"""
    d = synth.random_model_3l(lmax=2, n_elements=2, element_names=("Mo", "W"), embedding_size=8, nradbase=10, channels=16,
                              hidden=32, rho_n_out=9, energy_hidden=16, rcut=5.0, inv_avg_n_neigh=1.0 / 26.0, seed=21)
    d["has_bond_specific_cutoff"] = np.array([1], dtype=np.int64)
    d["bond_cutoff_map"] = np.array([[5.0, 4.5], [4.5, 4.25]])
    return d


def model_l3wide():
    """GRACE-3L, four elements, lmax 3 with messages up to l = 2, a hidden width that needs padding (48 -> 64), full
    RMSNorm of the densities, tanh readout"""
    d = synth.random_model_3l(lmax=3, lmsg=2, n_elements=4, element_names=("Al", "Co", "Ni", "Ti"), embedding_size=6, nradbase=8,
                              channels=32, hidden=48, rho_n_out=12, energy_hidden=24, rcut=5.5, p=6,
                              inv_avg_n_neigh=1.0 / 30.0, rms_type=0, seed=22)
    d["energy_mlp_activation"] = np.array([1], dtype=np.int64)
    return d


def model_l3pad():
    """GRACE-3L with 20 channels (padded to 32 on the GPU; the reference's CPU engine wants multiples of 16, so this
    model is checked against the oracle only)"""
    return synth.random_model_3l(lmax=2, lmsg=1, n_elements=2, element_names=("Mo", "W"), embedding_size=5, nradbase=6,
                                 channels=20, hidden=24, rho_n_out=7, energy_hidden=12, rcut=5.0, inv_avg_n_neigh=1.0 / 26.0,
                                 seed=24)


def model_l3el():
    """GRACE-3L whose eq reduces and SPBF reduces carry one weight set per element of the central atom"""
    return synth.random_model_3l(lmax=2, lmsg=1, elem_dep=True, n_elements=2, element_names=("Mo", "W"), embedding_size=6,
                                 nradbase=8, channels=16, hidden=32, rho_n_out=8, energy_hidden=16, rcut=5.0,
                                 inv_avg_n_neigh=1.0 / 26.0, seed=25)


def model_l3nat():
    """GRACE-3L with natural-parity messages only, one element, lmax 2"""
    return synth.random_model_3l(lmax=2, pseudo_message=False, n_elements=1, element_names=("W",), embedding_size=4, nradbase=8,
                                 channels=16, hidden=16, rho_n_out=8, energy_hidden=16, rcut=5.0, inv_avg_n_neigh=1.0 / 26.0,
                                 seed=23)


def model_uq2():
    """model_mix2 with a uqv6 UQ head whose GMM centroids sit next to the features of atoms of the alloy54 structure (three
    clusters for Mo, two for W), so that the atoms of a test structure fall into different clusters; the last W centroid
    IS the feature vector of an atom (sigma^2 = 1e-8 exactly there)"""
    from grace_runtime_amd import kk
    from oracle import grace_oracle as go
    d = model_mix2()
    synth.add_uq_head_1l(d, rp_dim=12, max_clusters=3, seed=31)
    pos, cell, pbc, types = structure_alloy54()
    perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, 5.0)
    x, t = pos[perm], types[perm]
    rij = x[j] - np.repeat(x, np.diff(offset), axis=0) + shifts[image]
    f = go.compute_1l(go.Model1L(d), t - 1, offset, j, rij, want_forces=False, uq=True)["uq_features"]
    cen = d["uq_centroids"]
    ncl = np.array([3, 2], np.int32)
    for e in range(2):
        at = np.nonzero(t - 1 == e)[0]
        for k in range(ncl[e]):
            cen[e, k] = f[at[(k * (len(at) - 1)) // max(ncl[e] - 1, 1)]] + (0.0 if (e, k) == (1, 1) else 0.003 * (k + 1))
    d["uq_centroids"], d["uq_n_clusters"] = cen, ncl
    return d


def model_uq2l():
    """the reference's fixture model grace_2l_small (max_order 4: the UQ head refuses max_order 3) with a generated uqv6 head
    of two basis blocks whose centroids sit next to features of atoms of the alloy54 structure, one exactly on an atom"""
    from grace_runtime_amd import kk
    from oracle import grace_oracle_2l as go2
    with np.load(os.path.join(REF_FIXTURES, "grace_2l_small.npz")) as z:
        d = {k: z[k] for k in z.files}
    synth.add_uq_head_2l(d, rp_dim=10, max_clusters=3, seed=47)
    pos, cell, pbc, types = structure_alloy54()
    perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, 5.0)
    x, t = pos[perm], types[perm]
    rij = x[j] - np.repeat(x, np.diff(offset), axis=0) + shifts[image]
    f = go2.compute_2l(go2.Model2L(d), t - 1, offset, j, rij, want_forces=False, uq=True)["uq_features"]
    cen = d["uq_centroids"]
    ncl = np.array([2, 3], np.int32)
    for e in range(2):
        at = np.nonzero(t - 1 == e)[0]
        for k in range(ncl[e]):
            cen[e, k] = f[at[(k * (len(at) - 1)) // max(ncl[e] - 1, 1)]] + (0.0 if (e, k) == (0, 1) else 0.002 * (k + 1))
    d["uq_centroids"], d["uq_n_clusters"] = cen, ncl
    return d


def model_uq3l():
    """model_l3mix with a generated uqv6 head of three basis blocks (the inputs of rho1, rho2, rho3) and four density
    channels, centroids next to features of atoms of the alloy54 structure, one exactly on an atom"""
    from grace_runtime_amd import kk
    from oracle import grace_oracle_3l as go3
    d = model_l3mix()
    synth.add_uq_head_3l(d, rp_dim=9, max_clusters=3, seed=53)
    pos, cell, pbc, types = structure_alloy54()
    perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, 5.0)
    x, t = pos[perm], types[perm]
    rij = x[j] - np.repeat(x, np.diff(offset), axis=0) + shifts[image]
    f = go3.compute_3l(go3.Model3L(d), t - 1, offset, j, rij, want_forces=False, uq=True)["uq_features"]
    cen = d["uq_centroids"]
    ncl = np.array([3, 3], np.int32)
    for e in range(2):
        at = np.nonzero(t - 1 == e)[0]
        for k in range(ncl[e]):
            cen[e, k] = f[at[(k * (len(at) - 1)) // max(ncl[e] - 1, 1)]] + (0.0 if (e, k) == (1, 2) else 0.002 * (k + 1))
    d["uq_centroids"], d["uq_n_clusters"] = cen, ncl
    return d


MODELS = {"ch20": model_ch20, "ch3": model_ch3, "chleg": model_chleg, "uq3l": model_uq3l, "uq2l": model_uq2l, "uq2": model_uq2, "l3mix": model_l3mix, "l3wide": model_l3wide, "l3pad": model_l3pad, "l3el": model_l3el, "l3nat": model_l3nat, "config4": model_config4, "config5": model_config5, "config1": model_config1, "mix2": model_mix2, "cut2": model_cut2, "config3": model_config3, "l2mix": model_l2mix}
LAYERS = {"ch20": 1, "ch3": 1, "chleg": 1, "uq3l": 3, "uq2l": 2, "uq2": 1, "l3mix": 3, "l3wide": 3, "l3pad": 3, "l3el": 3, "l3nat": 3, "config4": 3, "config5": 2, "config1": 1, "mix2": 1, "cut2": 1, "config3": 2, "l2mix": 2}


def write_model(name, directory):
    """the model's kokkos.npz in `directory`, written on first use (atomically: workers of a parallel run share the directory)"""
    path = os.path.join(directory, f"{name}.npz")
    if not os.path.exists(path):
        tmp = os.path.join(directory, f".{name}.{os.getpid()}.npz")
        synth.save_model(tmp, MODELS[name]())
        os.replace(tmp, path)
    return path


model_file = lambda directory, name: write_model(name, directory)    # noqa: E731  (argument order of os.path.join)


def structure_alloy54(seed=3):
    pos, cell = synth.bcc_supercell(3.0, 3)
    rng = np.random.default_rng(seed)
    types = rng.integers(1, 3, size=len(pos)).astype(np.int32)
    return synth.jitter(pos, 0.1, seed + 100), cell, np.array([True, True, True]), types


def structure_triclinic(seed=5):
    rng = np.random.default_rng(seed)
    cell = np.array([[5.5, 0.0, 0.0], [-0.9, 5.2, 0.0], [1.1, -1.3, 6.1]])
    frac = rng.uniform(-0.5, 1.5, (24, 3))        # also outside the cell: images of the atoms themselves
    types = rng.integers(1, 3, size=24).astype(np.int32)
    return frac @ cell, cell, np.array([True, True, True]), types


def structure_slab(seed=6):
    rng = np.random.default_rng(seed)
    cell = np.diag([9.0, 8.0, 25.0])
    pos = rng.uniform(0, 1, (40, 3)) * np.array([9.0, 8.0, 7.0])
    types = rng.integers(1, 3, size=40).astype(np.int32)
    return pos, cell, np.array([True, True, False]), types


def structure_molecule(seed=8):
    rng = np.random.default_rng(seed)
    pos = rng.uniform(0, 6, (17, 3))
    types = rng.integers(1, 3, size=17).astype(np.int32)
    return pos, np.zeros((3, 3)), np.array([False, False, False]), types


def structure_fcc108(seed=3):
    """3 x 3 x 3 cells of the fcc alloy of the two-layer benchmark (4 species; the box is shorter than two cutoffs)"""
    pos, cell = synth.fcc_supercell(3.6, 3)
    rng = np.random.default_rng(seed)
    types = rng.integers(1, 5, size=len(pos)).astype(np.int32)
    return synth.jitter(pos, 0.08, seed), cell, np.array([True, True, True]), types


STRUCTURES = {"fcc108": structure_fcc108, "config1": structure_config1, "alloy54": structure_alloy54, "triclinic": structure_triclinic,
              "slab": structure_slab, "molecule": structure_molecule}

# (model, structure, list cutoff or None for the model cutoff): the end-to-end golden cases
E2E_CASES = [("config1", "config1", None), ("mix2", "alloy54", 5.5), ("mix2", "triclinic", None),
             ("cut2", "alloy54", None), ("cut2", "slab", 6.0), ("mix2", "molecule", None)]
E2E_CASES_2L = [("config3", "fcc108", None), ("l2mix", "alloy54", 5.5), ("l2mix", "triclinic", None), ("l2mix", "slab", None),
                ("l2mix", "molecule", None)]
# reference fixture models (tests/golden/ref_fixtures) on the reference's fixture cells: goldens of the compiled reference
E2E_CASES_3L = [("l3mix", "alloy54", 5.5), ("l3mix", "triclinic", None), ("l3mix", "slab", None), ("l3mix", "molecule", None),
                ("l3wide", "fcc108", None), ("l3nat", "config1", None), ("l3el", "alloy54", None)]
# cases with per-atom virials of the compiled reference among the goldens
VATOM_CASES = [("mix2", "alloy54", 5.5), ("cut2", "slab", 6.0), ("l2mix", "triclinic", None), ("l2mix", "slab", None), ("l3mix", "alloy54", 5.5),
               ("l3el", "alloy54", None)]
UQ_CASES = [("uq2", "alloy54"), ("uq2", "triclinic"), ("uq2l", "alloy54"), ("uq2l", "triclinic"), ("uq3l", "alloy54"), ("uq3l", "triclinic")]
FIXTURE_CASES_2L = [(m, c) for m in ("grace_2l_small", "grace_2l_l3", "legacy_2l_small", "legacy_2l_wide") for c in ("W54", "WMo54")]


def bond_vectors(pos, perm, offset, j, image, shifts):
    x = pos[perm]
    return x[j] - np.repeat(x, np.diff(offset), axis=0) + (shifts[image] if len(shifts) else 0.0)


def oracle_reference(model_dir, model, pos, cell, pbc, types):
    """Energy, forces, virial, per-atom energies and per-atom virials of the CPU oracle for a structure on its own
    neighbour list (searched at the model's largest cutoff), in the caller's atom order.  `types` are 1-based indices
    into the model's element list.  The independent second source the call-level GPU tests compare with (the reference
    checks its LAMMPS bond source against its CSR source in the same way, tests/test_bonds.cpp:2-91)."""
    from grace_runtime_amd import kk
    from oracle import grace_oracle as g1
    from oracle import grace_oracle_2l as g2
    from oracle import grace_oracle_3l as g3
    make, compute = {1: (g1.Model1L, g1.compute_1l), 2: (g2.Model2L, g2.compute_2l), 3: (g3.Model3L, g3.compute_3l)}[LAYERS[model]]
    om = make(model_file(model_dir, model))
    rc = float(np.max(om.cut))
    pcell, shift = kk._padded_cell_arrays(cell, pos, rc, pbc)
    perm, offset, j, image, shifts = kk.neighbor_search(pos + shift, pcell, pbc, rc)
    out = compute(om, np.asarray(types)[perm] - 1, offset, j, bond_vectors(pos, perm, offset, j, image, shifts))
    res = {"energy": float(out["energy"]), "virial": np.asarray(out["virial"])}
    for key in ("forces", "energies", "virials"):
        if key in out:
            a = np.empty_like(out[key])
            a[perm] = out[key]
            res[key] = a
    return res


def golden_reference(gold, model, struct):
    """The committed outputs of the compiled reference for an e2e case, in the caller's atom order (the goldens are stored in
    the order of the reference's neighbour list)."""
    tag = f"e2e/{model}/{struct}"
    perm = gold[f"nl/{struct}@{float(gold[tag + '/rc_list']):g}/perm"]
    res = {"energy": float(gold[tag + "/energy"]), "virial": gold[tag + "/virial"]}
    for key in ("forces", "energies", "virials"):
        if f"{tag}/{key}" in gold:
            a = np.empty_like(gold[f"{tag}/{key}"])
            a[perm] = gold[f"{tag}/{key}"]
            res[key] = a
    return res


def check_against(out, ref, n, tol_e, tol_f, tol_ea, tol_v):
    """out (energy, forces [n..], virial, energies) against ref to the given bounds, forces and per-atom energies scaled by
    the largest reference force where that exceeds 1 eV/A"""
    fs = max(1.0, np.abs(ref["forces"]).max())
    assert abs(out["energy"] - ref["energy"]) / n < tol_e * fs
    assert np.abs(np.asarray(out["forces"])[:n] - ref["forces"]).max() < tol_f * fs
    assert np.abs(out["virial"] - ref["virial"]).max() < tol_v * max(1.0, np.abs(ref["virial"]).max())
    if "energies" in out and "energies" in ref:
        assert np.abs(np.asarray(out["energies"])[:n] - ref["energies"]).max() < tol_ea * fs
