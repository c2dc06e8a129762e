"""The synthetic benchmark workloads: the random-weight models and the structures of the five benchmark configurations,
generated from fixed numpy Generator seeds.  Used by bench.py, by the smoke check and by the tests."""
from __future__ import annotations

import os

import numpy as np

from . import synth


def model_config1():
    """GRACE-1L-shaped benchmark model: lmax 4, 32 channels, 8 Chebyshev functions, MLP 8-64-64-160, 1 species."""
    return synth.random_model_1l(seed=20260101)


def model_config3():
    """GRACE-2L-shaped benchmark model: two layers, lmax 4, 32 channels everywhere, radial MLPs 8-64-64-160, body
    order 3 per layer, 4 species"""
    return synth.random_model_2l(seed=20260103)


def model_config5():
    """the GRACE-2L-shaped benchmark model with 3 species (batched small-structure workload)"""
    return synth.random_model_2l(n_elements=3, element_names=("Al", "Ni", "Ti"), inv_avg_n_neigh=1.0 / 60.0, seed=20260105)


def model_config4():
    """GRACE-3L-shaped benchmark model: three layers, lmax 5, 64 radial channels, radial MLPs (8 + 2 x 32)-128-128-384,
    an embedding table of 89 species"""
    return synth.random_model_3l(lmax=5, n_elements=89, embedding_size=32, nradbase=8, channels=64, hidden=128, rho_n_out=32,
                                 energy_hidden=64, rcut=6.0, inv_avg_n_neigh=1.0 / 72.0, seed=20260104)


def structure_config1():
    pos, cell = synth.bcc_supercell(3.165, 4)
    return synth.jitter(pos, 0.05, 1), cell, np.array([True, True, True]), np.ones(128, np.int32)


def structure_config2():
    pos, cell = synth.bcc_supercell(3.165, 16)
    return synth.jitter(pos, 0.05, 2), cell, np.array([True, True, True]), np.ones(8192, np.int32)


def structure_config3():
    pos, cell = synth.fcc_supercell(3.6, 20)
    rng = np.random.default_rng(3)
    types = rng.integers(1, 5, size=len(pos)).astype(np.int32)
    return synth.jitter(pos, 0.08, 3), cell, np.array([True, True, True]), types


CONFIG4_SPECIES = (6, 8, 13, 14, 22, 26, 28, 74)    # 1-based types = model element + 1: C O Al Si Ti Fe Ni W


def structure_config4(natoms=10000, density=0.08, dmin=1.8, seed=4):
    """Amorphous periodic cube: random sequential packing of `natoms` atoms at `density` atoms / A^3 with a minimum
    distance `dmin`; 8 species of the 89-element table drawn uniformly."""
    rng = np.random.default_rng(seed)
    side = (natoms / density) ** (1.0 / 3.0)
    nc = max(1, int(side / dmin))
    w = side / nc
    grid = {}
    pos = np.zeros((natoms, 3))
    k = 0
    while k < natoms:
        cand = rng.uniform(0.0, side, (4 * (natoms - k) + 64, 3))
        for x in cand:
            c = tuple((x / w).astype(int) % nc)
            ok = True
            for dx in (-1, 0, 1):
                for dy in (-1, 0, 1):
                    for dz in (-1, 0, 1):
                        for q in grid.get(((c[0] + dx) % nc, (c[1] + dy) % nc, (c[2] + dz) % nc), ()):
                            d = x - pos[q]
                            d -= side * np.round(d / side)
                            if d @ d < dmin * dmin:
                                ok = False
                                break
                        if not ok:
                            break
                    if not ok:
                        break
                if not ok:
                    break
            if ok:
                pos[k] = x
                grid.setdefault(c, []).append(k)
                k += 1
                if k == natoms:
                    break
    types = np.array(CONFIG4_SPECIES, dtype=np.int32)[rng.integers(0, 8, natoms)]
    return pos, np.eye(3) * side, np.array([True, True, True]), types


def structures_config5(nstruct=512, seed=5):
    """Independent periodic cells of 32 .. 128 atoms: random bcc / fcc / hcp lattice with lattice constant U(2.8, 4.0) A,
    cell strain U(-3 %, 3 %), N(0, 0.1 A) jitter, 3 species drawn uniformly; atoms removed at random from the smallest
    supercell that holds the drawn size.  Returns lists (positions, cell, types) and pbc = True."""
    rng = np.random.default_rng(seed)
    s3 = np.sqrt(3.0)
    lattices = {
        "bcc": (np.eye(3), np.array([[0, 0, 0], [0.5, 0.5, 0.5]])),
        "fcc": (np.eye(3), np.array([[0, 0, 0], [0.5, 0.5, 0], [0.5, 0, 0.5], [0, 0.5, 0.5]])),
        "hcp": (np.diag([1.0, s3, np.sqrt(8.0 / 3.0)]), np.array([[0, 0, 0], [0.5, 0.5, 0], [0.5, 5.0 / 6.0, 0.5], [0, 1.0 / 3.0, 0.5]])),
    }
    out = []
    for _ in range(nstruct):
        n = int(rng.integers(32, 129))
        unit, basis = lattices[["bcc", "fcc", "hcp"][int(rng.integers(0, 3))]]
        a = rng.uniform(2.8, 4.0)
        reps = [1, 1, 1]
        while reps[0] * reps[1] * reps[2] * len(basis) < n:
            reps[int(np.argmin([reps[k] * unit[k, k] for k in range(3)]))] += 1
        g = np.stack(np.meshgrid(*[np.arange(r) for r in reps], indexing="ij"), -1).reshape(-1, 1, 3)
        frac = (g + basis[None]).reshape(-1, 3)
        keep = np.sort(rng.permutation(len(frac))[:n])
        cell = np.diag([reps[k] * unit[k, k] * a for k in range(3)])
        pos = frac[keep] * np.array([unit[k, k] * a for k in range(3)])
        eps = rng.uniform(-0.03, 0.03, (3, 3))
        F = np.eye(3) + 0.5 * (eps + eps.T)
        pos = pos @ F.T + rng.normal(0.0, 0.1, (n, 3))
        out.append((pos, cell @ F.T, rng.integers(1, 4, n).astype(np.int32)))
    return out


def model_small_3l():
    """a small GRACE-3L-shaped model (two elements, lmax 2, 16 channels, messages of both parities) for quick checks"""
    return synth.random_model_3l(lmax=2, n_elements=2, element_names=("Mo", "W"), embedding_size=8, nradbase=10, channels=16,
                                 hidden=32, rho_n_out=9, energy_hidden=16, rcut=5.0, inv_avg_n_neigh=1.0 / 26.0, seed=21)


BENCHMARK_MODELS = {"small_3l": model_small_3l, "config1": model_config1, "config3": model_config3, "config4": model_config4, "config5": model_config5}


def write_model(name, directory):
    """kokkos.npz file of a benchmark model in `directory` (written once); config 2 uses the model of config 1."""
    name = "config1" if name == "config2" else name
    path = os.path.join(directory, f"{name}.npz")
    if not os.path.exists(path):
        synth.save_model(path, BENCHMARK_MODELS[name]())
    return path


def config4_types(t89):
    """engine atom types 1 .. 8 of config 4's atoms (the 8 species present, in ascending element order, as a LAMMPS
    pair_coeff line would map them) from their 1-based indices into the 89-element table"""
    return (np.searchsorted(np.array(CONFIG4_SPECIES), t89) + 1).astype(np.int32)


def config4_species(element_names):
    return [element_names[t - 1] for t in CONFIG4_SPECIES]


def batch_arrays(structs):
    """(natoms, types, positions, cells, pbc) of a list of (positions, cell, types) for the batch entry points"""
    natoms = np.array([len(s[0]) for s in structs], np.int32)
    types = np.concatenate([s[2] for s in structs]).astype(np.int32)
    pos = np.concatenate([s[0] for s in structs])
    cells = np.stack([s[1] for s in structs])
    pbc = np.ones((len(structs), 3), dtype=bool)
    return natoms, types, pos, cells, pbc
