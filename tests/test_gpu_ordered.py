"""Ordered (atomic-free) sums of the engines (gr_engine_set_ordered_sums): forces, virial, energy and, for GRACE-2L and
3L, the message adjoints added in a fixed order.  The reference's GPU engines have no such mode and document last-bit variation from run to run
(python/tests/test_gpu_several_calculators.py); the tests hold the ordered mode to the atomic mode at the parity bounds of
the other GPU tests (1e-10 eV/atom, 1e-9 eV/A) and to ITSELF bit for bit: repeated calls, a fresh engine, chunked passes."""
import numpy as np
import pytest

import cases
from grace_runtime_amd import kk, workloads
from test_gpu_lammps import lammps_inputs

pytestmark = pytest.mark.gpu

KEYS = ("forces", "virial", "energies")


def _same_bits(a, b):
    assert a["energy"] == b["energy"]
    for k in KEYS:
        if k in a:
            assert np.array_equal(a[k], b[k]), k


def _close(a, b, n, tol):
    fs = max(1.0, np.abs(b["forces"]).max())
    assert abs(a["energy"] - b["energy"]) / n < tol * fs
    assert np.abs(a["forces"] - b["forces"]).max() < 10 * tol * fs
    assert np.abs(a["virial"] - b["virial"]).max() < 100 * tol * fs
    assert np.abs(a["energies"] - b["energies"]).max() < tol * fs


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("model,struct,species", [("mix2", "alloy54", ["Mo", "W"]), ("cut2", "slab", ["Al", "Ni"]), ("config1", "config1", ["W"]),
                                                  ("l2mix", "alloy54", ["Mo", "W"]), ("l2mix", "slab", ["Mo", "W"]), ("config3", "fcc108", ["Al", "Co", "Ni", "Ti"]),
                                                  ("l3mix", "alloy54", ["Mo", "W"]), ("l3wide", "fcc108", ["Al", "Ni"]), ("l3el", "alloy54", ["Mo", "W"])])
def test_ordered_sums_equal_atomic_sums_and_repeat_bit_for_bit(model_dir, model, struct, species, precision):
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    types = np.minimum(types, len(species)).astype(np.int32)
    n = len(pos)
    m = kk.Model(cases.model_file(model_dir, model))
    ref = kk.System(m, species, skin=0.0, chunksize=0, precision=precision).compute(types, pos, cell, pbc, energies=True)
    s = kk.System(m, species, skin=0.0, chunksize=0, precision=precision)
    assert not s.engine.ordered_sums
    s.engine.set_ordered_sums(True)
    assert s.engine.ordered_sums
    out = s.compute(types, pos, cell, pbc, energies=True)
    _close(out, ref, n, 1e-10 if precision == 64 else 2e-6)
    assert np.abs(out["forces"].sum(0)).max() < 1e-9 * max(1.0, np.abs(out["forces"]).max()) * (1 if precision == 64 else 1e4)
    for _ in range(3):                                          # the same call again, other work in between
        s.compute(types, pos + 1e-2, cell, pbc)
        _same_bits(s.compute(types, pos, cell, pbc, energies=True), out)
    fresh = kk.System(m, species, skin=0.0, chunksize=0, precision=precision)
    fresh.engine.set_ordered_sums(True)
    _same_bits(fresh.compute(types, pos, cell, pbc, energies=True), out)
    # GRACE-1L: chunks change neither a bond's force nor the order of the sums.  GRACE-2L / 3L: a neighbour's message adjoint
    # is added chunk by chunk, so a chunked pass equals the one-pass result to rounding, and itself bit for bit
    one_layer = m.layers == 1
    for cs in (7, 16, n - 1):
        c = kk.System(m, species, skin=0.0, chunksize=cs, precision=precision)
        c.engine.set_ordered_sums(True)
        first = c.compute(types, pos, cell, pbc, energies=True)
        if one_layer:
            _same_bits(first, out)
        else:
            _close(first, out, n, 1e-10 if precision == 64 else 2e-6)
            c.compute(types, pos + 1e-2, cell, pbc)
            _same_bits(c.compute(types, pos, cell, pbc, energies=True), first)
    eo = s.compute(types, pos, cell, pbc, energy_only=True)
    assert eo["energy"] == out["energy"]
    s.engine.set_ordered_sums(False)                            # and back: the atomic sums again
    _close(s.compute(types, pos, cell, pbc, energies=True), ref, n, 1e-10 if precision == 64 else 2e-6)


@pytest.mark.parametrize("model", ["mix2", "l2mix", "l3mix"])
def test_ordered_sums_of_a_batch(model_dir, model):
    """several structures in one list: a record per structure, summed over its rows in ascending order"""
    structs = workloads.structures_config5(6)
    natoms, types, pos, cells, pbc = workloads.batch_arrays(structs)
    types = np.minimum(types, 2).astype(np.int32)
    m = kk.Model(cases.model_file(model_dir, model))
    ref = kk.Batch(m, ["Mo", "W"], chunksize=0).compute(natoms, types, pos, cells, pbc, energies=True)
    b = kk.Batch(m, ["Mo", "W"], chunksize=0)
    b.engine.set_ordered_sums(True)
    out = b.compute(natoms, types, pos, cells, pbc, energies=True)
    fs = max(1.0, np.abs(ref["forces"]).max())
    assert np.abs(out["energy"] - ref["energy"]).max() < 1e-9 * fs
    assert np.abs(out["forces"] - ref["forces"]).max() < 1e-9 * fs
    assert np.abs(out["virial"] - ref["virial"]).max() < 1e-8 * fs
    assert np.abs(out["energies"] - ref["energies"]).max() < 1e-9 * fs
    for cs in (0, 50) if model == "mix2" else (0,):
        c = kk.Batch(m, ["Mo", "W"], chunksize=cs)
        c.engine.set_ordered_sums(True)
        again = c.compute(natoms, types, pos, cells, pbc, energies=True)
        for k in ("energy", "forces", "virial", "energies"):
            assert np.array_equal(again[k], out[k]), (cs, k)


@pytest.mark.parametrize("model,struct", [("mix2", "alloy54"), ("l2mix", "triclinic"), ("l3mix", "alloy54")])
def test_ordered_sums_with_ghost_atoms(model_dir, model, struct):
    """the LAMMPS call: the neighbours of a bond are ghost rows, whose forces are folded onto their owners afterwards"""
    eng = kk.Engine(kk.Model(cases.model_file(model_dir, model)), ["Mo", "W"], 64)
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    n = len(pos)
    rc = max(eng.cutoff(a, b) for a in (1, 2) for b in (1, 2))
    x, t, owner, rows = lammps_inputs(pos, cell, types, rc + 0.7)
    args = (n, t, x, np.arange(n), [len(r) for r in rows], rows)
    ref = eng.compute_lammps(*args, owner=owner, energies=True)
    eng.set_ordered_sums(True)
    out = eng.compute_lammps(*args, owner=owner, energies=True)
    fs = max(1.0, np.abs(ref["forces"]).max())
    assert abs(out["energy"] - ref["energy"]) < 1e-10 * max(1.0, abs(ref["energy"]))
    assert np.abs(out["forces"] - ref["forces"]).max() < 1e-9 * fs
    assert np.abs(out["virial"] - ref["virial"]).max() < 1e-9 * max(1.0, np.abs(ref["virial"]).max())
    again = eng.compute_lammps(*args, owner=owner, energies=True)
    assert again["energy"] == out["energy"] and np.array_equal(again["forces"], out["forces"]) and np.array_equal(again["virial"], out["virial"])
    with pytest.raises(ValueError, match="per-atom virials"):
        eng.compute_lammps(*args, owner=owner, vatom=np.zeros((len(x), 6)))


@pytest.mark.parametrize("name", ["config2", "config3", "config4"])
def test_full_size_passes_repeat_bit_for_bit(name, tmp_path):
    """benchmark configurations 2 (GRACE-1L, 8192 atoms), 3 (GRACE-2L, 32000 atoms, 2.5 M bonds) and the model of 4 (GRACE-3L,
    lmax 5, 64 channels) on 2000 atoms: at this size the atomic sums of two engines rarely agree in every bit; the ordered
    sums of two engines do, and agree with the atomic ones"""
    if name == "config2":
        pos, cell, pbc, types = workloads.structure_config2()
        path, species = workloads.write_model("config1", str(tmp_path)), ["W"]
    elif name == "config3":
        pos, cell, pbc, types = workloads.structure_config3()
        path, species = workloads.write_model("config3", str(tmp_path)), ["Al", "Co", "Ni", "Ti"]
    else:
        pos, cell, pbc, t89 = workloads.structure_config4(natoms=2000)
        path = workloads.write_model("config4", str(tmp_path))
        species, types = workloads.config4_species(kk.Model(path).element_names), workloads.config4_types(t89)
    m = kk.Model(path)
    n = len(pos)
    ref = kk.System(m, species, skin=0.0, precision=64).compute(types, pos, cell, pbc, energies=True)
    outs = []
    for _ in range(2):
        s = kk.System(m, species, skin=0.0, precision=64)
        s.engine.set_ordered_sums(True)
        outs.append(s.compute(types, pos, cell, pbc, energies=True))
        outs.append(s.compute(types, pos, cell, pbc, energies=True))
        del s
    for o in outs[1:]:
        _same_bits(o, outs[0])
    _close(outs[0], ref, n, 1e-10)
    assert np.abs(outs[0]["forces"].sum(axis=0)).max() < 1e-8 * max(1.0, np.abs(ref["forces"]).max()) * np.sqrt(n)
