"""Radial tables on the GPU (gr_engine_set_spline; `spline` of System / Batch): the engines take the radial functions of a
bond from cubic tables as the reference's engines do (FusedSettings::spline_n = 1024, libgrace/include/grace/system.h:78;
tables libgrace/src/fused_1l.cpp:102-129, evaluation libgrace/include/grace/fused_cpu.h:1052-1074; GRACE-3L: one table per
ordered pair of species and layer, libgrace/src/fused_3l.cpp:491-533).
Parity: against the oracle evaluating the same tables in fp64 (tests/test_spline.py pins it) at the bounds of the other GPU
tests, 1e-10 eV/atom and 1e-9 eV/A in fp64; against the pass without tables at the reference's gate."""
import numpy as np
import pytest

import cases
from grace_runtime_amd import kk, workloads
from oracle import grace_oracle as g1
from oracle import grace_oracle_2l as g2
from oracle import grace_oracle_3l as g3

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("intervals", [1024, 100])
@pytest.mark.parametrize("model,struct,species", [("mix2", "alloy54", ["Mo", "W"]), ("cut2", "slab", ["Al", "Ni"]), ("l2mix", "alloy54", ["Mo", "W"]),
                                                  ("config3", "fcc108", ["Al", "Co", "Ni", "Ti"]), ("l3mix", "alloy54", ["Mo", "W"]),
                                                  ("l3el", "alloy54", ["Mo", "W"])])
def test_tables_equal_the_oracle_with_the_same_tables(model_dir, model, struct, species, intervals, precision):
    layers = cases.LAYERS[model]
    path = cases.model_file(model_dir, model)
    om = {1: g1.Model1L, 2: g2.Model2L, 3: g3.Model3L}[layers](path)
    compute = {1: g1.compute_1l, 2: g2.compute_2l, 3: g3.compute_3l}[layers]
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    types = np.minimum(types, len(species)).astype(np.int32)
    n = len(pos)
    s = kk.System(kk.Model(path), species, skin=0.0, spline=intervals, chunksize=0, precision=precision)
    assert s.engine.spline == intervals
    out = s.compute(types, pos, cell, pbc, energies=True)
    perm, offset, j, image, shifts = s.neighbor_list()
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    om.spline = intervals
    want = compute(om, types[perm] - 1, offset, j, rij)
    om.spline = 0
    exact = compute(om, types[perm] - 1, offset, j, rij)
    fs = max(1.0, np.abs(want["forces"]).max())
    tol = 1e-10 if precision == 64 else 2e-6
    assert abs(out["energy"] - want["energy"]) / n < tol * fs
    assert np.abs(out["forces"][perm] - want["forces"]).max() < 10 * tol * fs
    assert np.abs(out["energies"][perm] - want["energies"]).max() < tol * fs
    assert np.abs(out["virial"] - want["virial"]).max() < 100 * tol * fs
    if intervals == 1024 and precision == 64:
        # the tables change something, and stay inside the reference's gate (1e-6 eV/atom, 1e-5 eV/A)
        assert 1e-12 < abs(out["energy"] - exact["energy"]) / n < 1e-6
        assert np.abs(out["forces"][perm] - exact["forces"]).max() < 1e-5
    # chunks, and the switch back
    c = kk.System(kk.Model(path), species, skin=0.0, spline=intervals, chunksize=13, precision=precision).compute(types, pos, cell, pbc)
    assert np.abs(c["forces"] - out["forces"]).max() < 10 * tol * fs
    s.engine.set_spline(0)
    back = s.compute(types, pos, cell, pbc)
    assert abs(back["energy"] - exact["energy"]) / n < tol * fs
    s.engine.set_spline(intervals)
    s.release_buffers()                                          # the tables are work memory: built again on the next pass
    again = s.compute(types, pos, cell, pbc)
    assert abs(again["energy"] - out["energy"]) / n < tol * fs


def test_arguments(model_dir):
    eng = kk.Engine(kk.Model(cases.model_file(model_dir, "mix2")), ["Mo", "W"], 64)
    assert eng.spline == 0
    for bad in (-1, 7, 1 << 21):
        with pytest.raises(ValueError, match="spline"):
            eng.set_spline(bad)
    assert eng.spline == 0
    assert kk.Model(cases.model_file(model_dir, "mix2")).spline == 1024          # what the reference's calculator passes on


def test_three_layer_tables_above_the_memory_limit_keep_the_mlp(model_dir, monkeypatch):
    """GRACE-3L: tables of the three layers that together exceed the limit are not built (the reference's spline_mb,
    libgrace/src/fused_3l.cpp:405-418): one message, and the results of the pass without tables"""
    pos, cell, pbc, types = cases.structure_alloy54()
    m3 = kk.Model(cases.model_file(model_dir, "l3mix"))
    ref = kk.System(m3, ["Mo", "W"], skin=0.0).compute(types, pos, cell, pbc)
    tab = kk.System(m3, ["Mo", "W"], skin=0.0, spline=1024).compute(types, pos, cell, pbc)
    assert abs(tab["energy"] - ref["energy"]) / len(pos) > 1e-12
    monkeypatch.setenv("GRACE_HIP_TABLE_MB", "0.5")
    msgs = []
    kk.set_logger(lambda level, text: msgs.append(text))
    try:
        out = kk.System(m3, ["Mo", "W"], skin=0.0, spline=1024).compute(types, pos, cell, pbc)
    finally:
        kk.set_logger(None)
    assert sum("radial MLPs are evaluated for every bond" in t for t in msgs) == 1
    assert abs(out["energy"] - ref["energy"]) / len(pos) < 1e-14               # sums by atomic adds: not bit for bit
    assert np.abs(out["forces"] - ref["forces"]).max() < 1e-13 * max(1.0, np.abs(ref["forces"]).max())


@pytest.mark.parametrize("name", ["config2", "config3", "config4"])
def test_full_size_with_tables(name, tmp_path):
    """benchmark configurations 2, 3 and 4 with tables of 1024 intervals against the passes without: inside the gate"""
    if name == "config2":
        pos, cell, pbc, types = workloads.structure_config2()
        path, species = workloads.write_model("config1", str(tmp_path)), ["W"]
    elif name == "config4":                                       # 8 of the model's 89 elements: 64 tables a layer, 0.8 GB
        pos, cell, pbc, t89 = workloads.structure_config4()
        path = workloads.write_model("config4", str(tmp_path))
        species = workloads.config4_species(kk.Model(path).element_names)
        types = workloads.config4_types(t89)
    else:
        pos, cell, pbc, types = workloads.structure_config3()
        path, species = workloads.write_model("config3", str(tmp_path)), ["Al", "Co", "Ni", "Ti"]
    m = kk.Model(path)
    n = len(pos)
    exact = kk.System(m, species, skin=0.0).compute(types, pos, cell, pbc)
    tab = kk.System(m, species, skin=0.0, spline=1024).compute(types, pos, cell, pbc)
    assert 0 < abs(tab["energy"] - exact["energy"]) / n < 1e-6
    assert np.abs(tab["forces"] - exact["forces"]).max() < 1e-5 * max(1.0, np.abs(exact["forces"]).max())
    vol = abs(np.linalg.det(cell))
    assert np.abs(tab["virial"] - exact["virial"]).max() / vol < 1e-6
    assert np.abs(tab["forces"].sum(axis=0)).max() < 1e-8 * max(1.0, np.abs(exact["forces"]).max()) * np.sqrt(n)
