"""Atom chunking of an engine pass (System(chunksize=...), python/kk/kk_api.h:72-75,86): a structure evaluated in chunks of
atoms equals the one-pass result for GRACE-1L, 2L and 3L; the automatic choice follows the memory the library may use; an
allocation failure halves the chunk."""
import os

import numpy as np
import pytest

import cases
from grace_runtime_amd import _lib, kk, workloads

pytestmark = pytest.mark.gpu


def _same(a, b, n, tol=1e-10):
    fs = max(1.0, np.abs(b["forces"]).max())
    assert abs(a["energy"] - b["energy"]) / n < tol * fs
    assert np.abs(a["forces"] - b["forces"]).max() < 10 * tol * fs
    assert np.abs(a["virial"] - b["virial"]).max() < 100 * tol * fs
    if "energies" in b:
        assert np.abs(a["energies"] - b["energies"]).max() < tol * fs


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("model,struct,species", [("mix2", "alloy54", ["Mo", "W"]), ("cut2", "slab", ["Al", "Ni"]), ("config1", "config1", ["W"]),
                                                  ("l2mix", "alloy54", ["Mo", "W"]), ("l2mix", "slab", ["Mo", "W"]), ("config3", "fcc108", ["Al", "Co", "Ni", "Ti"]),
                                                  ("l3mix", "alloy54", ["Mo", "W"]), ("l3wide", "fcc108", ["Al", "Ni"]), ("l3el", "alloy54", ["Mo", "W"])])
def test_chunked_pass_equals_one_pass(model_dir, model, struct, species, precision):
    """chunk sizes that split the tiles of 16 atoms of one element, a chunk of one atom, a chunk larger than the structure"""
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    types = np.minimum(types, len(species)).astype(np.int32)
    n = len(pos)
    m = kk.Model(cases.model_file(model_dir, model))
    one = kk.System(m, species, skin=0.0, chunksize=0, precision=precision)
    ref = one.compute(types, pos, cell, pbc, energies=True)
    assert one.chunksize == 0
    tol = 1e-10 if precision == 64 else 2e-6
    for cs in (7, 16, 21, 1, n - 1, n, 5 * n):
        s = kk.System(m, species, skin=0.0, chunksize=cs, precision=precision)
        out = s.compute(types, pos, cell, pbc, energies=True)
        assert s.chunksize == (cs if cs < n else 0)
        _same(out, ref, n, tol)
        again = s.compute(types, pos + 1e-3, cell, pbc, energies=True)          # a second call reuses the chunk layout
        _same(again, one.compute(types, pos + 1e-3, cell, pbc, energies=True), n, tol)
        del s


@pytest.mark.parametrize("model", ["uq2", "uq2l", "uq3l"])
def test_chunked_uq_and_energy_only(model_dir, model):
    pos, cell, pbc, types = cases.structure_alloy54()
    m = kk.Model(cases.model_file(model_dir, model))
    ref = kk.System(m, ["Mo", "W"], skin=0.0, chunksize=0).compute(types, pos, cell, pbc, uq=True, energies=True)
    s = kk.System(m, ["Mo", "W"], skin=0.0, chunksize=13)
    out = s.compute(types, pos, cell, pbc, uq=True, energies=True)
    _same(out, ref, len(pos))
    for k in ("gamma", "atomic_sigma"):
        assert np.abs(out[k] / ref[k] - 1).max() < 1e-9
    assert np.array_equal(out["gmm_cluster"], ref["gmm_cluster"])
    eo = s.compute(types, pos, cell, pbc, energy_only=True)
    assert abs(eo["energy"] - ref["energy"]) < 1e-9


@pytest.mark.parametrize("model", ["mix2", "l2mix", "l3mix"])
def test_chunked_batch_equals_one_pass(model_dir, model):
    """several structures in one list, chunks that cut through structures"""
    structs = workloads.structures_config5(6)
    natoms, types, pos, cells, pbc = workloads.batch_arrays(structs)
    types = np.minimum(types, 2).astype(np.int32)
    m = kk.Model(cases.model_file(model_dir, model))
    ref = kk.Batch(m, ["Mo", "W"], chunksize=0).compute(natoms, types, pos, cells, pbc, energies=True)
    b = kk.Batch(m, ["Mo", "W"], chunksize=50)
    out = b.compute(natoms, types, pos, cells, pbc, energies=True)
    fs = max(1.0, np.abs(ref["forces"]).max())
    assert np.abs(out["energy"] - ref["energy"]).max() < 1e-9 * fs
    assert np.abs(out["forces"] - ref["forces"]).max() < 1e-9 * fs
    assert np.abs(out["virial"] - ref["virial"]).max() < 1e-8 * fs
    assert np.abs(out["energies"] - ref["energies"]).max() < 1e-9 * fs


def test_automatic_chunk_follows_the_memory_the_library_may_use(tmp_path):
    """configuration 2 (8192 atoms) under a cap on the library's device memory: the automatic choice splits the structure,
    the result is the one-pass result; a cap that even 512 atoms per pass do not fit is reported, and the engine recovers"""
    pos, cell, pbc, types = workloads.structure_config2()
    m = kk.Model(workloads.write_model("config1", str(tmp_path)))
    L = _lib.lib()
    ref = kk.System(m, ["W"], skin=0.0, chunksize=0).compute(types, pos, cell, pbc)
    s = kk.System(m, ["W"], skin=0.0)                    # chunksize -1: automatic
    out = s.compute(types, pos, cell, pbc)
    assert s.chunksize == 0                              # fits: one pass
    _same(out, ref, len(pos))
    s.release_buffers()
    said = []
    kk.set_logger(lambda level, msg: said.append((level, msg)))
    try:
        s2 = kk.System(m, ["W"], skin=0.0)
        L.gr_set_memory_limit(L.gr_memory_in_use() + 900 * 1024 * 1024)
        out = s2.compute(types, pos, cell, pbc)
        assert s2.chunksize == 1024                      # the largest power of two whose work buffers fit 70 % of 900 MB
        assert any(level == 0 and "chunksize auto: 1024 atoms per pass" in msg for level, msg in said)
        _same(out, ref, len(pos))
        # a fixed chunk that does not fit: reported, not retried
        s2.release_buffers()
        L.gr_set_memory_limit(0)
        s3 = kk.System(m, ["W"], skin=0.0, chunksize=8000)
        L.gr_set_memory_limit(L.gr_memory_in_use() + 900 * 1024 * 1024)
        with pytest.raises(RuntimeError, match="does not fit"):
            s3.compute(types, pos, cell, pbc)
        L.gr_set_memory_limit(L.gr_memory_in_use() + 60 * 1024 * 1024)
        with pytest.raises(RuntimeError, match="does not fit"):
            s2.compute(types, pos, cell, pbc)
        assert any(level == 0 and "chunksize auto: 512 atoms per pass" in msg for level, msg in said)
    finally:
        L.gr_set_memory_limit(0)
        kk.set_logger(None)
    out = s2.compute(types, pos, cell, pbc)              # the engine is usable again
    _same(out, ref, len(pos))


def test_outputs_accumulate_on_request(model_dir):
    """GR_FLAG_ACCUMULATE: the outputs of a call are added to the caller's values (libgrace/include/grace/system.h:66-75)"""
    pos, cell, pbc, types = cases.structure_alloy54()
    perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, 5.0)
    eng = kk.Engine(kk.Model(cases.model_file(model_dir, "mix2")), ["Mo", "W"], 64)
    args = dict(positions=pos[perm], image=image, shifts=shifts, energies=True)
    one = eng.compute(types[perm], offset, j, **args)
    two = eng.compute(types[perm], offset, j, add_to=one, **args)
    for k in ("energy", "forces", "virial", "energies"):
        assert np.allclose(two[k], 2.0 * np.asarray(one[k]), rtol=0, atol=1e-11 * max(1.0, np.abs(one[k]).max()))
