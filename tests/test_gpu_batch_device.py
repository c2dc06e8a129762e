"""`Batch.compute_device` (gr_compute_batch_device through the C ABI): atoms and results in device memory, neighbour
lists built on the device.  Checked against `Batch.compute` (host lists, the reference's list order) on the same
structures: periodic, triclinic with atoms outside the cell, slab, molecule, and the small cells of the batched
workload.  The two paths sum the same bonds in different orders: 1e-9 relative.  Needs an MI355X: run with -m gpu."""
import os

import numpy as np
import pytest

import cases
from grace_runtime_amd import kk

pytestmark = pytest.mark.gpu


def _engine(model_dir, name, species):
    return kk.Engine(kk.Model(cases.model_file(model_dir, name)), species, 64)


def _pack(structs):
    natoms = np.array([len(s[0]) for s in structs], np.int32)
    pos = np.concatenate([s[0] for s in structs])
    cells = np.stack([s[1] for s in structs])
    pbc = np.stack([np.asarray(s[2], bool) for s in structs])
    types = np.concatenate([s[3] for s in structs]).astype(np.int32)
    return natoms, types, pos, cells, pbc


def _device_run(b, natoms, types, pos, cells, pbc, energy_only=False, energies=True, **kw):
    import torch
    dev = torch.device("cuda", kk.device() if kk.initialized() else 0)
    S, N = len(natoms), len(types)
    t = torch.as_tensor(types, device=dev)
    x = torch.as_tensor(pos, device=dev)
    e = torch.full((S,), 7.0, dtype=torch.float64, device=dev)
    f = None if energy_only else torch.full((N, 3), 7.0, dtype=torch.float64, device=dev)
    v = None if energy_only else torch.full((S, 6), 7.0, dtype=torch.float64, device=dev)
    ea = torch.full((N,), 7.0, dtype=torch.float64, device=dev) if energies else None
    b.compute_device(natoms, t, x, cells, pbc, e, forces=f, virial=v, energies=ea, energy_only=energy_only, **kw)
    out = {"energy": e.cpu().numpy()}
    if f is not None:
        out["forces"], out["virial"] = f.cpu().numpy(), v.cpu().numpy()
    if ea is not None:
        out["energies"] = ea.cpu().numpy()
    return out


def _compare(out, ref):
    fs = max(1.0, np.abs(ref["forces"]).max())
    assert np.abs(out["energy"] - ref["energy"]).max() < 1e-9 * max(1.0, np.abs(ref["energy"]).max())
    assert np.abs(out["forces"] - ref["forces"]).max() < 1e-9 * fs
    assert np.abs(out["virial"] - ref["virial"]).max() < 1e-9 * max(1.0, np.abs(ref["virial"]).max())
    assert np.abs(out["energies"] - ref["energies"]).max() < 1e-9 * fs


@pytest.mark.parametrize("name", ["mix2", "l2mix", "l3mix"])
def test_device_batch_equals_host_batch(model_dir, name):
    eng = _engine(model_dir, name, ["Mo", "W"])
    mol = cases.structure_molecule()
    structs = [cases.structure_alloy54(), cases.structure_triclinic(), cases.structure_slab(),
               (mol[0], np.zeros((3, 3)), mol[2], mol[3])]
    natoms, types, pos, cells, pbc = _pack(structs)
    b = kk.Batch(eng.model, ["Mo", "W"])
    ref = b.compute(natoms, types, pos, cells, pbc, energies=True)
    out = _device_run(b, natoms, types, pos, cells, pbc)
    assert b.passes == 1
    _compare(out, ref)
    eo = _device_run(b, natoms, types, pos, cells, pbc, energy_only=True, energies=False)
    assert np.abs(eo["energy"] - ref["energy"]).max() < 1e-9 * max(1.0, np.abs(ref["energy"]).max())
    # a second call with fewer structures reuses the buffers
    sub = _pack(structs[1:3])
    out2 = _device_run(b, *sub)
    ref2 = b.compute(*sub, energies=True)
    _compare(out2, ref2)


def test_small_cells_with_several_images_per_direction(model_dir):
    """cells shorter than the cutoff: every atom sees several images of itself and of each neighbour"""
    eng = _engine(model_dir, "config5", ["Al", "Ni", "Ti"])
    structs = [(p, c, [True, True, True], t) for p, c, t in cases.structures_config5(24)]
    rng = np.random.default_rng(11)
    tiny = np.array([[2.9, 0.0, 0.0], [0.3, 3.1, 0.0], [-0.2, 0.4, 3.3]])
    structs.append((rng.uniform(-1, 2, (2, 3)) @ tiny * 0.5 + np.array([[0, 0, 0], [1.4, 1.5, 1.6]]), tiny, [True, True, True],
                    np.array([1, 3], np.int32)))
    structs.append((np.array([[0.1, 0.2, 0.3]]), np.diag([3.0, 3.2, 2.8]), [True, True, True], np.array([2], np.int32)))
    natoms, types, pos, cells, pbc = _pack(structs)
    b = kk.Batch(eng.model, ["Al", "Ni", "Ti"])
    ref = b.compute(natoms, types, pos, cells, pbc, energies=True)
    out = _device_run(b, natoms, types, pos, cells, pbc)
    assert b.passes == 1
    _compare(out, ref)
    # the same batch in passes of at most 300 atoms (whole structures; a structure above the limit is a pass of its own)
    out = _device_run(b, natoms, types, pos, cells, pbc, max_nall=300)
    start = np.concatenate([[0], np.cumsum(natoms)])
    want, g0 = 0, 0
    while g0 < len(natoms):
        g1 = g0 + 1
        while g1 < len(natoms) and start[g1 + 1] - start[g0] <= 300:
            g1 += 1
        want, g0 = want + 1, g1
    assert b.passes == want and want > 3
    _compare(out, ref)
    host = b.compute(natoms, types, pos, cells, pbc, energies=True, max_nall=300)
    assert b.passes == want
    _compare(host, ref)
    with pytest.raises(ValueError, match="max_nall"):
        b.compute(natoms, types, pos, cells, pbc, max_nall=0)


def test_argument_errors(model_dir):
    import torch
    eng = _engine(model_dir, "mix2", ["Mo", "W"])
    b = kk.Batch(eng.model, ["Mo", "W"])
    p, c, pb, t = cases.structure_alloy54()
    dev = torch.device("cuda", 0)
    x, ty = torch.as_tensor(p, device=dev), torch.as_tensor(t, device=dev)
    e = torch.zeros(1, dtype=torch.float64, device=dev)
    with pytest.raises(ValueError, match="must be on the module's GPU"):
        b.compute_device([len(p)], ty, torch.as_tensor(p), c[None], pb[None], e)
    with pytest.raises(ValueError, match="must be on the module's GPU"):
        b.compute_device([len(p)], t, x, c[None], pb[None], e)
    with pytest.raises(ValueError, match="positions: expected"):
        b.compute_device([len(p)], ty, x.float(), c[None], pb[None], e)
    with pytest.raises(ValueError, match="forces: expected"):
        b.compute_device([len(p)], ty, x, c[None], pb[None], e, forces=torch.zeros(len(p) - 1, 3, dtype=torch.float64, device=dev))
    with pytest.raises(ValueError, match="differ in length"):
        b.compute_device([len(p)], ty, x, np.stack([c, c]), pb[None], e)
    with pytest.raises(ValueError, match="no UQ head"):
        b.compute_device([len(p)], ty, x, c[None], pb[None], e, gamma=torch.zeros(len(p), dtype=torch.float64, device=dev))
    bad = ty.clone()
    bad[3] = 3
    with pytest.raises(ValueError, match="types must be 1"):
        b.compute_device([len(p)], bad, x, c[None], pb[None], e)
    # no atoms at all: nothing to do, energies of empty structures are 0
    e2 = torch.full((2,), 5.0, dtype=torch.float64, device=dev)
    b.compute_device([0, 0], ty[:0], x[:0], np.stack([c, c]), np.stack([pb, pb]), e2)
    assert e2.tolist() == [0.0, 0.0]


def test_allocation_failure_halves_the_passes_and_keeps_the_limit(model_dir):
    """python/kk/kk_core.cpp:1452-1484: after an allocation failure the batch runs again from its first structure in
    passes of half as many atoms (not below 16384), on a fresh engine, and later calls start from the limit found.  The
    failure is forced with the library's own memory cap (the GPU is never exhausted)."""
    eng = _engine(model_dir, "config5", ["Al", "Ni", "Ti"])
    structs = [(p, c, [True, True, True], t) for p, c, t in cases.structures_config5(440)]
    natoms, types, pos, cells, pbc = _pack(structs)
    N = int(natoms.sum())
    assert 33000 < N < 65000                      # one halving reaches a pass size above the floor of 16384
    b = kk.Batch(eng.model, ["Al", "Ni", "Ti"], chunksize=0)      # engine passes are not split into chunks of atoms: the batch is
    b.keep_buffers = True                         # the buffers of a call stay, so that what they hold can be measured
    try:
        ref = _device_run(b, natoms, types, pos, cells, pbc, max_nall=N // 2)
        assert b.passes >= 2
        held = kk.memory_in_use()
        b.engine.reset()
        base = kk.memory_in_use()                 # the weights of the engines alive in this process
        assert 0 < base < held
        # enough for passes of N / 2 atoms, not for one pass of N
        kk.set_memory_limit(base + int(1.35 * (held - base)))
        out = _device_run(b, natoms, types, pos, cells, pbc)
        assert b.passes >= 2
        _compare(out, ref)
        p_first = b.passes
        out = _device_run(b, natoms, types, pos, cells, pbc)        # the limit is kept: no failure this time, the same passes
        assert b.passes == p_first
        _compare(out, ref)
        host = b.compute(natoms, types, pos, cells, pbc, energies=True)
        assert b.passes >= 2
        _compare(host, ref)
        # nothing fits (the buffers of the passes that fitted are given back first): an error that says so, and an engine
        # that works again once the cap is lifted
        b.release_buffers()
        kk.set_memory_limit(base + (held - base) // 50)
        with pytest.raises(RuntimeError, match="does not fit the GPU memory"):
            _device_run(b, natoms, types, pos, cells, pbc)
        with pytest.raises(RuntimeError, match="does not fit the GPU memory"):
            b.compute(natoms, types, pos, cells, pbc)
        kk.set_memory_limit(0)
        sub = _pack(structs[:20])
        _compare(_device_run(b, *sub), b.compute(*sub, energies=True))
        # with the automatic chunk size the engine splits the pass itself: one batch pass, chunks of atoms inside it
        b.release_buffers()
        auto = kk.Batch(eng.model, ["Al", "Ni", "Ti"])
        auto.keep_buffers = True
        kk.set_memory_limit(kk.memory_in_use() + int(0.6 * (held - base)))
        out = _device_run(auto, natoms, types, pos, cells, pbc)
        assert auto.passes == 1 and 512 <= auto.chunksize < N
        _compare(out, ref)
    finally:
        kk.set_memory_limit(0)


def test_engine_reset_is_seen_by_a_system(model_dir):
    model = kk.Model(cases.model_file(model_dir, "mix2"))
    s = kk.System(model, ["Mo", "W"], skin=0.3)
    p, c, pb, t = cases.structure_alloy54()
    a = s.compute(t, p, c, pb)
    s.engine.reset()
    b = s.compute(t, p, c, pb)
    assert s.rebuilds == 2 and abs(a["energy"] - b["energy"]) < 1e-9 and np.abs(a["forces"] - b["forces"]).max() < 1e-9


def test_release_buffers_gives_the_work_memory_back(model_dir):
    """Batch.release_buffers / keep_buffers and System.release_buffers (python/kk/kk_api.h:66-156): after a release the
    library holds what it held right after the engine was made (weights, tables), and the next call gives the same
    results"""
    model = kk.Model(cases.model_file(model_dir, "l2mix"))
    structs = [cases.structure_alloy54(), cases.structure_triclinic(), cases.structure_slab()]
    natoms, types, pos, cells, pbc = _pack(structs)
    before = kk.memory_in_use()
    b = kk.Batch(model, ["Mo", "W"])
    built = kk.memory_in_use()
    assert built > before
    b.keep_buffers = True
    ref = b.compute(natoms, types, pos, cells, pbc, energies=True)
    grown = kk.memory_in_use()
    assert grown > built
    b.release_buffers()
    assert kk.memory_in_use() <= built + 4096          # one small record is allocated again at once
    _compare(b.compute(natoms, types, pos, cells, pbc, energies=True), ref)
    assert kk.memory_in_use() > built
    b.keep_buffers = False                              # the reference's default: a batch is a job
    _compare(b.compute(natoms, types, pos, cells, pbc, energies=True), ref)
    assert kk.memory_in_use() <= built + 4096
    _compare(_device_run(b, natoms, types, pos, cells, pbc), ref)
    assert kk.memory_in_use() <= built + 4096
    # a System on a released engine builds its list again
    s = kk.System(model, ["Mo", "W"], skin=0.3)
    p, c, pb, t = structs[0]
    a = s.compute(t, p, c, pb)
    held = kk.memory_in_use()
    s.release_buffers()
    assert kk.memory_in_use() < held
    a2 = s.compute(t, p, c, pb)
    assert s.rebuilds == 2 and abs(a["energy"] - a2["energy"]) < 1e-9 and np.abs(a["forces"] - a2["forces"]).max() < 1e-9
    # an engine with nothing uploaded after a release: an empty pass, not a fault
    eng = _engine(model_dir, "mix2", ["Mo", "W"])
    eng.release_buffers()
    eng.run()
    assert eng.fetch()["energy"] == 0.0
