"""Per-atom virials on the GPU (GR_FLAG_VATOM; Outputs::vatom / RunInput::vatom of the reference: libgrace/include/grace/
system.h:71,115, kk/grace_1l_kk.h:93,101) through the C ABI, against the CPU oracles (themselves pinned by the compiled
reference's vatom, tests/test_vatom.py) and the committed reference rows.  Needs an MI355X."""
import numpy as np
import pytest

import cases
from grace_runtime_amd import kk
from test_gpu_lammps import lammps_inputs
from test_vatom import _oracle

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("model,struct,rc", cases.VATOM_CASES)
def test_virials_equal_the_oracle_and_the_reference(model_dir, gold, model, struct, rc, precision):
    m, compute = _oracle(model_dir, model)
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    types = np.minimum(types, m.n_elements).astype(np.int32)
    tag = f"e2e/{model}/{struct}"
    key = f"nl/{struct}@{float(gold[tag + '/rc_list']):g}"
    perm, offset, j, image, shifts = (gold[f"{key}/{k}"] for k in ("perm", "offset", "j", "image", "shifts"))
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    want = compute(m, types[perm] - 1, offset, j, rij)
    species = list(kk.Model(cases.model_file(model_dir, model)).element_names)
    eng = kk.Engine(kk.Model(cases.model_file(model_dir, model)), species, precision)
    eng.upload(types[perm], offset, j, rij=rij)
    eng.run(virials=True)
    out = eng.fetch()
    va = eng.fetch_vatom()
    scale = max(1.0, np.abs(want["virials"]).max())
    tol = 1e-10 if precision == 64 else 2e-5
    assert np.abs(va - want["virials"]).max() < tol * scale
    assert np.abs(va - gold[tag + "/virials"]).max() < 2e-5 * scale
    assert np.abs(va.sum(0) - out["virial"]).max() < 1e-10 * max(1.0, np.abs(out["virial"]).max())
    # a run without the flag has no rows to give; an energy-only run neither
    eng.run()
    with pytest.raises(RuntimeError, match="per-atom virial"):
        eng.fetch_vatom()
    eng.run(virials=True, energy_only=True)
    with pytest.raises(RuntimeError, match="per-atom virial"):
        eng.fetch_vatom()


@pytest.mark.parametrize("model", ["mix2", "l2mix", "l3mix"])
def test_virials_of_a_system_in_chunks_and_through_the_lammps_calls(model_dir, model):
    import torch
    mdl = kk.Model(cases.model_file(model_dir, model))
    pos, cell, pbc, types = cases.structure_alloy54()
    n = len(pos)
    one = kk.System(mdl, ["Mo", "W"], skin=0.0, chunksize=0).compute(types, pos, cell, pbc, virials=True)
    va = one["virials"]                                                    # in the caller's atom order
    # the rows every path below is compared with are the oracle's rows (the independent source)
    orc = cases.oracle_reference(model_dir, model, pos, cell, pbc, types)
    assert np.abs(va - orc["virials"]).max() < 1e-10 * max(1.0, np.abs(orc["virials"]).max())
    assert va.shape == (n, 6) and np.abs(va.sum(0) - one["virial"]).max() < 1e-10 * max(1.0, np.abs(one["virial"]).max())
    chunked = kk.System(mdl, ["Mo", "W"], skin=0.0, chunksize=13).compute(types, pos, cell, pbc, virials=True)
    assert np.abs(chunked["virials"] - va).max() < 1e-10 * max(1.0, np.abs(va).max())
    # LAMMPS call with an owner map: the ghosts' halves land on their owners, so the owned rows are the system's rows
    eng = kk.Engine(mdl, ["Mo", "W"], 64)
    rcut = max(eng.cutoff(a, b) for a in (1, 2) for b in (1, 2))
    x, t, owner, rows = lammps_inputs(pos, cell, types, rcut + 0.4)
    inv = np.linalg.inv(cell)
    wrapped = pos - np.floor(pos @ inv) @ cell                              # lammps_inputs wraps the owned atoms: same order
    assert np.allclose(x[:n], wrapped)
    v0 = np.random.default_rng(3).standard_normal((len(x), 6))            # rows are ADDED
    out = eng.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows, owner=owner, vatom=v0.copy())
    assert np.abs(out["vatom"][:n] - v0[:n] - va).max() < 1e-9 * max(1.0, np.abs(va).max())
    assert np.abs(out["vatom"][:n] - v0[:n] - orc["virials"]).max() < 1e-9 * max(1.0, np.abs(va).max())
    assert np.array_equal(out["vatom"][n:], v0[n:])
    with pytest.raises(RuntimeError, match="follow a gr_compute_lammps_device call"):
        kk._lib.check(kk._lib.lib().gr_lammps_add_vatom_device(eng._h, len(x), v0.ctypes.data))
    # device arrays
    dev = torch.device("cuda", 0)
    nbh = np.zeros((n, max(len(r) for r in rows)), np.int32)
    for i, r in enumerate(rows):
        nbh[i, :len(r)] = r
    vd = torch.as_tensor(v0.copy(), device=dev)
    f = torch.zeros((len(x), 3), dtype=torch.float64, device=dev)
    eng.compute_lammps_device(n, torch.as_tensor(t, device=dev), torch.as_tensor(x, device=dev), torch.arange(n, dtype=torch.int32, device=dev),
                              torch.as_tensor(np.array([len(r) for r in rows], np.int32), device=dev), torch.as_tensor(nbh, device=dev),
                              owner=torch.as_tensor(owner, device=dev), forces=f, vatom=vd)
    assert np.abs(vd.cpu().numpy()[:n] - v0[:n] - va).max() < 1e-9 * max(1.0, np.abs(va).max())
    assert np.abs(vd.cpu().numpy()[:n] - v0[:n] - orc["virials"]).max() < 1e-9 * max(1.0, np.abs(va).max())
    assert np.array_equal(vd.cpu().numpy()[n:], v0[n:])


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("model", ["mix2", "l2mix", "l3mix"])
def test_centroid_form(model_dir, model, precision):
    """cvatom of the reference's GPU engines (kk/grace_1l_kk.h:94; kk/grace_1l_kk_impl.h:1344-1362): the six components of
    vatom followed by yx zx zy.  The lower three are held to the upper three of the same structure with its axes exchanged
    (the upper three are pinned by the reference's vatom), to the 1L oracle's centroid rows, and to the symmetric total."""
    from test_vatom import permuted_centroid
    mdl = kk.Model(cases.model_file(model_dir, model))
    pos, cell, pbc, types = cases.structure_alloy54()
    n = len(pos)
    tol = 1e-9 if precision == 64 else 2e-5
    s = kk.System(mdl, ["Mo", "W"], skin=0.0, chunksize=0, precision=precision)
    one = s.compute(types, pos, cell, pbc, virials=True)
    cv = one["centroid_virials"]
    scale = max(1.0, np.abs(cv).max())
    assert cv.shape == (n, 9) and np.array_equal(cv[:, :6], one["virials"])
    assert np.abs(cv[:, 6:] - cv[:, 3:6]).max() > 1e-6
    tot = cv.sum(0)
    assert np.abs(tot[6:] - tot[3:6]).max() < tol * max(1.0, np.abs(tot).max()) * 10
    for p in ([1, 0, 2], [1, 2, 0]):
        outp = s.compute(types, pos[:, p], cell[:, p], pbc, virials=True)
        assert abs(outp["energy"] - one["energy"]) < tol * max(1.0, abs(one["energy"]))
        assert np.abs(outp["centroid_virials"] - permuted_centroid(cv, p)).max() < tol * scale
    chunked = kk.System(mdl, ["Mo", "W"], skin=0.0, chunksize=13, precision=precision).compute(types, pos, cell, pbc, virials=True)
    assert np.abs(chunked["centroid_virials"] - cv).max() < tol * scale
    s.compute(types, pos, cell, pbc)                                       # the list of the structure as given again
    if model == "mix2":
        m, compute = _oracle(model_dir, model)
        perm, offset, j, image, shifts = s.neighbor_list()
        rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
        want = compute(m, types[perm] - 1, offset, j, rij)["centroid_virials"]
        assert np.abs(cv[perm] - want).max() < tol * scale
    # the LAMMPS calls: rows are ADDED, ghosts' halves on their owners
    eng = kk.Engine(mdl, ["Mo", "W"], precision)
    rcut = max(eng.cutoff(a, b) for a in (1, 2) for b in (1, 2))
    x, t, owner, rows = lammps_inputs(pos, cell, types, rcut + 0.4)
    v0 = np.random.default_rng(5).standard_normal((len(x), 9))
    out = eng.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows, owner=owner, cvatom=v0.copy())
    assert np.abs(out["cvatom"][:n] - v0[:n] - cv).max() < tol * scale
    assert np.array_equal(out["cvatom"][n:], v0[n:])
    import torch
    dev = torch.device("cuda", 0)
    nbh = np.zeros((n, max(len(r) for r in rows)), np.int32)
    for i, r in enumerate(rows):
        nbh[i, :len(r)] = r
    vd = torch.as_tensor(v0.copy(), device=dev)
    f = torch.zeros((len(x), 3), dtype=torch.float64, device=dev)
    eng.compute_lammps_device(n, torch.as_tensor(t, device=dev), torch.as_tensor(x, device=dev), torch.arange(n, dtype=torch.int32, device=dev),
                              torch.as_tensor(np.array([len(r) for r in rows], np.int32), device=dev), torch.as_tensor(nbh, device=dev),
                              owner=torch.as_tensor(owner, device=dev), forces=f, cvatom=vd)
    assert np.abs(vd.cpu().numpy()[:n] - v0[:n] - cv).max() < tol * scale
    assert np.array_equal(vd.cpu().numpy()[n:], v0[n:])
    # the rows of the engine call
    eng.upload(*_csr(s, types, pos))
    eng.run(virials=True)
    assert np.abs(eng.fetch_cvatom()[np.argsort(s.neighbor_list()[0])] - cv).max() < tol * scale


def _csr(system, types, pos):
    perm, offset, j, image, shifts = system.neighbor_list()
    return types[perm], offset, j, cases.bond_vectors(pos, perm, offset, j, image, shifts)
