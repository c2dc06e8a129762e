"""The UQ head of GRACE-1L, GRACE-2L and GRACE-3L on the GPU (k_uq through the C ABI) against the CPU oracle: gamma and sigma to 1e-9 relative in
fp64 (1e-4 with the fp32 network), the cluster index exactly.  Needs an MI355X: run with -m gpu."""
import os

import numpy as np
import pytest

import cases
from grace_runtime_amd import kk
from oracle import grace_oracle as go
from oracle import grace_oracle_2l as go2
from oracle import grace_oracle_3l as go3

pytestmark = pytest.mark.gpu


def _bonds(struct, rc=5.0):
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, rc)
    x, t = pos[perm], types[perm]
    rij = x[j] - np.repeat(x, np.diff(offset), axis=0) + shifts[image]
    return t, offset, j, rij


def _oracle(path, name, t, offset, j, rij):
    if cases.LAYERS[name] == 3:
        return go3.compute_3l(go3.Model3L(path), t - 1, offset, j, rij, uq=True)
    if cases.LAYERS[name] == 2:
        return go2.compute_2l(go2.Model2L(path), t - 1, offset, j, rij, uq=True)
    return go.compute_1l(go.Model1L(path), t - 1, offset, j, rij, uq=True)


# GRACE-2L and GRACE-3L engines compute in fp64 only
@pytest.mark.parametrize("name,precision,tol", [("uq2", 64, 1e-9), ("uq2", 32, 1e-4), ("uq2l", 64, 1e-9), ("uq2l", 32, 1e-4), ("uq3l", 64, 1e-9),
                                                ("uq3l", 32, 1e-4)])
@pytest.mark.parametrize("struct", ["alloy54", "triclinic"])
def test_uq_matches_oracle(model_dir, name, struct, precision, tol):
    path = cases.model_file(model_dir, name)
    eng = kk.Engine(kk.Model(path), ["Mo", "W"], precision)
    t, offset, j, rij = _bonds(struct)
    ref = _oracle(path, name, t, offset, j, rij)
    eng.upload(t, offset, j, rij)
    eng.run(uq=True)
    out, uq = eng.fetch(), eng.fetch_uq()
    full = {k: v.copy() for k, v in uq.items()}
    if precision == 64:
        assert np.array_equal(uq["gmm_cluster"], ref["gmm_cluster"])
        assert abs(out["energy"] - ref["energy"]) < 1e-9 and np.abs(out["forces"] - ref["forces"]).max() < 1e-9
    else:
        far = ref["atomic_sigma"] > 1e-3          # the atom that sits ON a centroid: its sigma is rounding noise in fp32
        assert np.array_equal(uq["gmm_cluster"][far], ref["gmm_cluster"][far])
        uq = {k: v[far] for k, v in uq.items()}
        ref = {k: ref[k][far] for k in ("gamma", "atomic_sigma")}
    assert np.abs(uq["gamma"] / ref["gamma"] - 1).max() < tol
    assert np.abs(uq["atomic_sigma"] / ref["atomic_sigma"] - 1).max() < tol
    # forward only: the same values without the reverse pass
    eng.run(uq=True, energy_only=True)
    fwd = eng.fetch_uq()
    for k in ("gamma", "atomic_sigma", "gmm_cluster"):
        assert np.array_equal(fwd[k], full[k]), k       # the forward pass is the same code at both precisions


@pytest.mark.parametrize("name", ["uq2", "uq2l", "uq3l"])
def test_calculator_level_call_returns_uq_in_the_callers_order(model_dir, name):
    path = cases.model_file(model_dir, name)
    model = kk.Model(path)
    pos, cell, pbc, types = cases.structure_alloy54()
    s = kk.System(model, ["Mo", "W"], skin=0.3)
    out = s.compute(types, pos, cell, pbc, uq=True, energies=True)
    perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, 5.0)
    x, t = pos[perm], types[perm]
    rij = x[j] - np.repeat(x, np.diff(offset), axis=0) + shifts[image]
    ref = _oracle(path, name, t, offset, j, rij)
    for k in ("gamma", "atomic_sigma", "gmm_cluster"):
        want = np.empty(len(t))
        want[perm] = ref[k]
        assert np.abs(out[k] / want - 1).max() < 1e-9 if k != "gmm_cluster" else np.array_equal(out[k], want)
    # a second call on the kept list (positions moved within the skin)
    p2 = pos + np.random.default_rng(2).uniform(-0.05, 0.05, pos.shape)
    o2 = s.compute(types, p2, cell, pbc, uq=True)
    fresh = kk.System(model, ["Mo", "W"], skin=0.0).compute(types, p2, cell, pbc, uq=True)
    assert s.rebuilds == 1 and not np.array_equal(o2["gamma"], out["gamma"])
    assert np.abs(o2["gamma"] / fresh["gamma"] - 1).max() < 1e-9 and np.array_equal(o2["gmm_cluster"], fresh["gmm_cluster"])


def test_uq_errors(model_dir):
    plain = kk.Engine(kk.Model(cases.model_file(model_dir, "mix2")), ["Mo", "W"], 64)
    t, offset, j, rij = _bonds("alloy54")
    plain.upload(t, offset, j, rij)
    with pytest.raises(ValueError, match="no usable UQ head"):
        plain.run(uq=True)
    plain.run()
    with pytest.raises(RuntimeError, match="needs a run with the UQ flag"):
        plain.fetch_uq()
    two = kk.System(kk.Model(cases.model_file(model_dir, "l2mix")), ["Mo", "W"])
    pos, cell, pbc, types = cases.structure_alloy54()
    with pytest.raises(ValueError, match="no usable UQ head"):
        two.compute(types, pos, cell, pbc, uq=True)


@pytest.mark.parametrize("name", ["uq2", "uq2l", "uq3l"])
def test_batches_return_uq_per_atom_in_the_callers_order(model_dir, name):
    """Batch.compute(uq=True) and the gamma / atomic_sigma / gmm_cluster outputs of Batch.compute_device
    (python/kk/kk_api.h:116-156) against one System call per structure, in one pass and in passes of one structure"""
    import torch
    model = kk.Model(cases.model_file(model_dir, name))
    structs = [cases.structure_alloy54(), cases.structure_triclinic(), cases.structure_slab()]
    natoms = np.array([len(s[0]) for s in structs], np.int32)
    pos = np.concatenate([s[0] for s in structs])
    cells = np.stack([s[1] for s in structs])
    pbc = np.stack([np.asarray(s[2], bool) for s in structs])
    types = np.concatenate([s[3] for s in structs]).astype(np.int32)
    one = [kk.System(model, ["Mo", "W"], skin=0.0).compute(s[3], s[0], s[1], s[2], uq=True) for s in structs]
    want = {k: np.concatenate([o[k] for o in one]) for k in ("gamma", "atomic_sigma", "gmm_cluster")}
    b = kk.Batch(model, ["Mo", "W"])
    dev = torch.device("cuda", kk.device())
    for max_nall in (1 << 21, 1):
        out = b.compute(natoms, types, pos, cells, pbc, uq=True, max_nall=max_nall)
        assert b.passes == (1 if max_nall > 1 else 3)
        assert np.array_equal(out["gmm_cluster"], want["gmm_cluster"])
        assert np.abs(out["gamma"] / want["gamma"] - 1).max() < 1e-9 and np.abs(out["atomic_sigma"] / want["atomic_sigma"] - 1).max() < 1e-9
        assert np.abs(out["energy"] - np.array([o["energy"] for o in one])).max() < 1e-9
        g, sg, cl = (torch.full((len(types),), 7.0, dtype=torch.float64, device=dev) for _ in range(3))
        e = torch.zeros(3, dtype=torch.float64, device=dev)
        b.compute_device(natoms, torch.as_tensor(types, device=dev), torch.as_tensor(pos, device=dev), cells, pbc, e, gamma=g,
                         atomic_sigma=sg, gmm_cluster=cl, energy_only=True, max_nall=max_nall)
        assert np.array_equal(cl.cpu().numpy(), want["gmm_cluster"])
        assert np.abs(g.cpu().numpy() / want["gamma"] - 1).max() < 1e-9 and np.abs(sg.cpu().numpy() / want["atomic_sigma"] - 1).max() < 1e-9
    # only one of the three outputs
    g = torch.zeros(len(types), dtype=torch.float64, device=dev)
    b.compute_device(natoms, torch.as_tensor(types, device=dev), torch.as_tensor(pos, device=dev), cells, pbc, e, gamma=g)
    assert np.abs(g.cpu().numpy() / want["gamma"] - 1).max() < 1e-9
    plain = kk.Batch(kk.Model(cases.model_file(model_dir, "mix2")), ["Mo", "W"])
    with pytest.raises(ValueError, match="no UQ head"):
        plain.compute(natoms, types, pos, cells, pbc, uq=True)
