"""The LAMMPS-style entry point (gr_compute_lammps): owned and ghost atoms with a full neighbour list, against the CSR
call on the same structure.  The inputs are built as a LAMMPS rank would hold them: ghosts = periodic images of the owned
atoms within cutoff + skin of the box, the list of every owned atom with all neighbours inside cutoff + skin (more than
the model's cutoff: the engine filters), neighbour indices in shuffled order and with special-bond bits set in the two top
bits, the owner of every ghost from the tag map.  Needs an MI355X."""
import os

import numpy as np
import pytest

import cases
from grace_runtime_amd import kk

pytestmark = pytest.mark.gpu


def lammps_inputs(pos, cell, types, reach, seed=0):
    n = len(pos)
    inv = np.linalg.inv(cell)
    pos = pos - np.floor(pos @ inv) @ cell                          # wrapped into the box
    h = 1.0 / np.linalg.norm(inv, axis=0)                           # distances between the faces
    m = np.ceil(reach / h).astype(int)
    x, t, owner = [pos], [types], [np.arange(n)]
    for a in range(-m[0], m[0] + 1):
        for b in range(-m[1], m[1] + 1):
            for c in range(-m[2], m[2] + 1):
                if (a, b, c) == (0, 0, 0):
                    continue
                p = pos + a * cell[0] + b * cell[1] + c * cell[2]
                f = p @ inv
                keep = np.all((f > -reach / h) & (f < 1.0 + reach / h), axis=1)
                x.append(p[keep])
                t.append(types[keep])
                owner.append(np.arange(n)[keep])
    x, t, owner = np.concatenate(x), np.concatenate(t).astype(np.int32), np.concatenate(owner).astype(np.int32)
    rng = np.random.default_rng(seed)
    rows = []
    for i in range(n):
        d = x - x[i]
        nb = np.nonzero(((d * d).sum(1) < reach * reach) & (np.arange(len(x)) != i))[0].astype(np.int32)
        rng.shuffle(nb)
        nb = nb | (rng.integers(0, 4, nb.size).astype(np.int32) << 30)       # special-bond bits, removed by neighmask
        rows.append(nb)
    return x, t, owner, rows


@pytest.mark.parametrize("model,species,struct", [("mix2", ["Mo", "W"], "alloy54"), ("l2mix", ["Mo", "W"], "triclinic"),
                                                  ("l3mix", ["Mo", "W"], "alloy54")])
def test_lammps_call_equals_csr_call(model_dir, model, species, struct):
    eng = kk.Engine(kk.Model(cases.model_file(model_dir, model)), species, 64)
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    n = len(pos)
    ref = kk.System(eng.model, species, skin=0.0).compute(types, pos, cell, pbc, energies=True)
    rc = max(eng.cutoff(a, b) for a in (1, 2) for b in (1, 2))
    x, t, owner, rows = lammps_inputs(pos, cell, types, rc + 0.7)
    f0 = np.random.default_rng(1).standard_normal((len(x), 3))              # forces are added to what the array holds
    out = eng.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows, owner=owner, energies=True, forces=f0.copy())
    fs = max(1.0, np.abs(ref["forces"]).max())
    assert abs(out["energy"] - ref["energy"]) < 1e-10 * max(1.0, abs(ref["energy"]))
    assert np.abs(out["forces"][:n] - f0[:n] - ref["forces"]).max() < 1e-9 * fs
    assert np.array_equal(out["forces"][n:], f0[n:])                        # nothing is left on the ghosts
    assert np.abs(out["virial"] - ref["virial"]).max() < 1e-9 * max(1.0, np.abs(ref["virial"]).max())
    assert np.abs(out["energies"][:n] - ref["energies"]).max() < 1e-10 * fs and np.all(out["energies"][n:] == 0)
    eo = eng.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows, owner=owner, energy_only=True)
    assert abs(eo["energy"] - ref["energy"]) < 1e-10 * max(1.0, abs(ref["energy"])) and "forces" not in eo


@pytest.mark.parametrize("layout", ["right", "left"])
@pytest.mark.parametrize("model,species,struct", [("mix2", ["Mo", "W"], "alloy54"), ("l2mix", ["Mo", "W"], "triclinic")])
def test_device_arrays_equal_host_arrays(model_dir, model, species, struct, layout):
    """the KOKKOS form of the call (every array on the device, the 2-d neighbour view in either layout) = the host form"""
    import torch
    eng = kk.Engine(kk.Model(cases.model_file(model_dir, model)), species, 64)
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    n = len(pos)
    rc = max(eng.cutoff(a, b) for a in (1, 2) for b in (1, 2))
    x, t, owner, rows = lammps_inputs(pos, cell, types, rc + 0.7)
    f0 = np.random.default_rng(1).standard_normal((len(x), 3))
    ref = eng.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows, owner=owner, energies=True, forces=f0.copy())
    dev = torch.device("cuda", 0)
    maxn = max(len(r) for r in rows) + 3
    nbh = np.full((n, maxn), -7, np.int32)                                  # entries beyond numneigh are never read
    for i, r in enumerate(rows):
        nbh[i, :len(r)] = r
    nb = torch.as_tensor(nbh, device=dev)
    if layout == "left":
        nb = nb.t().contiguous().t()                                        # column-major storage, same shape
        assert nb.stride(0) == 1
    td, xd, od = torch.as_tensor(t, device=dev), torch.as_tensor(x, device=dev), torch.as_tensor(owner, device=dev)
    il = torch.arange(n, dtype=torch.int32, device=dev)
    nn = torch.as_tensor(np.array([len(r) for r in rows], np.int32), device=dev)
    f, ea = torch.as_tensor(f0.copy(), device=dev), torch.zeros(len(x), dtype=torch.float64, device=dev)
    out = eng.compute_lammps_device(n, td, xd, il, nn, nb, owner=od, forces=f, eatom=ea)
    fs = max(1.0, np.abs(ref["forces"]).max())
    assert abs(out["energy"] - ref["energy"]) < 1e-10 * max(1.0, abs(ref["energy"]))
    assert np.abs(f.cpu().numpy() - ref["forces"]).max() < 1e-9 * fs
    assert np.abs(out["virial"] - ref["virial"]).max() < 1e-9 * max(1.0, np.abs(ref["virial"]).max())
    assert np.abs(ea.cpu().numpy() - ref["energies"]).max() < 1e-10 * fs
    eo = eng.compute_lammps_device(n, td, xd, il, nn, nb, owner=od, energy_only=True)
    assert abs(eo["energy"] - ref["energy"]) < 1e-10 * max(1.0, abs(ref["energy"]))
    with pytest.raises(ValueError, match="owner"):
        eng.compute_lammps_device(n, td, xd, il, nn, nb, owner=None, forces=f)
    bad = od.clone()
    bad[n:] = n + 5
    with pytest.raises(ValueError, match="owner of a ghost"):
        eng.compute_lammps_device(n, td, xd, il, nn, nb, owner=bad, forces=f)
    with pytest.raises(ValueError, match="must be on the module's GPU"):
        eng.compute_lammps_device(n, td, torch.as_tensor(x), il, nn, nb, owner=od, forces=f)


def test_unmapped_types_take_no_part_and_argument_errors(model_dir):
    """pair_style hybrid: atoms of a type without a model element are neither central atoms nor neighbours"""
    model = kk.Model(cases.model_file(model_dir, "mix2"))
    eng2 = kk.Engine(model, ["Mo", "W"], 64)
    pos, cell, pbc, types = cases.structure_alloy54()
    n = len(pos)
    x, t, owner, rows = lammps_inputs(pos, cell, types, 5.6)
    ref = eng2.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows, owner=owner)
    # a third atom type the engine does not know (C API: type2mu = -1), sprinkled in as extra owned atoms and neighbours
    eng3 = kk.Engine(model, ["Mo", "W", None], 64)
    if True:
        extra = np.random.default_rng(2).uniform(0, 1, (5, 3)) @ cell
        x3 = np.concatenate([x[:n], extra, x[n:]])
        t3 = np.concatenate([t[:n], np.full(5, 3, np.int32), t[n:]])
        shift = lambda a: np.where(a >= n, a + 5, a)
        owner3 = np.concatenate([owner[:n], np.arange(n, n + 5), shift(owner[n:])]).astype(np.int32)
        rows3 = [np.concatenate([(shift(r & 0x1FFFFFFF) | (r & ~0x1FFFFFFF)).astype(np.int32), np.arange(n, n + 5, dtype=np.int32)]) for r in rows]
        rows3 += [np.arange(10, dtype=np.int32)] * 5
        mapped = np.arange(n)
        out = eng3.compute_lammps(n + 5, t3, x3, mapped, [len(r) for r in rows3], rows3, owner=owner3)
        assert abs(out["energy"] - ref["energy"]) < 1e-10 * abs(ref["energy"])
        assert np.abs(out["forces"][:n] - ref["forces"][:n]).max() < 1e-9 and np.all(out["forces"][n:n + 5] == 0)
        with pytest.raises(RuntimeError, match="unmapped type"):
            eng3.compute_lammps(n + 5, t3, x3, np.arange(n + 5), [len(r) for r in rows3], rows3, owner=owner3)
    with pytest.raises(ValueError, match="owner map"):
        eng2.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows)
    with pytest.raises(ValueError, match="must be in ilist"):
        eng2.compute_lammps(n, t, x, np.arange(n - 1), [len(r) for r in rows], rows, owner=owner)
    bad = owner.copy()
    bad[n] = (owner[n] + 1) % n if t[(owner[n] + 1) % n] != t[n] else (owner[n] + 2) % n
    if t[bad[n]] != t[n]:
        with pytest.raises(ValueError, match="owner of ghost"):
            eng2.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows, owner=bad)

