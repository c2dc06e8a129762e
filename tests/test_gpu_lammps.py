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
def test_lammps_call_equals_csr_call(model_dir, gold, model, species, struct):
    eng = kk.Engine(kk.Model(cases.model_file(model_dir, model)), species, 64)
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    n = len(pos)
    ref = kk.System(eng.model, species, skin=0.0).compute(types, pos, cell, pbc, energies=True)
    # the independent sources: the fp64 oracle on the structure's own list and the compiled reference's committed outputs
    orc = cases.oracle_reference(model_dir, model, pos, cell, pbc, types)
    gref = cases.golden_reference(gold, model, struct)
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
    mine = dict(out, forces=out["forces"][:n] - f0[:n])
    cases.check_against(mine, orc, n, 1e-10, 1e-9, 1e-10, 1e-9)                 # fp64 oracle
    cases.check_against(mine, gref, n, 1e-6, 2e-5, 1e-5, 1e-5)                  # compiled reference (fp32 + tables): its gate
    eo = eng.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows, owner=owner, energy_only=True)
    assert abs(eo["energy"] - ref["energy"]) < 1e-10 * max(1.0, abs(ref["energy"])) and "forces" not in eo
    assert abs(eo["energy"] - orc["energy"]) / n < 1e-10 * fs
    # ghosts as atoms of their own (no owner map; GRACE-1L has no message to exchange): forces folded onto the owners
    if eng.comm_layers == 0:
        loose = eng.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows, energies=True)
        folded = loose["forces"][:n].copy()
        np.add.at(folded, owner[n:], loose["forces"][n:])
        cases.check_against(dict(loose, forces=folded), orc, n, 1e-10, 1e-9, 1e-10, 1e-9)


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
    orc = cases.oracle_reference(model_dir, model, pos, cell, pbc, types)
    cases.check_against({"energy": out["energy"], "virial": out["virial"], "forces": f.cpu().numpy()[:n] - f0[:n],
                         "energies": ea.cpu().numpy()}, orc, n, 1e-10, 1e-9, 1e-10, 1e-9)
    eo = eng.compute_lammps_device(n, td, xd, il, nn, nb, owner=od, energy_only=True)
    assert abs(eo["energy"] - ref["energy"]) < 1e-10 * max(1.0, abs(ref["energy"]))
    if eng.comm_layers:                                                     # a message needs the map or an exchange
        with pytest.raises(ValueError, match="owner map"):
            eng.compute_lammps_device(n, td, xd, il, nn, nb, owner=None, forces=f)
    else:                                                                   # GRACE-1L: the ghosts keep what they receive
        f2 = torch.zeros_like(f)
        loose = eng.compute_lammps_device(n, td, xd, il, nn, nb, owner=None, forces=f2)
        folded = f2[:n].cpu().numpy().copy()
        np.add.at(folded, owner[n:], f2[n:].cpu().numpy())
        assert abs(loose["energy"] - ref["energy"]) < 1e-10 * max(1.0, abs(ref["energy"]))
        assert np.abs(folded - (ref["forces"][:n] - f0[:n])).max() < 1e-9 * fs
    bad = od.clone()
    bad[n:] = n + 5
    with pytest.raises(ValueError, match="owner of a ghost"):
        eng.compute_lammps_device(n, td, xd, il, nn, nb, owner=bad, forces=f)
    with pytest.raises(ValueError, match="must be on the module's GPU"):
        eng.compute_lammps_device(n, td, torch.as_tensor(x), il, nn, nb, owner=od, forces=f)


@pytest.mark.parametrize("model,species,struct", [("mix2", ["Mo", "W"], "alloy54"), ("l3mix", ["Mo", "W"], "triclinic")])
def test_same_list_renews_only_the_bond_vectors(model_dir, model, species, struct):
    """the steps between two reneighbourings: the arrays stay, the positions in them move; a call with same_list gives what a
    call that converts the list anew gives, and falls back to the conversion when the engine holds another list"""
    import torch
    eng = kk.Engine(kk.Model(cases.model_file(model_dir, model)), species, 64)
    fresh = kk.Engine(eng.model, species, 64)
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    n = len(pos)
    rc = max(eng.cutoff(a, b) for a in (1, 2) for b in (1, 2))
    x, t, owner, rows = lammps_inputs(pos, cell, types, rc + 0.7)
    dev = torch.device("cuda", 0)
    nbh = np.zeros((n, max(len(r) for r in rows)), np.int32)
    for i, r in enumerate(rows):
        nbh[i, :len(r)] = r
    td, xd, od, nb = (torch.as_tensor(a, device=dev) for a in (t, x, owner, nbh))
    il = torch.arange(n, dtype=torch.int32, device=dev)
    nn = torch.as_tensor(np.array([len(r) for r in rows], np.int32), device=dev)
    rng = np.random.default_rng(5)

    def call(e, same):
        f, ea = torch.zeros((len(x), 3), dtype=torch.float64, device=dev), torch.zeros(len(x), dtype=torch.float64, device=dev)
        out = e.compute_lammps_device(n, td, xd, il, nn, nb, owner=od, forces=f, eatom=ea, same_list=same)
        return out["energy"], out["virial"], f.cpu().numpy(), ea.cpu().numpy()

    first = call(eng, True)                                  # nothing kept yet: converts
    e0 = first[0]
    for step in range(3):
        d = 0.02 * rng.standard_normal((n, 3))
        xd += torch.as_tensor(d[owner], device=dev)          # owners and their images move together
        got, want = call(eng, True), call(fresh, False)
        assert abs(got[0] - want[0]) < 1e-11 * max(1.0, abs(want[0])) and abs(got[0] - e0) > 1e-6
        for a, b in zip(got[1:], want[1:]):                  # sums by atomic adds: equal up to their order
            assert np.abs(a - b).max() < 1e-11 * max(1.0, np.abs(b).max())
        # the same_list step against the oracle on the moved atoms (its own list, searched anew)
        moved = xd[:n].cpu().numpy()
        orc = cases.oracle_reference(model_dir, model, moved, cell, pbc, types)
        cases.check_against({"energy": got[0], "virial": got[1], "forces": got[2][:n], "energies": got[3]}, orc, n, 1e-10, 1e-9, 1e-10, 1e-9)
    # another list on the engine in between: the hint is dropped and the list converted again
    eng.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows, owner=owner)
    got, want = call(eng, True), call(fresh, False)
    assert abs(got[0] - want[0]) < 1e-11 * max(1.0, abs(want[0]))
    assert all(np.abs(a - b).max() < 1e-11 * max(1.0, np.abs(b).max()) for a, b in zip(got[1:], want[1:]))


def test_cxx_adapter_header_runs_a_pair_style_pass(model_dir, tmp_path):
    """include/grace_hip_lammps.hpp (set_model / setup / run(RunInput) -> RunOutput, as a KOKKOS pair style would use it) from
    a C++ program: two passes, the second with same_list on moved atoms, against the Python mirror on the same arrays"""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "build", "adapter_run")
    if not os.path.exists(exe) or os.path.getmtime(exe) < os.path.getmtime(os.path.join(root, "include", "grace_hip_lammps.hpp")):
        sys.path.insert(0, root)
        import __graft_entry__
        exe = __graft_entry__.build_adapter_driver()
    path = cases.model_file(model_dir, "l2mix")
    eng = kk.Engine(kk.Model(path), ["Mo", "W"], 64)
    pos, cell, pbc, types = cases.structure_triclinic()
    n = len(pos)
    x, t, owner, rows = lammps_inputs(pos, cell, types, eng.cutoff(1, 2) + 0.7)
    maxn = max(len(r) for r in rows)
    nbh = np.zeros((n, maxn), np.int32)
    for i, r in enumerate(rows):
        nbh[i, :len(r)] = r
    dx = (0.03 * np.random.default_rng(3).standard_normal((n, 3)))[owner]
    with open(tmp_path / "in.bin", "wb") as f:
        for a in (np.array([n, len(x), maxn, 2], np.int32), np.array(eng.model.type2mu(["Mo", "W"]), np.int32), t,
                  np.array([len(r) for r in rows], np.int32), nbh, owner, x, dx):
            f.write(np.ascontiguousarray(a).tobytes())
    res = subprocess.run([exe, path, str(tmp_path / "in.bin")], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr
    lines = res.stdout.strip().split("\n")
    nall = len(x)
    assert len(lines) == 2 * (nall + 1) + 1 and lines[-1].startswith("cutoff ") and lines[-1].endswith("layers 1")
    for k, xs in enumerate((x, x + dx)):
        want = eng.compute_lammps(n, t, xs, np.arange(n), [len(r) for r in rows], rows, owner=owner, energies=True)
        head = np.array(lines[k * (nall + 1)].split(), float)
        body = np.array([ln.split() for ln in lines[k * (nall + 1) + 1:(k + 1) * (nall + 1)]], float)
        fs = max(1.0, np.abs(want["forces"]).max())
        assert abs(head[0] - want["energy"]) < 1e-11 * max(1.0, abs(want["energy"]))
        assert np.abs(head[1:] - want["virial"]).max() < 1e-10 * max(1.0, np.abs(want["virial"]).max())
        assert np.abs(body[:, :3] - want["forces"]).max() < 1e-11 * fs and np.abs(body[:, 3] - want["energies"]).max() < 1e-11 * fs


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
    # without an owner map a GRACE-1L engine keeps the ghosts as atoms of their own (no message to exchange): the forces they
    # receive stay on them, and folded back onto their owners they give the result of the call with the map
    loose = eng2.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows)
    folded = loose["forces"][:n].copy()
    np.add.at(folded, owner[n:], loose["forces"][n:])
    assert abs(loose["energy"] - ref["energy"]) < 1e-10 * abs(ref["energy"]) and np.abs(folded - ref["forces"][:n]).max() < 1e-9
    # an engine with a message needs the map or an exchange
    two = kk.Engine(kk.Model(cases.model_file(model_dir, "l2mix")), ["Mo", "W"], 64)
    with pytest.raises(ValueError, match="owner map"):
        two.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows)
    with pytest.raises(ValueError, match="must be in ilist"):
        eng2.compute_lammps(n, t, x, np.arange(n - 1), [len(r) for r in rows], rows, owner=owner)
    bad = owner.copy()
    bad[n] = (owner[n] + 1) % n if t[(owner[n] + 1) % n] != t[n] else (owner[n] + 2) % n
    if t[bad[n]] != t[n]:
        with pytest.raises(ValueError, match="owner of ghost"):
            eng2.compute_lammps(n, t, x, np.arange(n), [len(r) for r in rows], rows, owner=bad)

