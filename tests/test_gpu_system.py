"""The device-resident structure (gr_system_*, kk.System): the neighbour list whose pair search runs on the GPU against
the host list of the library and the list of the compiled reference (tests/golden/reference_outputs.npz), bit for bit
with the order of the bonds included; the rebuild policy; results in the caller's atom order.  Needs an MI355X."""
import os

import numpy as np
import pytest

import cases
from grace_runtime_amd import kk

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def model(model_dir):
    return kk.Model(cases.model_file(model_dir, "mix2"))


def test_device_list_equals_reference_list(model, gold):
    """every golden structure (cubic, triclinic with images of the atoms themselves, slab, molecule, fcc alloy): with
    skin = list cutoff - model cutoff the system searches at exactly the golden list's cutoff"""
    keys = sorted({k.split("/")[1] for k in gold if k.startswith("nl/")})
    assert len(keys) >= 5
    rc_model = 5.0
    done = 0
    for key in keys:
        struct, rc = key.split("@")
        rc = float(rc)
        if rc < rc_model:
            continue
        pos, cell, pbc, types = cases.STRUCTURES[struct]()
        types = np.minimum(types, 2).astype(np.int32)
        s = kk.System(model, ["Mo", "W"], skin=rc - rc_model)
        assert s.cutoff == rc_model
        s.compute(types, pos, cell, pbc)
        assert s.list_on_device
        perm, offset, j, image, shifts = s.neighbor_list()
        for name, got in (("perm", perm), ("offset", offset), ("j", j), ("image", image)):
            assert np.array_equal(got, gold[f"nl/{key}/{name}"]), (key, name)      # bit-exact, order included
        ref = gold[f"nl/{key}/shifts"]
        assert shifts.shape == ref.shape and np.abs(shifts - ref).max() <= 4e-16 * max(1.0, np.abs(ref).max())
        # and the host search of the library, shift table included
        pcell, shift = kk._padded_cell_arrays(cell, pos, rc, pbc)
        host = kk.neighbor_search(pos + shift, pcell, pbc, rc)
        assert all(np.array_equal(a, b) for a, b in zip(host, (perm, offset, j, image, shifts)))
        done += 1
    assert done >= 5


def test_device_list_at_benchmark_size(model):
    pos, cell, pbc, types = cases.structure_config2()
    s = kk.System(model, ["Mo", "W"], skin=1.0)
    out = s.compute(types, pos, cell, pbc)
    dev = s.neighbor_list()
    host = kk.neighbor_search(pos, cell, pbc, 6.0, num_threads=8)
    assert len(dev[2]) == len(host[2]) > 400000
    assert all(np.array_equal(a, b) for a, b in zip(host, dev))
    assert np.abs(out["forces"].sum(0)).max() < 1e-9


def test_far_images_fall_back_to_the_host_search(model):
    """an atom shifted by 2^20 cells: the image differences do not fit the device table"""
    pos, cell, pbc, types = cases.structure_alloy54()
    ref = kk.System(model, ["Mo", "W"], skin=0.0).compute(types, pos, cell, pbc)
    p2 = pos.copy()
    p2[7] += 600000.0 * cell[0]
    s = kk.System(model, ["Mo", "W"], skin=0.0)
    out = s.compute(types, p2, cell, pbc)
    assert not s.list_on_device
    assert abs(out["energy"] - ref["energy"]) < 1e-6 and np.abs(out["forces"] - ref["forces"]).max() < 1e-5


def test_rebuild_policy_and_results(model):
    pos, cell, pbc, types = cases.structure_alloy54()
    eng = kk.Engine(model, ["Mo", "W"], 64)
    s = kk.System(model, ["Mo", "W"], skin=0.5)
    r0 = s.compute(types, pos, cell, pbc, energies=True)
    perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, 5.0)
    direct = eng.compute(types[perm], offset, j, positions=pos[perm], image=image, shifts=shifts, energies=True)
    f = np.empty_like(pos)
    f[perm] = direct["forces"]
    e = np.empty(len(pos))
    e[perm] = direct["energies"]
    assert abs(r0["energy"] - direct["energy"]) < 1e-10 and np.abs(r0["forces"] - f).max() < 1e-10
    assert np.abs(r0["energies"] - e).max() < 1e-10 and np.abs(r0["virial"] - direct["virial"]).max() < 1e-9
    rng = np.random.default_rng(0)
    p1 = pos + rng.uniform(-0.1, 0.1, pos.shape)          # below skin / 2: positions only
    r1 = s.compute(types, p1, cell, pbc)
    assert s.rebuilds == 1
    r1x = kk.System(model, ["Mo", "W"], skin=0.0).compute(types, p1, cell, pbc)
    assert abs(r1["energy"] - r1x["energy"]) < 1e-10 and np.abs(r1["forces"] - r1x["forces"]).max() < 1e-10
    p2 = p1.copy()
    p2[3] += 0.4                                              # above skin / 2
    s.compute(types, p2, cell, pbc)
    assert s.rebuilds == 2
    s.compute(types, p2, cell * 1.001, pbc)                   # another cell
    assert s.rebuilds == 3
    t2 = types.copy()
    t2[0] = 3 - t2[0]
    s.compute(t2, p2, cell * 1.001, pbc)                      # other types
    assert s.rebuilds == 4
    s.compute(t2[:-1], p2[:-1], cell * 1.001, pbc)            # another atom count
    assert s.rebuilds == 5
    eo = s.compute(t2[:-1], p2[:-1], cell * 1.001, pbc, energy_only=True)
    assert s.rebuilds == 5 and "forces" not in eo
    empty = s.compute(np.zeros(0, np.int32), np.zeros((0, 3)), cell, pbc)
    assert empty["energy"] == 0.0 and empty["forces"].shape == (0, 3)
    with pytest.raises(ValueError, match="types must be"):
        s.compute(np.full(3, 5, np.int32), pos[:3], cell, pbc)
    with pytest.raises(ValueError):
        kk.System(model, ["Mo", "W"], skin=-1.0)
