"""The comm surface of the engines (Exchange, comm_width, pack / unpack of the message rows; libgrace/include/grace/system.h:53-60,
kk/grace_2l_kk.h:141-157, kk/grace_3l_kk.h:313-324) on one GPU: a periodic structure is cut into two "ranks", each with its owned
atoms and the ghosts its bonds reach (images of its own atoms and atoms of the other rank).  Two engines run the LAMMPS call
side by side in two host threads; their exchange callbacks move the message rows and the adjoint rows through host buffers, as
MPI would.  The energies of the ranks add up to, and the forces folded back onto their atoms equal, the single-engine result,
the fp64 CPU oracle on the uncut structure and the committed outputs of the compiled reference."""
import threading

import numpy as np
import pytest

import cases
from grace_runtime_amd import kk

pytestmark = pytest.mark.gpu


def two_ranks(pos, cell, pbc, types, rc):
    """per rank: owned global atoms, ghost (global atom, shift) pairs, LAMMPS arrays (x, type, numneigh, firstneigh)"""
    perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, rc)
    n = len(pos)
    inv = np.empty(n, np.int64)
    inv[perm] = np.arange(n)                      # atom -> slot
    rank_of = (pos[:, 0] > np.median(pos[:, 0])).astype(int)
    ranks = []
    for r in (0, 1):
        owned = np.nonzero(rank_of == r)[0]
        local = {(int(a), -1): k for k, a in enumerate(owned)}          # (atom, image) -> local index; image -1: the atom itself
        ghosts, rows = [], []
        zero = [k for k in range(len(shifts)) if not shifts[k].any()]
        for a in owned:
            q = inv[a]
            row = []
            for b in range(offset[q], offset[q + 1]):
                nb_atom, im = int(perm[j[b]]), int(image[b])
                key = (nb_atom, -1) if (im in zero and rank_of[nb_atom] == r) else (nb_atom, im)
                if key not in local:
                    local[key] = len(owned) + len(ghosts)
                    ghosts.append(key)
                row.append(local[key])
            rows.append(np.array(row, np.int32))
        x = np.concatenate([pos[owned], np.array([pos[a] + shifts[im] for a, im in ghosts]).reshape(-1, 3)])
        t = np.concatenate([types[owned], np.array([types[a] for a, _ in ghosts], np.int32)]).astype(np.int32)
        ranks.append(dict(owned=owned, ghosts=ghosts, x=x, type=t, rows=rows, nlocal=len(owned), nall=len(x),
                          index_of={int(a): k for k, a in enumerate(owned)}))
    return ranks, rank_of


def device_call(eng, me, **kw):
    """the rank's arrays as a KOKKOS pair style holds them (device memory, padded 2-d neighbour view); results as the host call's"""
    import torch
    dev = torch.device("cuda", 0)
    nl, nall = me["nlocal"], me["nall"]
    nbh = np.full((nl, max(len(r) for r in me["rows"]) + 1), -3, np.int32)
    for i, r in enumerate(me["rows"]):
        nbh[i, :len(r)] = r
    f, ea = torch.zeros((nall, 3), dtype=torch.float64, device=dev), torch.zeros(nall, dtype=torch.float64, device=dev)
    va = torch.zeros((nall, 6), dtype=torch.float64, device=dev)
    out = eng.compute_lammps_device(nl, torch.as_tensor(me["type"], device=dev), torch.as_tensor(me["x"], device=dev),
                                    torch.arange(nl, dtype=torch.int32, device=dev),
                                    torch.as_tensor(np.array([len(r) for r in me["rows"]], np.int32), device=dev),
                                    torch.as_tensor(nbh, device=dev), owner=None, forces=f, eatom=ea, vatom=va, **kw)
    out["forces"], out["energies"], out["vatom"] = f.cpu().numpy(), ea.cpu().numpy(), va.cpu().numpy()
    return out


@pytest.mark.parametrize("arrays", ["host", "device"])
@pytest.mark.parametrize("model,rc", [("l2mix", 5.0), ("l3mix", 5.0), ("mix2", 5.0)])
def test_two_ranks_with_an_exchange_equal_one_engine(model_dir, gold, model, rc, arrays):
    pos, cell, pbc, types = cases.structure_alloy54()
    m = kk.Model(cases.model_file(model_dir, model))
    ref = kk.System(m, ["Mo", "W"], skin=0.0).compute(types, pos, cell, pbc, energies=True, virials=True)
    ranks, rank_of = two_ranks(pos, cell, pbc, types, rc)
    engines = [kk.Engine(m, ["Mo", "W"], 64) for _ in ranks]
    assert engines[0].comm_layers == {"l2mix": 1, "l3mix": 2, "mix2": 0}[model]
    barrier = threading.Barrier(2, timeout=60)
    shared = [{}, {}]
    calls = [[], []]

    def make(r):
        me, eng, other = ranks[r], engines[r], ranks[1 - r]

        def forward(layer):
            calls[r].append(("f", layer))
            shared[r]["rows"] = eng.pack_forward_host(layer, np.arange(me["nlocal"], dtype=np.int32))
            barrier.wait()
            buf = np.zeros((len(me["ghosts"]), eng.comm_width(layer)))
            for g, (atom, _) in enumerate(me["ghosts"]):
                s = rank_of[atom]
                buf[g] = shared[s]["rows"][ranks[s]["index_of"][atom]]
            eng.unpack_forward_host(layer, me["nlocal"], buf)
            barrier.wait()

        def reverse(layer):
            calls[r].append(("r", layer))
            shared[r]["grows"] = eng.pack_reverse_host(layer, me["nlocal"], len(me["ghosts"]))
            barrier.wait()
            sendlist, rows = [], []
            for s in (0, 1):                      # ghosts of either rank that are images of my atoms
                for g, (atom, _) in enumerate(ranks[s]["ghosts"]):
                    if rank_of[atom] == r:
                        sendlist.append(me["index_of"][atom])
                        rows.append(shared[s]["grows"][g])
            if sendlist:
                eng.unpack_reverse_host(layer, np.array(sendlist, np.int32), np.array(rows))
            barrier.wait()
        return forward, reverse

    out, err = [None, None], [None, None]

    def run(r):
        try:
            me = ranks[r]
            fw, rv = make(r)
            engines[r].set_exchange(fw, rv)
            numneigh = np.array([len(x) for x in me["rows"]], np.int32)
            if arrays == "device":
                out[r] = device_call(engines[r], me)
            else:
                out[r] = engines[r].compute_lammps(me["nlocal"], me["type"], me["x"], np.arange(me["nlocal"], dtype=np.int32), numneigh,
                                                   me["rows"], owner=None, energies=True, vatom=np.zeros((me["nall"], 6)))
        except Exception as e:      # noqa: BLE001
            err[r] = e
            barrier.abort()

    threads = [threading.Thread(target=run, args=(r,)) for r in (0, 1)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert err == [None, None], err
    layers = engines[0].comm_layers
    want = [("f", k) for k in range(1, layers + 1)] + [("r", k) for k in range(layers, 0, -1)]
    assert calls[0] == want and calls[1] == want
    n = len(pos)
    f, ea, va = np.zeros((n, 3)), np.zeros(n), np.zeros((n, 6))
    for r in (0, 1):
        me = ranks[r]
        f[me["owned"]] += out[r]["forces"][:me["nlocal"]]
        ea[me["owned"]] += out[r]["energies"][:me["nlocal"]]
        va[me["owned"]] += out[r]["vatom"][:me["nlocal"]]
        for g, (atom, _) in enumerate(me["ghosts"]):            # LAMMPS' reverse communication of f (and of vatom)
            f[atom] += out[r]["forces"][me["nlocal"] + g]
            va[atom] += out[r]["vatom"][me["nlocal"] + g]
    fs = max(1.0, np.abs(ref["forces"]).max())
    assert abs(out[0]["energy"] + out[1]["energy"] - ref["energy"]) / n < 1e-10 * fs
    assert np.abs(f - ref["forces"]).max() < 1e-9 * fs
    assert np.abs(ea - ref["energies"]).max() < 1e-10 * fs
    assert np.abs(out[0]["virial"] + out[1]["virial"] - ref["virial"]).max() < 1e-8 * fs
    assert np.abs(va - ref["virials"]).max() < 1e-9 * max(1.0, np.abs(ref["virials"]).max())
    # and against the independent sources: the fp64 oracle on the uncut structure's own list, and (5.0 A is the cutoff of these
    # models, so the ranks' lists hold the bonds of the reference's list) the compiled reference's committed outputs
    two = {"energy": out[0]["energy"] + out[1]["energy"], "virial": out[0]["virial"] + out[1]["virial"], "forces": f, "energies": ea}
    orc = cases.oracle_reference(model_dir, model, pos, cell, pbc, types)
    cases.check_against(two, orc, n, 1e-10, 1e-9, 1e-10, 1e-8)
    assert np.abs(va - orc["virials"]).max() < 1e-9 * max(1.0, np.abs(orc["virials"]).max())
    gref = cases.golden_reference(gold, model, "alloy54")
    cases.check_against(two, gref, n, 1e-6, 2e-5, 1e-5, 1e-5)
    if "virials" in gref:
        assert np.abs(va - gref["virials"]).max() < 2e-5 * max(1.0, np.abs(gref["virials"]).max())


def test_device_row_movers_equal_the_host_forms(model_dir):
    import torch
    pos, cell, pbc, types = cases.structure_alloy54()
    m = kk.Model(cases.model_file(model_dir, "l2mix"))
    ranks, rank_of = two_ranks(pos, cell, pbc, types, 5.0)
    me = ranks[0]
    eng = kk.Engine(m, ["Mo", "W"], 64)
    dev = torch.device("cuda", 0)
    seen = {}

    def forward(layer):
        sl = np.arange(0, me["nlocal"], 2, dtype=np.int32)
        host = eng.pack_forward_host(layer, sl)
        d = torch.zeros(host.shape, dtype=torch.float64, device=dev)
        eng.pack_forward(layer, torch.tensor(sl, device=dev), d)
        seen["pack"] = np.array_equal(d.cpu().numpy(), host)
        rows = np.arange(len(me["ghosts"]) * eng.comm_width(layer), dtype=np.float64).reshape(len(me["ghosts"]), -1) * 1e-3
        eng.unpack_forward(layer, me["nlocal"], torch.tensor(rows, device=dev))
        back = eng.pack_forward_host(layer, np.arange(me["nlocal"], me["nall"], dtype=np.int32))
        seen["unpack"] = np.array_equal(back, rows)

    def reverse(layer):
        g = len(me["ghosts"])
        host = eng.pack_reverse_host(layer, me["nlocal"], g)
        d = torch.zeros(host.shape, dtype=torch.float64, device=dev)
        eng.pack_reverse(layer, me["nlocal"], d)
        seen["pack_r"] = np.array_equal(d.cpu().numpy(), host)
        before = eng.pack_reverse_host(layer, 0, 3)
        add = np.full((2, eng.comm_width(layer)), 0.25)
        eng.unpack_reverse(layer, torch.tensor(np.array([1, 1], np.int32), device=dev), torch.tensor(add, device=dev))      # one atom twice
        after = eng.pack_reverse_host(layer, 0, 3)
        seen["unpack_r"] = np.allclose(after[1], before[1] + 0.5) and np.array_equal(after[[0, 2]], before[[0, 2]])

    eng.set_exchange(forward, reverse)
    numneigh = np.array([len(x) for x in me["rows"]], np.int32)
    eng.compute_lammps(me["nlocal"], me["type"], me["x"], np.arange(me["nlocal"], dtype=np.int32), numneigh, me["rows"], owner=None)
    assert seen == {"pack": True, "unpack": True, "pack_r": True, "unpack_r": True}
    # outside a pass of a GRACE-1L engine there is nothing to move
    one = kk.Engine(kk.Model(cases.model_file(model_dir, "mix2")), ["Mo", "W"], 64)
    with pytest.raises(RuntimeError, match="no message rows"):
        one.pack_forward_host(1, np.zeros(1, np.int32))
