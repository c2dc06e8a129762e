"""Writes tests/golden/reference_outputs.npz: outputs of the COMPILED REFERENCE (oracle/_ref, built by
oracle/Makefile from the reference checkout) on the synthetic cases of tests/cases.py:

* its neighbour list (perm, offset, j, image, shifts) per structure            -> pins the host / device list
* its energy, per-atom energies, forces, virial per (model, structure) case    -> pins the oracle and the HIP path
  on models the reference's own TF goldens do not cover (AAAA stage, A width != FC width, pair cutoffs, lmax 3/4,
  GRACE-2L at lmax 4 and with unequal stage widths, the reference's 2L fixture models with the BBBB stage, and every
  GRACE-3L case: the reference checkout holds no 3L model file, so its compiled drivers on generated models are the
  only reference outputs there are)

Run in the build container (needs oracle/_ref):  python tests/golden/make_golden.py [--all]
Cases already in the file are kept as they are unless --all is given.
"""
import os
import sys
import tempfile

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import cases  # noqa: E402
from grace_runtime_amd.kk import _padded_cell_arrays  # noqa: E402
from oracle import ref_lib  # noqa: E402


def main():
    out = {}
    target = os.path.join(cases.GOLDEN, "reference_outputs.npz")
    if "--all" not in sys.argv and os.path.exists(target):
        with np.load(target) as z:
            out = {k: z[k] for k in z.files}
    tmp = tempfile.mkdtemp()
    lists = {}
    for model, struct, rc_list in cases.E2E_CASES + cases.E2E_CASES_2L + cases.E2E_CASES_3L:
        if f"e2e/{model}/{struct}/energy" in out:
            continue
        path = cases.write_model(model, tmp)
        d = cases.MODELS[model]()
        nel = int(d["n_elements"][0])
        ref = ref_lib.RefModel(path, list(range(nel)))
        pos, cell, pbc, types = cases.STRUCTURES[struct]()
        types = np.minimum(types, nel).astype(np.int32)
        rc = rc_list if rc_list is not None else max(ref.cutoff(a, b) for a in range(1, nel + 1) for b in range(1, nel + 1))
        pcell, shift = _padded_cell_arrays(cell, pos, rc, pbc)
        nl = ref_lib.neighbor_search(pos + shift, pcell, pbc, rc, 2)
        key = f"{struct}@{rc:g}"
        if key not in lists:
            lists[key] = nl
            for k, v in nl.items():
                out.setdefault(f"nl/{key}/{k}", v)
        r = ref.compute(types[nl["perm"]], nl["offset"], nl["j"], positions=pos[nl["perm"]], image=nl["image"],
                        shifts=nl["shifts"] if len(nl["shifts"]) else np.zeros((1, 3)), nthreads=2)
        tag = f"e2e/{model}/{struct}"
        out[f"{tag}/rc_list"] = np.array(rc)
        for k in ("energy", "energies", "forces", "virial"):
            out[f"{tag}/{k}"] = np.asarray(r[k])
        print(tag, key, "bonds", len(nl["j"]), "E", r["energy"], "max|F|", np.abs(r["forces"]).max())
    # per-atom virials (ComputeFlags::vflag_atom) of a 1L, 2L and 3L case each, on the golden list of the structure
    for model, struct, rc_list in cases.VATOM_CASES:
        tag = f"e2e/{model}/{struct}"
        if f"{tag}/virials" in out:
            continue
        path = cases.write_model(model, tmp)
        nel = int(cases.MODELS[model]()["n_elements"][0])
        ref = ref_lib.RefModel(path, list(range(nel)))
        pos, cell, pbc, types = cases.STRUCTURES[struct]()
        types = np.minimum(types, nel).astype(np.int32)
        key = f"{struct}@{float(out[tag + '/rc_list']):g}"
        nl = {k: out[f"nl/{key}/{k}"] for k in ("perm", "offset", "j", "image", "shifts")}
        rij = cases.bond_vectors(pos, nl["perm"], nl["offset"], nl["j"], nl["image"], nl["shifts"])
        r = ref.compute_vatom(types[nl["perm"]], nl["offset"], nl["j"], rij, nthreads=2)
        assert abs(r["energy"] - float(out[tag + "/energy"])) < 1e-9 * max(1.0, abs(r["energy"]))
        out[f"{tag}/virials"] = r["virials"]                     # rows in the order of the list (perm)
        print(tag, "virials: sum - virial", np.abs(r["virials"].sum(0) - r["virial"]).max())
    # the reference's own 2L fixture models without TF goldens, on its fixture cells (CSR bonds as stored there)
    for model, cell in cases.FIXTURE_CASES_2L:
        if f"fixture/{model}/{cell}/energy" in out:
            continue
        with np.load(os.path.join(cases.REF_FIXTURES, cell + ".npz")) as c:
            types = np.array([2 if z == 74 else 1 for z in c["numbers"]], dtype=np.int32)
            offset, j, rij = c["offset"], c["j"], c["rij"]
        ref = ref_lib.RefModel(os.path.join(cases.REF_FIXTURES, model + ".npz"), [0, 1])    # species (Mo, W)
        r = ref.compute(types, offset, j, rij=rij, nthreads=2)
        tag = f"fixture/{model}/{cell}"
        for k in ("energy", "energies", "forces", "virial"):
            out[f"{tag}/{k}"] = np.asarray(r[k])
        print(tag, "E", r["energy"], "max|F|", np.abs(r["forces"]).max())
    # the UQ head (generated: no fixture of the reference carries one) through the compiled reference, forward only
    for model, struct in cases.UQ_CASES:
        if f"uq/{model}/{struct}/gamma" in out:
            continue
        path = cases.write_model(model, tmp)
        pos, cell, pbc, types = cases.STRUCTURES[struct]()
        nl = ref_lib.neighbor_search(pos, cell, pbc, 5.0, 2)
        rij = cases.bond_vectors(pos, nl["perm"], nl["offset"], nl["j"], nl["image"], nl["shifts"])
        r = ref_lib.RefModel(path, [0, 1]).compute_uq(types[nl["perm"]], nl["offset"], nl["j"], rij, nthreads=2)
        tag = f"uq/{model}/{struct}"
        for k in ("gamma", "atomic_sigma", "gmm_cluster"):
            out[f"{tag}/{k}"] = np.asarray(r[k])
        out[f"{tag}/perm"] = nl["perm"]
        print(tag, "gamma", r["gamma"].min(), r["gamma"].max(), "clusters", np.unique(r["gmm_cluster"]))
    np.savez(target, **out)


if __name__ == "__main__":
    main()


def structure_golden(reference_fixtures="/root/reference/tests/fixtures"):
    """tests/golden/structure_ref.npz: the STRUCTURE arrays (index tables and coupling coefficients, no weights) of
    the reference's own lmax-2/3/4 GRACE-1L fixture models, to check the structure generator of
    grace_runtime_amd/synth.py against the training code's real exports."""
    out = {}
    for name in ("grace_1l_small", "grace_1l_l3", "grace_1l_w48"):
        with np.load(os.path.join(reference_fixtures, name + ".npz")) as z:
            for k in z.files:
                if (k.startswith("prod_") or k.startswith("rho_collect_ind") or k.startswith("rho_w_l_tile") or
                        k.startswith("rho_total_sum") or k.startswith("rho_w_shape") or
                        (k.startswith("fc_") and any(s in k for s in ("tile", "collect", "norm_out_factor")))):
                    out[f"{name}/{k}"] = z[k]
            out[f"{name}/lmax"] = z["lmax"]
    np.savez_compressed(os.path.join(cases.GOLDEN, "structure_ref.npz"), **out)


if __name__ == "__main__" and os.path.isdir("/root/reference/tests/fixtures"):
    structure_golden()
