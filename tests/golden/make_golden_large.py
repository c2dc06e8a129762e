"""Writes tests/golden/reference_large.npz: outputs of the COMPILED REFERENCE (oracle/_ref) on the benchmark
configurations at FULL size, reduced to what a small fixture can hold:

* configurations 2, 3, 4 (8192 / 32 000 / 10 000 atoms): SHA-256 digests of the reference's neighbour list (perm, offset,
  j, image) and its shift table, the bond count; energy, virial; forces and per-atom energies of every `STRIDE`-th atom
  (caller's atom order); the sums of all forces and of all per-atom energies
* configuration 5 (512 cells of 32 .. 128 atoms): energy and virial of EVERY cell, bond count of every cell, forces of
  the cells in `forces_cells`; and for the cells in `oracle_cells` the fp64 outputs of oracle/grace_oracle_2l.py (the
  reference computes in fp32 with spline tables, so a 1e-10 comparison needs the fp64 restatement)

Run in the build container (needs oracle/_ref):  python tests/golden/make_golden_large.py
"""
import hashlib
import os
import sys
import tempfile

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from grace_runtime_amd import workloads  # noqa: E402
from oracle import grace_oracle_2l as g2  # noqa: E402
from oracle import ref_lib  # noqa: E402

STRIDE = {"config2": 32, "config3": 125, "config4": 40}
NTH = len(os.sched_getaffinity(0))


def digest(a):
    return np.frombuffer(hashlib.sha256(np.ascontiguousarray(a).tobytes()).digest(), dtype=np.uint8).copy()


def large_config(name, out, tmp):
    if name == "config2":
        pos, cell, pbc, types = workloads.structure_config2()
        path, t2mu = workloads.write_model("config1", tmp), [0]
    elif name == "config3":
        pos, cell, pbc, types = workloads.structure_config3()
        path, t2mu = workloads.write_model("config3", tmp), [0, 1, 2, 3]
    else:
        pos, cell, pbc, t89 = workloads.structure_config4()
        path = workloads.write_model("config4", tmp)
        types, t2mu = workloads.config4_types(t89), [t - 1 for t in workloads.CONFIG4_SPECIES]
    nl = ref_lib.neighbor_search(pos, cell, pbc, 6.0, NTH)
    perm = nl["perm"]
    ref = ref_lib.RefModel(path, t2mu)
    r = ref.compute(types[perm], nl["offset"], nl["j"], positions=pos[perm], image=nl["image"], shifts=nl["shifts"], nthreads=NTH)
    n = len(pos)
    f = np.zeros((n, 3))
    f[perm] = r["forces"]
    e = np.zeros(n)
    e[perm] = r["energies"]
    idx = np.arange(0, n, STRIDE[name])
    for k in ("perm", "offset", "j", "image"):
        out[f"{name}/nl_sha256_{k}"] = digest(nl[k])
    out[f"{name}/nl_shifts"] = nl["shifts"]
    out[f"{name}/nbonds"] = np.array(len(nl["j"]), np.int64)
    out[f"{name}/energy"] = np.array(r["energy"])
    out[f"{name}/virial"] = r["virial"]
    out[f"{name}/atoms"] = idx
    out[f"{name}/forces"] = f[idx]
    out[f"{name}/energies"] = e[idx]
    out[f"{name}/max_abs_force"] = np.array(np.abs(f).max())
    print(name, n, "atoms", len(nl["j"]), "list bonds, E", r["energy"], "max|F|", np.abs(f).max())


def config5(out, tmp, forces_cells=16, oracle_cells=4):
    structs = workloads.structures_config5()
    path = workloads.write_model("config5", tmp)
    ref = ref_lib.RefModel(path, [0, 1, 2])
    S = len(structs)
    energy, virial, nbonds = np.zeros(S), np.zeros((S, 6)), np.zeros(S, np.int64)
    sizes = np.array([len(s[0]) for s in structs])
    fcells = np.linspace(0, S - 1, forces_cells).astype(np.int64)
    ocells = np.argsort(sizes, kind="stable")[:oracle_cells].astype(np.int64)
    model = g2.Model2L(path)
    pbc = np.array([True, True, True])
    for k, (pos, cell, types) in enumerate(structs):
        nl = ref_lib.neighbor_search(pos, cell, pbc, 6.0, 2)
        perm = nl["perm"]
        r = ref.compute(types[perm], nl["offset"], nl["j"], positions=pos[perm], image=nl["image"], shifts=nl["shifts"], nthreads=NTH)
        energy[k], virial[k], nbonds[k] = r["energy"], r["virial"], len(nl["j"])
        if k in fcells:
            f = np.zeros((len(pos), 3))
            f[perm] = r["forces"]
            out[f"config5/forces_{k}"] = f
        if k in ocells:
            x = pos[perm]
            rij = x[nl["j"]] - np.repeat(x, np.diff(nl["offset"]), axis=0) + nl["shifts"][nl["image"]]
            o = g2.compute_2l(model, types[perm] - 1, nl["offset"], nl["j"], rij)
            f = np.zeros((len(pos), 3))
            f[perm] = o["forces"]
            out[f"config5/oracle_energy_{k}"] = np.array(o["energy"])
            out[f"config5/oracle_forces_{k}"] = f
            out[f"config5/oracle_virial_{k}"] = o["virial"]
            print("config5 cell", k, len(pos), "atoms: oracle E", o["energy"], "reference E", r["energy"])
    out["config5/energy"], out["config5/virial"], out["config5/nbonds"] = energy, virial, nbonds
    out["config5/natoms"] = sizes.astype(np.int32)
    out["config5/forces_cells"], out["config5/oracle_cells"] = fcells, ocells
    print("config5", S, "cells", sizes.sum(), "atoms", nbonds.sum(), "list bonds, sum E", energy.sum())


def main():
    out = {}
    tmp = tempfile.mkdtemp()
    for name in ("config2", "config3", "config4"):
        large_config(name, out, tmp)
    config5(out, tmp)
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "reference_large.npz"), **out)


if __name__ == "__main__":
    main()
