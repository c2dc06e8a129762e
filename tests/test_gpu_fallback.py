"""The table-driven kernels behind the generated ones.  An engine normally runs the Clebsch-Gordan products of its model
as code generated and compiled when it is created; with GRACE_HIP_JIT=0 (or without a working hiprtc) it keeps the
table-driven kernels: k_prod_fwd / k_prod_bwd for the products of GRACE-1L / 2L, k_couple_fwd_lds / k_couple_bwd_lds
for the cp_l couples of GRACE-3L (the reference's generic path next to its shape-specialised one:
libgrace/include/grace/kk/fused_dense.h:610-645).  Same bars as the other parity tests: the fp64 engine against the
fp64 oracle to 1e-10 eV/atom and 1e-9 eV/A, and against the engine with generated kernels to the same bars.
Needs an MI355X: run with -m gpu."""
import os

import numpy as np
import pytest

import cases
from grace_runtime_amd import kk
from oracle import grace_oracle as g1
from oracle import grace_oracle_2l as g2
from oracle import grace_oracle_3l as g3

pytestmark = pytest.mark.gpu

F64 = {"energy": 1e-10, "forces": 1e-9, "energies": 1e-10, "virial": 1e-9}


def _check(out, ref, n, tol):
    fs = max(1.0, np.abs(ref["forces"]).max())
    assert abs(out["energy"] - ref["energy"]) / n < tol["energy"] * fs
    assert np.abs(out["forces"] - ref["forces"]).max() < tol["forces"] * fs
    assert np.abs(out["energies"] - ref["energies"]).max() < tol["energies"] * fs
    assert np.abs(out["virial"] - ref["virial"]).max() < tol["virial"] * max(1.0, np.abs(ref["virial"]).max())


@pytest.fixture
def no_jit():
    old = os.environ.get("GRACE_HIP_JIT")
    os.environ["GRACE_HIP_JIT"] = "0"
    yield
    if old is None:
        del os.environ["GRACE_HIP_JIT"]
    else:
        os.environ["GRACE_HIP_JIT"] = old


CASES = [("config1", 1, "alloy54"), ("l2mix", 2, "triclinic"), ("l3mix", 3, "slab"), ("config4", 3, None)]


@pytest.mark.parametrize("model,layers,struct", CASES)
def test_table_driven_kernels_match_the_oracle_and_the_generated_kernels(model_dir, no_jit, model, layers, struct):
    path = cases.model_file(model_dir, model)
    if layers == 1:
        om = g1.Model1L(path)
        names, oracle = om.names, g1.compute_1l
    elif layers == 2:
        om = g2.Model2L(path)
        names, oracle = om.names, g2.compute_2l
    else:
        om = g3.Model3L(path)
        names, oracle = [x.decode() for x in om.d["element_names"]], g3.compute_3l
    plain = kk.Engine(kk.Model(path), names, 64)          # created with GRACE_HIP_JIT=0
    os.environ["GRACE_HIP_JIT"] = "1"
    generated = kk.Engine(kk.Model(path), names, 64)
    if struct is None:
        pos, cell, pbc, types = cases.structure_config4(natoms=40, seed=11)
        rc = 6.0
    else:
        pos, cell, pbc, types = cases.STRUCTURES[struct]()
        types = np.minimum(types, len(names)).astype(np.int32)
        rc = plain.cutoff(1, min(2, len(names)))
    pcell, shift = kk._padded_cell_arrays(cell, pos, rc, pbc)
    perm, offset, j, image, shifts = kk.neighbor_search(pos + shift, pcell, pbc, rc)
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    n = len(types)
    out = plain.compute(types[perm], offset, j, rij, energies=True)
    _check(out, oracle(om, types[perm] - 1, offset, j, rij), n, F64)
    _check(out, generated.compute(types[perm], offset, j, rij, energies=True), n, F64)
