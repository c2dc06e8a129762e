"""Host side of libgrace_hip.so without a GPU: the library loads and exports exactly the symbols the header declares,
the model loader accepts the reference's fixture files and rejects malformed ones the way the reference loader does
(libgrace/src/model_1l.cpp, tests/test_model_shapes.cpp of the reference), and the neighbour list equals the reference
list (tests/golden/reference_outputs.npz, written by the compiled reference) and a brute-force O(N^2) search."""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest

import cases
from grace_runtime_amd import _lib, kk, synth


def test_header_symbols_are_exported():
    hdr = open(os.path.join(os.path.dirname(cases.HERE), "include", "grace_hip.h")).read()
    declared = set(re.findall(r"\b(gr_[a-z_0-9]+)\s*\(", hdr))
    assert declared == set(_lib.SYMBOLS)
    L = _lib.lib()
    for s in declared:
        assert getattr(L, s) is not None
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True).stdout
    exported = set(re.findall(r"\bT (gr_[a-z_0-9]+)", out))
    assert declared <= exported
    assert L.gr_abi_version() == 7 == kk.ABI


def test_cxx_adapter_header_compiles_and_links(tmp_path):
    """include/grace_hip_lammps.hpp: the RunInput / RunOutput / Exchange shape of the reference's GPU engines over the C ABI;
    a translation unit that uses every member compiles without warnings as C++17 and links against the library (no GPU call)"""
    root = os.path.dirname(cases.HERE)
    src = tmp_path / "use.cpp"
    src.write_text("""
#include "grace_hip_lammps.hpp"
struct Comm : grace_hip::Exchange { int f = 0, r = 0; void forward(int) override { f++; } void reverse(int) override { r++; } };
int main() {
  grace_hip::Engine eng;
  Comm comm;
  eng.set_exchange(&comm);
  grace_hip::RunInput in;
  grace_hip::RunOutput out;
  (void) in; (void) out;
  try { eng.setup(); return 3; } catch (const std::runtime_error &) {}
  try { eng.set_model("/nonexistent/kokkos.npz", {-1, 0}); return 4; } catch (const std::exception &) {}
  return eng.comm_layers() + eng.comm_width(1) + eng.auto_chunk_size() + (eng.cutoff(1, 1) != 0.0);
}
""")
    exe = tmp_path / "use"
    lib = os.path.dirname(_lib.LIB_PATH)
    res = subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-I" + os.path.join(root, "include"), str(src), "-o", str(exe),
                          "-L" + lib, "-lgrace_hip", "-Wl,-rpath," + lib], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    assert subprocess.run([str(exe)]).returncode == 0


def test_product_does_not_touch_the_oracle():
    root = os.path.dirname(cases.HERE)
    for dp, _, files in os.walk(os.path.join(root, "grace_runtime_amd")):
        for f in files:
            if f.endswith((".py", ".hpp", ".cpp", ".hip", ".h")):
                txt = open(os.path.join(dp, f)).read()
                assert "import oracle" not in txt and "from oracle" not in txt and "oracle/" not in txt, f


@pytest.mark.parametrize("name,lmax,C_,order", [("grace_1l_order3", 2, 16, 3), ("legacy_1l_order3", 2, 16, 3)])
def test_loads_reference_fixture_models(name, lmax, C_, order):
    m = kk.Model(os.path.join(cases.REF_FIXTURES, name + ".npz"))
    assert (m.layers, m.lmax, m.n_radial, m.max_order, m.element_names) == (1, lmax, C_, order, ["Mo", "W"])
    assert m.rcut == 5.0
    with pytest.raises(ValueError):
        m.type2mu(["W", "Xx"])
    assert list(m.type2mu(["W", "Mo"])) == [-1, 1, 0]


@pytest.mark.parametrize("name,lmax,C_,order", [("grace_2l_order3", 2, 16, 3), ("legacy_2l_order3", 2, 16, 3), ("grace_2l_small", 2, 16, 4),
                                                ("grace_2l_l3", 3, 20, 3), ("legacy_2l_wide", 1, 40, 4)])
def test_loads_reference_2l_fixture_models(name, lmax, C_, order):
    m = kk.Model(os.path.join(cases.REF_FIXTURES, name + ".npz"))
    assert (m.layers, m.lmax, m.n_radial, m.max_order, m.element_names) == (2, lmax, C_, order, ["Mo", "W"])
    assert m.rcut == 5.0


def _mutated_2l(tmp_path, fn):
    d = cases.model_l2mix()
    fn(d)
    p = str(tmp_path / "m2.npz")
    np.savez(p, **{k: v for k, v in d.items() if not k.startswith("_")})
    return p


BAD_2L = [
    (lambda d: d.pop("B0_lin_transform_W"), "'B0_lin_transform_W' is absent or empty"),
    (lambda d: d.update(YI_lr_inds=d["YI_lr_inds"] + 7), "'YI_lr_inds' "),
    (lambda d: d.update(I_n_out=np.array([11])), "I_n_out"),
    (lambda d: d.update(B_total_sum_ind_YI=d["B_total_sum_ind_YI"] + 100), "'B_total_sum_ind_YI' [0] = 101 points outside"),
    (lambda d: d.update(I1_is_central_atom_type_dependent=np.array([0])), "I1_is_central_atom_type_dependent"),
    (lambda d: d.update(I_0_LN_scale=d["I_0_LN_scale"][:-1]), "'I_0_LN_scale' holds 8 values, expected 9"),
    (lambda d: d.update(I2_n_out=np.array([7])), "I2_n_out"),
    (lambda d: d.update(prod_BBBB_n_cg_terms=np.array([1])), "prod_AAAA_n_cg_terms"),
    (lambda d: d.update(fc_BB1_w_left=d["fc_BB1_w_left"][:, :-1]), "'fc_BB1_w_left' is stored as 24 x 23 x 9"),
    (lambda d: d.update(mlp_rad_R1_has_chem_emb=np.array([1])), "mlp_rad_R1_has_chem_emb"),
    (lambda d: d.update(I2_reduce_BB_W=d["I2_reduce_BB_W"][:1]), "'I2_reduce_BB_W' is stored as 1 x 9 x 24 x 3"),
]


@pytest.mark.parametrize("k", range(len(BAD_2L)))
def test_malformed_2l_models_are_rejected(tmp_path, k):
    fn, msg = BAD_2L[k]
    with pytest.raises((RuntimeError, ValueError), match=re.escape(msg)):
        kk.Model(_mutated_2l(tmp_path, fn))


def _mutated_3l(tmp_path, fn):
    d = cases.model_l3mix()
    fn(d)
    p = str(tmp_path / "m3.npz")
    np.savez(p, **{k: v for k, v in d.items() if not k.startswith("_")})
    return p


def test_3l_model_loads(tmp_path):
    m = kk.Model(_mutated_3l(tmp_path, lambda d: None))
    assert m.layers == 3 and m.element_names == ["Mo", "W"] and m.rcut == 5.0


def _drop_name(d, key, name):
    d[key] = np.array([x for x in d[key] if x != name.encode()], dtype=d[key].dtype)


BAD_3L = [
    (lambda d: d.pop("A2_cg_W"), "'A2_cg_W' is absent or empty"),
    (lambda d: d.update(A2_cg_W=d["A2_cg_W"][:-1]), "'A2_cg_W' is stored as 80 x 35 where 81 x 35 is needed"),
    (lambda d: d.update(A1_mlp_W0=d["A1_mlp_W0"][:-1]), "A1_mlp_W0"),
    (lambda d: d.update(A1_mlp_b0=d["A1_mlp_b0"][:-1]), "'A1_mlp_b0' holds 31 values, expected 32"),
    (lambda d: d.update(A3_equivariant=np.array([0]), A3_lin_transform_W=d["A1_lin_transform_W"]), "A3_equivariant' is 0, expected 1"),
    (lambda d: d.update(A1_equivariant=np.array([1])), "A1_"),
    (lambda d: _drop_name(d, "prod_names", "A2_3"), "'prod_names' does not list 'A2_3'"),
    (lambda d: d.update(prod_names=np.concatenate([d["prod_names"], np.array([b"A1_2"], dtype=d["prod_names"].dtype)])), "lists 'A1_2' 2 times"),
    (lambda d: _drop_name(d, "reduce_names", "eq1"), "'reduce_names' does not list 'eq1'"),
    (lambda d: d.update(A1_2_left_ind=d["A1_2_left_ind"] + 1000), "'A1_2_left_ind' [0] = 1000 points outside"),
    (lambda d: d.update(A1_2_group_left=d["A1_2_group_left"][:-1]), "'A1_2_left_ind' [22] = 8 points outside the 8 entries"),
    (lambda d: d.update(A2_3_U=d["A2_3_U"][:, :, :-1]), "'A2_3_U' is stored as 6 x 16 x 15"),
    (lambda d: d.update(fc_A1_2a_left_coefs=np.array([1])), "fc_A1_2a_left_coefs"),
    (lambda d: d.update(fc_A1_2a_collect_from=d["fc_A1_2a_collect_from"] + 100), "'fc_A1_2a_collect_from' [0] = 100 points outside the 9 functions of A1"),
    (lambda d: d.update(eq1_instruction_names=d["eq1_instruction_names"][:-1]), "eq1_instruction_names"),
    (lambda d: d.update(eq1_norm_l0_mask=d["eq1_norm_l0_mask"][:-1]), "'eq1_norm_l0_mask' holds 8 values, expected 9"),
    (lambda d: d.update(rho2_norm_scale=d["rho2_norm_scale"][:-1]), "'rho2_norm_scale' holds 7 values, expected 8"),
    (lambda d: d.update(out1_origins=d["out1_origins"][:2], energy_mlp_n_origins=np.array([2])), "out1_origins"),
    (lambda d: d.update(energy_mlp_W0=d["energy_mlp_W0"][:-1]), "energy_mlp_W0"),
    (lambda d: d.update(A2_p=np.array([6])), "'A2_p' = 6 while A1 uses the envelope order 5"),
    (lambda d: d.update(radial_activation=np.array([0])), "'radial_activation' is a switch of the one- and two-layer formats"),
    (lambda d: d.update(A2_n_lm_ind=np.array([5])), "A2_"),
]


@pytest.mark.parametrize("k", range(len(BAD_3L)))
def test_malformed_3l_models_are_rejected(tmp_path, k):
    fn, msg = BAD_3L[k]
    with pytest.raises((RuntimeError, ValueError), match=re.escape(msg)):
        kk.Model(_mutated_3l(tmp_path, fn))


def test_rejects_other_model_kinds_and_missing_files(tmp_path):
    d = cases.model_cut2()
    d["grace_model_kind"] = np.array([b"GRACE-3L"], dtype="|S8")
    p3 = str(tmp_path / "m3.npz")
    np.savez(p3, **d)
    with pytest.raises(RuntimeError, match="n_elements|spbf_names|A1_"):     # a 1L file labelled 3L: no 3L component is found
        kk.Model(p3)
    with pytest.raises(RuntimeError, match="cannot read the model file"):
        kk.Model(str(tmp_path / "nope.npz"))
    p = tmp_path / "junk.npz"
    p.write_bytes(b"not a zip archive at all, just forty-odd bytes of text")
    with pytest.raises(RuntimeError, match="cannot read the model file"):
        kk.Model(str(p))


def _mutated(tmp_path, fn):
    d = cases.model_cut2()
    fn(d)
    p = str(tmp_path / "m.npz")
    np.savez(p, **d)
    return p


BAD = [
    (lambda d: d.pop("chem_embedding"), "'chem_embedding' is absent or empty"),
    (lambda d: d.update(mlp_rad_W1=d["mlp_rad_W1"][:, :-1]), "mlp_rad_W2"),
    (lambda d: d.update(prod_AA_left_ind=d["prod_AA_left_ind"] + 100), "'prod_AA_left_ind' [0] = 100 points outside the 9 entries"),
    (lambda d: d.update(fc_A1_w_tile_left=d["fc_A1_w_tile_left"][:-1]), "'fc_A1_w_tile_left' holds 8 values, expected 9"),
    (lambda d: d.update(rho_reduce_AA_W=d["rho_reduce_AA_W"][:, :, :, :1]), "rho_reduce_AA_W"),
    (lambda d: d.update(A_lin_transform_W=np.asfortranarray(d["A_lin_transform_W"])), "Fortran order"),
    (lambda d: d.update(mlp_rad_W0=np.where(np.arange(d["mlp_rad_W0"].size).reshape(d["mlp_rad_W0"].shape) == 3, np.nan, d["mlp_rad_W0"])), "is not a finite number"),
    (lambda d: d.update(lmax=np.array([300])), "'lmax' = 300 lies outside 0 .. 255"),
    (lambda d: d.update(rcut=np.array([-1.0])), "cutoff"),
    (lambda d: d.update(fc_A1_left_coefs=np.array([0])), "fc_A1_left_coefs"),
    (lambda d: d.update(grace_model_kind=np.array([b"GRACE-9L"], dtype="|S8")), "grace_model_kind"),
    (lambda d: d.update(prod_AAAA_left_ind=np.zeros(1, np.int32)), "the stage is incomplete"),
    (lambda d: d.update(energy_mlp_W1=d["energy_mlp_W1"].astype("U")), "unsupported dtype"),
]


@pytest.mark.parametrize("k", range(len(BAD)))
def test_malformed_models_are_rejected(tmp_path, k):
    fn, msg = BAD[k]
    with pytest.raises((RuntimeError, ValueError), match=re.escape(msg)):
        kk.Model(_mutated(tmp_path, fn))


def test_compressed_archive_is_rejected(tmp_path):
    p = str(tmp_path / "c.npz")
    np.savez_compressed(p, **cases.model_cut2())
    with pytest.raises(RuntimeError, match="compressed"):
        kk.Model(p)


def test_float32_and_integer_arrays_are_read_by_value(tmp_path):
    def fn(d):
        d["rcut"] = np.array([5], dtype=np.int32)                  # integer scalar where a float is expected
        d["chem_embedding"] = d["chem_embedding"].astype(np.float32)
        d["prod_AA_left_ind"] = d["prod_AA_left_ind"].astype(np.int64)
    m = kk.Model(_mutated(tmp_path, fn))
    assert m.rcut == 5.5        # bond_cutoff_map present: its maximum


def _brute(pos, cell, pbc, rc):
    n = len(pos)
    rng = [range(-3, 4) if p else range(0, 1) for p in pbc]
    s = set()
    for a in range(n):
        for b in range(n):
            for s0 in rng[0]:
                for s1 in rng[1]:
                    for s2 in rng[2]:
                        if a == b and (s0, s1, s2) == (0, 0, 0):
                            continue
                        d = pos[b] - pos[a] + s0 * cell[0] + s1 * cell[1] + s2 * cell[2]
                        if d @ d < rc * rc:
                            s.add((a, b, tuple(np.round(d, 9))))
    return s


@pytest.mark.parametrize("struct,rc", [("triclinic", 5.0), ("slab", 6.0), ("molecule", 5.0)])
def test_neighbor_list_matches_brute_force(struct, rc):
    pos, cell, pbc, _ = cases.STRUCTURES[struct]()
    pcell, shift = kk._padded_cell_arrays(cell, pos, rc, pbc)
    perm, offset, j, image, shifts = kk.neighbor_search(pos + shift, pcell, pbc, rc)
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    i = np.repeat(np.arange(len(pos)), np.diff(offset))
    got = {(int(perm[a]), int(perm[b]), tuple(np.round(d, 9))) for a, b, d in zip(i, j, rij)}
    assert len(got) == len(j)
    assert got == _brute(pos, pcell, pbc, rc)


def test_neighbor_list_equals_reference_list(gold):
    keys = sorted({k.split("/")[1] for k in gold if k.startswith("nl/")})
    assert len(keys) >= 5
    for key in keys:
        struct, rc = key.split("@")
        rc = float(rc)
        pos, cell, pbc, _ = cases.STRUCTURES[struct]()
        pcell, shift = kk._padded_cell_arrays(cell, pos, rc, pbc)
        perm, offset, j, image, shifts = kk.neighbor_search(pos + shift, pcell, pbc, rc, num_threads=3)
        for name, got in (("perm", perm), ("offset", offset), ("j", j), ("image", image)):
            assert np.array_equal(got, gold[f"nl/{key}/{name}"]), (key, name)      # bit-exact, order included
        ref = gold[f"nl/{key}/shifts"]
        # the shift vectors S cell: equal up to the reference's own FMA contraction (its build uses -march=native)
        assert shifts.shape == ref.shape and np.abs(shifts - ref).max() <= 4e-16 * max(1.0, np.abs(ref).max())


def test_neighbor_list_thread_count_independent():
    pos, cell, pbc, _ = cases.structure_config1()
    a = kk.neighbor_search(pos, cell, pbc, 6.0, num_threads=1)
    b = kk.neighbor_search(pos, cell, pbc, 6.0, num_threads=8)
    assert all(np.array_equal(x, y) for x, y in zip(a, b))
    assert len(a[2]) == 7424


def test_neighbor_list_argument_errors():
    pos = np.zeros((2, 3))
    with pytest.raises(ValueError, match="cutoff must be positive"):
        kk.neighbor_search(pos, np.eye(3), [1, 1, 1], 0.0)
    with pytest.raises(ValueError, match="full-rank"):
        kk.neighbor_search(pos, np.zeros((3, 3)), [1, 1, 1], 3.0)
    with pytest.raises(ValueError, match="finite"):
        kk.neighbor_search(np.full((2, 3), np.nan), np.eye(3) * 5, [1, 1, 1], 3.0)
    perm, offset, j, image, shifts = kk.neighbor_search(np.zeros((0, 3)), np.eye(3) * 5, [1, 1, 1], 3.0)
    assert offset.tolist() == [0] and j.size == 0
