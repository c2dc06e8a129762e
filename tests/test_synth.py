"""The model generator (grace_runtime_amd/synth.py): structure arrays against the training code's real exports
(tests/golden/structure_ref.npz: index tables of the reference's lmax-2/3/4 fixture models) and against the defining
property of the coupling coefficients.  No GPU."""
import os

import numpy as np
import pytest

import cases
from grace_runtime_amd import synth


@pytest.fixture(scope="module")
def sref():
    with np.load(os.path.join(cases.GOLDEN, "structure_ref.npz")) as z:
        return {k: z[k] for k in z.files}


@pytest.mark.parametrize("name,order4", [("grace_1l_small", True), ("grace_1l_l3", False), ("grace_1l_w48", True)])
def test_structure_equals_exported_models(sref, name, order4):
    lmax = int(sref[name + "/lmax"][0])
    s = synth.structure_1l(lmax, order4=order4)
    checked = 0
    for k, v in s.items():
        if k.startswith("_"):
            continue
        ref = sref[f"{name}/{k}"]
        assert ref.shape == v.shape, k
        if v.dtype.kind == "f":
            assert np.abs(ref - v).max() < 2e-7, k        # the exports hold fp32-rounded coefficients
        else:
            assert np.array_equal(ref, v), k
        checked += 1
    assert checked >= 30
    have = {k.split("/", 1)[1] for k in sref if k.startswith(name + "/")} - {"lmax"}
    assert have <= set(s.keys()), have - set(s.keys())


@pytest.mark.parametrize("lmax", [2, 4, 5])
def test_coupling_returns_harmonics(lmax):
    """sum_{m1 m2} C[m1, m2, M] Y_l1m1(r) Y_l2m2(r) = Y_LM(r)"""
    C = synth.coupling_tables(lmax)
    u = np.random.default_rng(0).standard_normal((7, 3))
    u /= np.linalg.norm(u, axis=1)[:, None]
    Y = synth.real_sh_np(u, lmax)
    for (l1, l2, L), T in C.items():
        got = np.einsum("abc,na,nb->nc", T, Y[:, l1 * l1:(l1 + 1) ** 2], Y[:, l2 * l2:(l2 + 1) ** 2])
        assert np.abs(got - Y[:, L * L:(L + 1) ** 2]).max() < 1e-11, (l1, l2, L)


def test_harmonics_match_oracle():
    from oracle.grace_oracle import real_sh
    u = np.random.default_rng(1).standard_normal((20, 3))
    u /= np.linalg.norm(u, axis=1)[:, None]
    assert np.abs(synth.real_sh_np(u, 6) - real_sh(u, 6)[0]).max() < 1e-12


def test_lmax5_structure_is_consistent():
    s = synth.structure_1l(5, order4=True)
    nAA = int(s["prod_AA_n_output_funcs"][0])
    assert s["prod_AA_m_sum_ind"].max() + 1 == nAA and s["fc_AA1_w_tile_left"].size == nAA
    assert s["prod_AAAA_left_ind"].max() < nAA and s["prod_AAA_right_ind"].max() < 36
    assert int(s["prod_AAAA_n_output_funcs"][0]) == s["rho_collect_ind_AAAA"].size > 0


def test_random_model_file_layout(tmp_path):
    d = cases.model_config1()
    p = str(tmp_path / "m.npz")
    synth.save_model(p, d)
    with np.load(p) as z:
        assert z["mlp_rad_W2"].shape == (64, 160) and z["mlp_rad_W0"].shape == (8, 64)
        assert z["fc_AA1_w_left"].shape == (32, 32, 27) and z["rho_reduce_AAAA_W"].shape == (1, 17, 32, 69)
        assert z["prod_AA_cg_coeff"].size == 623 and int(z["prod_AA_n_output_funcs"][0]) == 141
        assert abs(float(z["mlp_rad_norm0"][0]) - 1 / np.sqrt(8)) < 1e-15


@pytest.mark.parametrize("name", ["grace_2l_order3", "grace_2l_l3"])
def test_structure_2l_equals_exported_models(name):
    """every index table and coupling coefficient (the odd-parity couplings of YI and BB with their signs included) of
    the reference's max_order-3 GRACE-2L fixture models, lmax 2 and 3"""
    with np.load(os.path.join(cases.REF_FIXTURES, name + ".npz")) as z:
        ref = {k: z[k] for k in z.files}
    s = synth.structure_2l(int(ref["lmax"][0]))
    checked = 0
    for k, v in s.items():
        if k.startswith("_"):
            continue
        assert ref[k].shape == v.shape, k
        if v.dtype.kind == "f":
            assert np.abs(ref[k] - v).max() < 2e-7, k
        else:
            assert np.array_equal(ref[k], v), k
        checked += 1
    assert checked >= 90
    # nothing structural in the file that the generator leaves out
    structural = [k for k in ref if any(t in k for t in ("_ind", "_tile", "collect", "cg_coeff", "lr_inds", "n_cg_terms",
                                                         "n_output_funcs", "w_shape"))
                  and not k.startswith(("I_out_", "rho_LN", "I_1_LN")) and "indicator" not in k]
    assert set(structural) <= set(s.keys()), set(structural) - set(s.keys())


def test_odd_couplings_are_rotation_invariant_tensors():
    """real_cg(l1, l2, L) with l1 + l2 + L odd: unit norm per M and the vector product for l = 1"""
    T = synth.real_cg(1, 1, 1)
    a, b = np.random.default_rng(3).standard_normal((2, 3))
    yzx = [1, 2, 0]                                   # harmonics order m = -1, 0, 1  <->  y, z, x
    got = np.einsum("abc,a,b->c", T, a[yzx], b[yzx])
    assert np.abs(got - np.cross(a, b)[yzx] / np.sqrt(2.0)).max() < 1e-12
    for key in [(2, 1, 2), (3, 2, 2), (4, 1, 4), (3, 1, 3)]:
        T = synth.real_cg(*key)
        assert np.abs((T ** 2).sum((0, 1)) - 1.0).max() < 1e-10, key


def test_random_model_2l_file_layout(tmp_path):
    d = cases.model_config3()
    p = str(tmp_path / "m2.npz")
    synth.save_model(p, d)
    with np.load(p) as z:
        assert z["mlp_rad_R_W2"].shape == (64, 160) and z["mlp_rad_R1_W2"].shape == (64, 160)
        assert int(z["prod_AA_n_cg_terms"][0]) == 623 and int(z["YI_n_output_funcs"][0]) == 89
        assert int(z["B_n_funcs"][0]) == 49 and int(z["prod_BB_n_output_funcs"][0]) == 197
        assert z["B_reduce_YI_W"].shape[:2] == (32, 32) and z["I_reduce_I1_W"].shape == (32, 16, 2)
        assert "prod_AAAA_n_cg_terms" not in z.files and "prod_BBBB_n_cg_terms" not in z.files
