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
