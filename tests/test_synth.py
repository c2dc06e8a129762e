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


def test_structure_3l_shares_the_couplings_of_the_exported_1l_models(sref):
    """The first cp_l product of a GRACE-3L layer couples X with itself exactly as the AA product of GRACE-1L does: the
    same (l1 >= l2) -> L paths with the same coefficients.  Compared with the reference's lmax-4 export, term by term
    as a set of (left, right, coefficient) triples per (L, l1, l2, M)."""
    s = synth.structure_3l(4, pseudo_message=False)
    li, ri, oi, cg = s["A1_2_left_ind"], s["A1_2_right_ind"], s["A1_2_m_sum_ind"], s["A1_2_cg"]
    assert int(s["A1_2_nfunc"][0]) == int(sref["grace_1l_w48/prod_AA_n_output_funcs"][0]) == 141
    lm_l = np.repeat(np.arange(5), 2 * np.arange(5) + 1)
    out_l = s["A1_2_out_l"]

    def table(l, r, o, c, ol):
        # function o of a path (L, l1, l2) -> its M by counting within the run of equal (L, l1, l2)
        t = {}
        first = {}
        for a, b, f, v in zip(l, r, o, c):
            key = (int(ol[f]), int(lm_l[a]), int(lm_l[b]))
            first.setdefault(key, int(f))
            first[key] = min(first[key], int(f))
        for a, b, f, v in zip(l, r, o, c):
            key = (int(ol[f]), int(lm_l[a]), int(lm_l[b]))
            t.setdefault(key + (int(f) - first[key],), {})
            pair = (int(a), int(b)) if a >= b or lm_l[a] != lm_l[b] else (int(b), int(a))
            t[key + (int(f) - first[key],)][pair] = t[key + (int(f) - first[key],)].get(pair, 0.0) + float(v)
        return t
    rl, rr, ro, rc = (sref[f"grace_1l_w48/prod_AA_{k}"] for k in ("left_ind", "right_ind", "m_sum_ind", "cg_coeff"))
    # l of each AA function of the export: from the L = 0..4 block structure of its FC tiles
    ref_ol = np.zeros(141, int)
    groups = synth._aa_groups(4, 4)
    f = 0
    for (L, l1, l2) in groups:
        ref_ol[f:f + 2 * L + 1] = L
        f += 2 * L + 1
    a, b = table(li, ri, oi, cg, out_l), table(rl, rr, ro, rc, ref_ol)
    assert set(a) == set(b)
    for key in a:
        assert set(a[key]) == set(b[key]), key
        for pair in a[key]:
            assert abs(a[key][pair] - b[key][pair]) < 2e-7, (key, pair)


@pytest.mark.parametrize("lmax,pseudo", [(2, True), (3, False)])
def test_structure_3l_index_ranges(lmax, pseudo):
    s = synth.structure_3l(lmax, pseudo_message=pseudo)
    z = s["_sizes"]
    nlm = (lmax + 1) ** 2
    for k in (1, 2, 3):
        K = f"A{k}"
        for q in ("2", "3", "4"):
            P = f"{K}_{q}"
            assert s[P + "_m_sum_ind"].max() == z[P]["nfunc"] - 1
            assert s[P + "_left_ind"].max() < len(s[P + "_group_left"]) and s[P + "_right_ind"].max() < len(s[P + "_group_right"])
            R = P + "_red"
            assert len(s[f"{R}_collect_ind_{P}"]) == z[P]["nfunc"]
            assert s[f"{R}_w_l_tile_{P}"].max() == z[P]["npaths"] - 1
            assert s[f"{R}_total_sum_ind_{P}"].max() < int(s[R + "_n_funcs"][0])
        if k > 1:
            W = s[K + "_cg_W"]
            assert W.shape == (nlm * int(s[K + "_n_lm_ind"][0]), int(s[K + "_nfunc"][0]))
            assert (np.abs(W).sum(0) > 0).all()              # every coupled function has terms
    assert int(s["A2_n_lm_ind"][0]) == (lmax + 1) ** 2
    assert int(s["A3_n_lm_ind"][0]) == (2 if pseudo else 1) * (lmax + 1) ** 2


def test_random_model_3l_file_layout(tmp_path):
    d = cases.model_l3mix()
    p = str(tmp_path / "m.npz")
    synth.save_model(p, d)
    with np.load(p) as zf:
        assert [x.decode() for x in zf["spbf_names"]] == ["A1", "A2", "A3"]
        assert len(zf["prod_names"]) == 9 and len(zf["fc_names"]) == 6 and len(zf["reduce_names"]) == 16
        assert zf["A1_mlp_W0"].shape == (10 + 2 * 8, 32) and zf["A1_mlp_W2"].shape == (32, 16 * 3)
        assert zf["rho1_reduce_A1_W"].shape[0] == 2 and zf["eq1_reduce_A1_W"].ndim == 3
        assert not any(k.startswith("_") for k in zf.files)
