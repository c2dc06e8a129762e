"""The UQ head (uqv6, gamma only) of GRACE-1L, GRACE-2L and GRACE-3L: the CPU oracle against the compiled reference and against what the
definition fixes, and the loader's checks (no GPU needed).

No fixture of the reference carries a UQ head, so the head is a generated one (tests/cases.py model_uq2, and model_uq2l: the
reference's fixture model grace_2l_small with a generated head of two basis blocks, model_uq3l: three blocks).  The compiled
reference projects the basis in fp32 (libgrace/include/grace/fused_cpu.h:1275-1283: gamma within ~1e-5 of an fp64
projection): 1e-4 relative on gamma and sigma, the cluster index exactly."""
import os

import numpy as np
import pytest

import cases
from grace_runtime_amd import kk
from oracle import grace_oracle as go
from oracle import grace_oracle_2l as go2
from oracle import grace_oracle_3l as go3
from oracle import ref_lib


def _bonds(struct, rc=5.0):
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, rc)
    x, t = pos[perm], types[perm]
    rij = x[j] - np.repeat(x, np.diff(offset), axis=0) + shifts[image]
    return t, offset, j, rij


def _oracle(path, t, offset, j, rij, **kw):
    """the oracle of the model's kind (GRACE-1L, 2L or 3L) with the UQ head evaluated"""
    if cases.LAYERS[os.path.basename(path)[:-4]] == 3:
        return go3.compute_3l(go3.Model3L(path), t - 1, offset, j, rij, want_forces=False, uq=True, **kw), go3.Model3L(path)
    if cases.LAYERS[os.path.basename(path)[:-4]] == 2:
        return go2.compute_2l(go2.Model2L(path), t - 1, offset, j, rij, want_forces=False, uq=True, **kw), go2.Model2L(path)
    return go.compute_1l(go.Model1L(path), t - 1, offset, j, rij, want_forces=False, uq=True, **kw), go.Model1L(path)


@pytest.fixture(scope="module")
def uq_model(model_dir):
    return cases.model_file(model_dir, "uq2")


@pytest.mark.skipif(not ref_lib.available(), reason="compiled reference not built")
@pytest.mark.parametrize("model,struct", cases.UQ_CASES)
def test_oracle_matches_compiled_reference(model_dir, model, struct):
    path = cases.model_file(model_dir, model)
    t, offset, j, rij = _bonds(struct)
    o, m = _oracle(path, t, offset, j, rij)
    r = ref_lib.RefModel(path, [0, 1]).compute_uq(t, offset, j, rij)
    assert np.array_equal(o["gmm_cluster"], r["gmm_cluster"])
    if struct == "alloy54":                                           # every cluster of the head is some atom's nearest
        assert [len(np.unique(o["gmm_cluster"][t == e + 1])) for e in range(2)] == list(m.uq_ncl)
    assert np.abs(o["gamma"] / r["gamma"] - 1).max() < 1e-4
    assert np.abs(o["atomic_sigma"] / r["atomic_sigma"] - 1).max() < 1e-4


@pytest.mark.parametrize("model,struct", cases.UQ_CASES)
def test_oracle_matches_golden_of_the_compiled_reference(model_dir, gold, model, struct):
    """the committed outputs of the compiled reference (tests/golden/make_golden.py), for machines without it"""
    t, offset, j, rij = _bonds(struct)
    o, _ = _oracle(cases.model_file(model_dir, model), t, offset, j, rij)
    tag = f"uq/{model}/{struct}"
    assert np.array_equal(o["gmm_cluster"], gold[tag + "/gmm_cluster"])
    assert np.abs(o["gamma"] / gold[tag + "/gamma"] - 1).max() < 1e-4
    assert np.abs(o["atomic_sigma"] / gold[tag + "/atomic_sigma"] - 1).max() < 1e-4


@pytest.mark.parametrize("name", ["uq2", "uq2l", "uq3l"])
def test_what_the_definition_fixes(model_dir, name):
    """the atom whose feature vector IS a centroid has sigma = sqrt(1e-8) and gamma = sigma / threshold; the features are
    invariants of the neighbourhood: a rotated structure gives the same gamma; gamma = sigma / threshold everywhere"""
    path = cases.model_file(model_dir, name)
    t, offset, j, rij = _bonds("alloy54")
    o, m = _oracle(path, t, offset, j, rij)
    thr = m.uq_thr[t - 1, o["gmm_cluster"].astype(int)]
    assert np.abs(o["gamma"] * thr - o["atomic_sigma"]).max() < 1e-12
    assert abs(o["atomic_sigma"].min() - 1e-4) < 1e-9 and (o["atomic_sigma"] < 2e-4).sum() == 1
    # brute force over all clusters of the element: the chosen one is the nearest in the Euclidean sense
    f = o["uq_features"]
    for a in range(len(t)):
        e = t[a] - 1
        d2 = [((f[a] - m.uq_cen[e, k]) ** 2).sum() for k in range(m.uq_ncl[e])]
        assert int(o["gmm_cluster"][a]) == int(np.argmin(d2))
        dl = f[a] - m.uq_cen[e, int(np.argmin(d2))]
        assert abs(o["atomic_sigma"][a] ** 2 - (sum(dl[p] * m.uq_icov[e, int(np.argmin(d2)), p, q] * dl[q] for p in range(len(dl))
                                                   for q in range(len(dl))) + 1e-8)) < 1e-10
    assert np.abs(np.linalg.norm(f[:, :m.uq_rp], axis=1)).max() < np.linalg.norm(m.uq_R, 2) + 1e-9     # |B R| / |B| <= |R|
    if name == "uq2":
        assert np.abs(f[:, m.uq_rp] - f[:, m.uq_rp + 1]).max() == 0.0                                 # one basis block: equal channels
    else:                       # two / three blocks: |B|^2 = the sum of the blocks' |B_b|^2 (the 1e-12 inside the logs: 1e-9)
        s, nb = m.uq_scale, cases.LAYERS[name]
        assert m.uq_D == m.uq_rp + 1 + nb
        n2 = np.exp(2 * f[:, m.uq_rp:] / s)
        assert np.abs(n2[:, 0] - n2[:, 1:].sum(1)).max() < 1e-9 * n2[:, 0].max()
    rot = np.linalg.qr(np.random.default_rng(4).standard_normal((3, 3)))[0]
    o2, _ = _oracle(path, t, offset, j, rij @ rot.T)
    assert np.abs(o2["gamma"] - o["gamma"]).max() < 1e-9 * o["gamma"].max()


def _mutated(tmp_path, edit, name="uq2"):
    d = cases.MODELS[name]()
    edit(d)
    p = str(tmp_path / "m.npz")
    np.savez(p, **{k: v for k, v in d.items() if not k.startswith("_")})
    return p


BAD_UQ = [
    (lambda d: d.update(uq_schema_version=np.array([5])), "UQ head of schema 5; only schema 6"),
    (lambda d: d.update(uq_rp_matrix=d["uq_rp_matrix"][:-1]), "basis functions, the model has"),
    (lambda d: d.update(uq_rp_matrix=np.ascontiguousarray(d["uq_rp_matrix"].T)), "uq_rp_matrix"),
    (lambda d: d.update(uq_n_clusters=np.array([3, 0], np.int32)), "element 1 has no GMM cluster"),
    (lambda d: d.update(uq_n_clusters=np.array([3, 4], np.int32)), "uq_n_clusters\' \\[1\\] = 4 points outside"),
    (lambda d: d.update(uq_centroids=d["uq_centroids"][:, :2]), "uq_centroids"),
    (lambda d: d.update(uq_inv_cov=d["uq_inv_cov"][:, :, :, :-1]), "uq_inv_cov"),
    (lambda d: d.update(uq_rp_normalize=np.array([0])), "uq_rp_normalize = 0"),
    (lambda d: d.update(uq_feature_dim=np.array([15]), uq_centroids=np.zeros((2, 3, 15)), uq_inv_cov=np.zeros((2, 3, 15, 15))),
     "3 density channels where 2 belong"),
    (lambda d: d.update(uq_n_elements=np.array([3])), "uq_n_elements"),
    (lambda d: d.pop("uq_interp_thresholds"), "uq_interp_thresholds"),
]


@pytest.mark.parametrize("edit,msg", BAD_UQ)
def test_a_broken_head_is_reported_by_validate_uq_and_leaves_the_model_usable(tmp_path, edit, msg):
    m = kk.Model(_mutated(tmp_path, edit))                     # loads (libgrace/src/model_1l.cpp:216-271)
    assert m.has_uq and m.layers == 1
    with pytest.raises(ValueError, match=msg):
        m.validate_uq()


def test_heads_that_validate_and_models_without(tmp_path, uq_model, model_dir):
    m = kk.Model(uq_model)
    assert m.has_uq
    m.validate_uq()
    plain = kk.Model(cases.model_file(model_dir, "mix2"))
    assert not plain.has_uq
    with pytest.raises(ValueError, match="no UQ head"):
        plain.validate_uq()
    with pytest.raises(ValueError, match="no UQ head"):
        kk.Model(cases.model_file(model_dir, "l2mix")).validate_uq()
    with pytest.raises(ValueError, match="GRACE-3L: the model has no UQ head"):
        kk.Model(cases.model_file(model_dir, "l3mix")).validate_uq()
    three = kk.Model(cases.model_file(model_dir, "uq3l"))
    assert three.has_uq and three.layers == 3
    three.validate_uq()
    two = kk.Model(cases.model_file(model_dir, "uq2l"))
    assert two.has_uq and two.layers == 2
    two.validate_uq()
    o3 = kk.Model(_mutated(tmp_path, lambda d: synth_uq(d), "cut2"))          # max_order 3: refused (tests/test_driver.cpp:406-415)
    with pytest.raises(ValueError, match="max_order 3"):
        o3.validate_uq()


def synth_uq(d):
    from grace_runtime_amd import synth
    synth.add_uq_head_1l(d, rp_dim=6, max_clusters=2)


BAD_UQ_2L = [
    (lambda d: d.update(uq_rp_matrix=d["uq_rp_matrix"][:-1]), "basis functions, the model has"),
    (lambda d: d.update(uq_feature_dim=np.array([12]), uq_centroids=np.zeros((2, 3, 12)), uq_inv_cov=np.zeros((2, 3, 12, 12))),
     "2 density channels where 3 belong"),
    (lambda d: d.update(uq_schema_version=np.array([4])), "UQ head of schema 4; only schema 6"),
    (lambda d: d.update(uq_n_clusters=np.array([0, 3], np.int32)), "element 0 has no GMM cluster"),
]


@pytest.mark.parametrize("edit,msg", BAD_UQ_2L)
def test_a_broken_head_on_a_2l_model(tmp_path, edit, msg):
    m = kk.Model(_mutated(tmp_path, edit, "uq2l"))                     # loads (libgrace/src/model_2l.cpp:404-478)
    assert m.has_uq and m.layers == 2
    with pytest.raises(ValueError, match=msg):
        m.validate_uq()


def test_max_order_3_2l_model_with_a_head_is_refused(tmp_path):
    from grace_runtime_amd import synth
    m = kk.Model(_mutated(tmp_path, lambda d: synth.add_uq_head_2l(d, rp_dim=6, max_clusters=2), "l2mix"))
    assert m.has_uq
    with pytest.raises(ValueError, match="max_order 3"):
        m.validate_uq()


BAD_UQ_3L = [
    (lambda d: d.update(uq_rp_matrix=d["uq_rp_matrix"][:-1]), "uq_rp_matrix"),
    (lambda d: d.update(uq_feature_dim=np.array([14]), uq_centroids=np.zeros((2, 3, 14)), uq_inv_cov=np.zeros((2, 3, 14, 14))),
     "5 density channels; the three-layer kernels write at most 4"),
    (lambda d: d.update(uq_schema_version=np.array([3])), "UQ head of schema 3; only schema 6"),
    (lambda d: d.update(uq_n_clusters=np.array([3, 0], np.int32)), "element 1 has no GMM cluster"),
    (lambda d: d.update(uq_rp_normalize=np.array([0])), "uq_rp_normalize = 0"),
]


@pytest.mark.parametrize("edit,msg", BAD_UQ_3L)
def test_a_3l_file_with_a_broken_head_does_not_load(tmp_path, edit, msg):
    """libgrace/src/model_3l.cpp:453-463: the GRACE-3L loader throws where the 1L / 2L loaders keep the model usable"""
    with pytest.raises((ValueError, RuntimeError), match=msg):
        kk.Model(_mutated(tmp_path, edit, "uq3l"))


def test_a_3l_head_with_fewer_density_channels_loads(tmp_path):
    """the reference accepts 1 .. 4 density channels for GRACE-3L and writes the first uq_n_density of (total, rho1, rho2, rho3)"""
    def edit(d):
        D = int(d["uq_rp_dim"][0]) + 2
        d.update(uq_feature_dim=np.array([D]), uq_centroids=np.ascontiguousarray(d["uq_centroids"][:, :, :D]),
                 uq_inv_cov=np.ascontiguousarray(d["uq_inv_cov"][:, :, :D, :D]))
    p = _mutated(tmp_path, edit, "uq3l")
    kk.Model(p).validate_uq()
    t, offset, j, rij = _bonds("triclinic")
    o = go3.compute_3l(go3.Model3L(p), t - 1, offset, j, rij, want_forces=False, uq=True)
    if ref_lib.available():
        r = ref_lib.RefModel(p, [0, 1]).compute_uq(t, offset, j, rij)
        assert np.array_equal(o["gmm_cluster"], r["gmm_cluster"]) and np.abs(o["gamma"] / r["gamma"] - 1).max() < 1e-4
