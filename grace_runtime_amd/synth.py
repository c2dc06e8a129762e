"""Synthetic GRACE models (kokkos.npz layout, random-init weights) and synthetic periodic structures.

The structure arrays of a kokkos.npz file (FC tiles, Clebsch-Gordan term lists, reduce collect indices) are
normally written by the training code's exporter.  This module regenerates them from first principles so that
benchmark and test models of any lmax can be written without that exporter:

* real Gaunt coefficients by exact quadrature of products of real spherical harmonics (4 pi normalised, index
  lm = l(l+1)+m, Y_1,+1 = sqrt(3) x), normalised so that coupling Y_l1(r) x Y_l2(r) returns exactly Y_LM(r);
* AA functions ordered by L, then by the pair l1 >= l2 (parity-even couplings only), then by M; the symmetric
  terms (m1, m2)/(m2, m1) of a self product l1 == l2 merged into one term with left index >= right index;
* AAA = AA1 x A1 -> L = 0 for l1 >= l2 >= l3; AAAA = AA2 x AA2 -> L = 0 over pairs of AA groups of equal L
  (left group >= right group); for lmax <= 4 the candidates the training code's exporter leaves out (_AAAA_SKIP,
  read off its lmax-4 export) are skipped, for larger lmax a linearly independent set is kept (greedy numerical
  rank test on a single channel, in output order);
* FC: A1 one weight tile per l; AA1/AA2 one tile per (L, l1, l2) group, right input the A function (l = L, m = M);
* rho reduce: collects the invariant (L = 0) functions of each source, one weight tile per collected function.

File layout and key names follow the reference loader, libgrace/src/model_1l.cpp:18-273 (scalars as shape-(1,)
int64/float64 arrays, weights [n_in, n_out] float64 with a separate 1/sqrt(n_in) norm scalar, index arrays int32).
"""
from __future__ import annotations

import math

import numpy as np

__all__ = ["real_sh_np", "coupling_tables", "real_cg", "structure_1l", "structure_2l", "random_model_1l",
           "random_model_2l", "structure_3l", "random_model_3l", "save_model", "bcc_supercell", "fcc_supercell", "jitter"]


# ---------------------------------------------------------------------------------------------------------------
# real spherical harmonics (closed form through associated Legendre functions; used for the quadrature only)
# ---------------------------------------------------------------------------------------------------------------
def _legendre_no_cs(lmax, ct):
    """P_l^m(cos t) without the Condon-Shortley phase, dict[(l, m)], m >= 0."""
    st = np.sqrt(np.maximum(0.0, 1.0 - ct * ct))
    P = {(0, 0): np.ones_like(ct)}
    for m in range(1, lmax + 1):
        P[(m, m)] = P[(m - 1, m - 1)] * (2 * m - 1) * st
    for m in range(0, lmax):
        P[(m + 1, m)] = ct * (2 * m + 1) * P[(m, m)]
    for m in range(0, lmax + 1):
        for l in range(m + 2, lmax + 1):
            P[(l, m)] = ((2 * l - 1) * ct * P[(l - 1, m)] - (l + m - 1) * P[(l - 2, m)]) / (l - m)
    return P


def real_sh_np(u, lmax):
    """Y[n, (lmax+1)^2] of unit vectors u[n, 3]: 4 pi normalised real harmonics, lm = l(l+1)+m,
    Y(l, m>0) ~ cos(m phi), Y(l, m<0) ~ sin(|m| phi), all with positive leading sign (Y_1,1 = sqrt(3) x)."""
    u = np.asarray(u, dtype=np.float64)
    ct = u[:, 2]
    phi = np.arctan2(u[:, 1], u[:, 0])
    P = _legendre_no_cs(lmax, ct)
    Y = np.zeros((u.shape[0], (lmax + 1) ** 2))
    for l in range(lmax + 1):
        c = l * (l + 1)
        Y[:, c] = math.sqrt(2 * l + 1) * P[(l, 0)]
        for m in range(1, l + 1):
            N = math.sqrt(2.0 * (2 * l + 1) * math.factorial(l - m) / math.factorial(l + m))
            Y[:, c + m] = N * P[(l, m)] * np.cos(m * phi)
            Y[:, c - m] = N * P[(l, m)] * np.sin(m * phi)
    return Y


def _sphere_quadrature(deg):
    """nodes u[n, 3] and weights (sum 1) exact for polynomials of degree <= deg on the unit sphere."""
    nt = deg // 2 + 1
    x, w = np.polynomial.legendre.leggauss(nt)
    nphi = deg + 1
    phi = 2.0 * math.pi * np.arange(nphi) / nphi
    ct = np.repeat(x, nphi)
    ww = np.repeat(w, nphi) / (2.0 * nphi)
    ph = np.tile(phi, nt)
    st = np.sqrt(1.0 - ct * ct)
    return np.stack([st * np.cos(ph), st * np.sin(ph), ct], 1), ww


_GAUNT_CACHE = {}


def coupling_tables(lmax):
    """C[(l1, l2, L)] = array [2l1+1, 2l2+1, 2L+1]: the real coupling coefficients with
    sum_{m1 m2} C[m1, m2, M] Y_l1m1(r) Y_l2m2(r) = Y_LM(r) for every unit vector r (l1 + l2 + L even)."""
    if lmax in _GAUNT_CACHE:
        return _GAUNT_CACHE[lmax]
    u, w = _sphere_quadrature(3 * lmax + 2)
    Y = real_sh_np(u, lmax)
    out = {}
    for l1 in range(lmax + 1):
        for l2 in range(lmax + 1):
            for L in range(abs(l1 - l2), min(lmax, l1 + l2) + 1):
                if (l1 + l2 + L) % 2:
                    continue
                a = Y[:, l1 * l1:(l1 + 1) ** 2]
                b = Y[:, l2 * l2:(l2 + 1) ** 2]
                c = Y[:, L * L:(L + 1) ** 2]
                G = np.einsum("n,na,nb,nc->abc", w, a, b, c, optimize=True)
                G[np.abs(G) < 1e-12] = 0.0
                s = (G[:, :, 0] ** 2).sum()
                out[(l1, l2, L)] = G / s
    _GAUNT_CACHE[lmax] = out
    return out


# ---------------------------------------------------------------------------------------------------------------
# structure arrays of a GRACE-1L model
# ---------------------------------------------------------------------------------------------------------------
def _aa_groups(lmax, Lmax):
    groups = []
    for L in range(Lmax + 1):
        for l1 in range(lmax + 1):
            for l2 in range(l1 + 1):
                if abs(l1 - l2) <= L <= l1 + l2 and (l1 + l2 + L) % 2 == 0:
                    groups.append((L, l1, l2))
    return groups


# AAAA candidates (L, (l1, l2), (l3, l4)) absent from exported lmax <= 4 models
_AAAA_SKIP = {(1, (1, 0), (1, 0)), (2, (1, 1), (1, 1)), (2, (2, 0), (1, 1)), (2, (2, 0), (2, 0)), (2, (3, 1), (2, 0)),
              (3, (3, 0), (2, 1)), (3, (4, 1), (2, 1)), (2, (2, 2), (2, 2)), (4, (2, 2), (2, 2)), (4, (4, 0), (2, 2)),
              (4, (4, 2), (2, 2)), (3, (3, 0), (3, 0)), (3, (3, 2), (3, 0)), (3, (4, 1), (3, 0)), (4, (3, 3), (3, 1)),
              (4, (4, 0), (3, 1)), (4, (4, 0), (3, 3)), (4, (4, 0), (4, 0)), (4, (4, 2), (4, 0)), (4, (4, 4), (4, 2))}


def _prod_arrays(terms):
    """terms: list of (out, left, right, coeff) -> sorted int32/float64 arrays."""
    terms = sorted(terms, key=lambda t: t[4] if len(t) > 4 else (t[0], t[1], t[2]))
    o = np.array([t[0] for t in terms], dtype=np.int32)
    l = np.array([t[1] for t in terms], dtype=np.int32)
    r = np.array([t[2] for t in terms], dtype=np.int32)
    c = np.array([t[3] for t in terms], dtype=np.float64)
    return l, r, o, c


def structure_1l(lmax, order4=True, seed_indep=12345):
    """Structure arrays (no weights) of a GRACE-1L model with Lmax = lmax: dict of numpy arrays keyed like the
    kokkos.npz file, plus '_groups' (list of (L, l1, l2) of the AA tiles) for the weight generator."""
    C = coupling_tables(lmax)
    nl = lmax + 1
    nlm = nl * nl
    lm_l = np.repeat(np.arange(nl), 2 * np.arange(nl) + 1).astype(np.int32)
    groups = _aa_groups(lmax, lmax)
    g_first, fn_group, fn_M = [], [], []
    for g, (L, l1, l2) in enumerate(groups):
        g_first.append(len(fn_group))
        for M in range(-L, L + 1):
            fn_group.append(g)
            fn_M.append(M)
    nAA = len(fn_group)
    s = {}
    # ---- AA = A1 x A1
    terms = []
    for g, (L, l1, l2) in enumerate(groups):
        T = C[(l1, l2, L)]
        for M in range(-L, L + 1):
            o = g_first[g] + M + L
            acc = {}
            for m1 in range(-l1, l1 + 1):
                for m2 in range(-l2, l2 + 1):
                    v = T[m1 + l1, m2 + l2, M + L]
                    if v == 0.0:
                        continue
                    a, b = l1 * (l1 + 1) + m1, l2 * (l2 + 1) + m2
                    if l1 == l2 and a < b:      # self product: (m1, m2) and (m2, m1) are the same term
                        a, b = b, a
                    acc[(a, b)] = acc.get((a, b), 0.0) + v
            for (a, b), v in acc.items():
                if abs(v) > 1e-12:    # self products keep the order of the unswapped (smaller, larger) pair
                    terms.append((o, a, b, v, (o, b, a) if l1 == l2 else (o, a, b)))
    l, r, o, c = _prod_arrays(terms)
    s.update(prod_AA_left_ind=l, prod_AA_right_ind=r, prod_AA_m_sum_ind=o, prod_AA_cg_coeff=c,
             prod_AA_n_output_funcs=np.array([nAA], np.int64), prod_AA_n_cg_terms=np.array([c.size], np.int64),
             prod_AA_lmax=np.array([lmax], np.int64), prod_AA_Lmax=np.array([lmax], np.int64))
    # ---- FCs
    s.update(fc_A1_w_tile_left=lm_l.copy(), fc_A1_w_tile_right=lm_l.copy(),
             fc_A1_collect_to=np.arange(nlm, dtype=np.int32), fc_A1_collect_from=np.arange(nlm, dtype=np.int32),
             fc_A1_norm_out_factor=np.full((nlm, 1, 1), 1.0 / math.sqrt(2.0)))
    frm = np.array([groups[g][0] * (groups[g][0] + 1) + M for g, M in zip(fn_group, fn_M)], dtype=np.int32)
    for k in (["AA1", "AA2"] if order4 else ["AA1"]):
        s.update({f"fc_{k}_w_tile_left": np.array(fn_group, np.int32), f"fc_{k}_w_tile_right": np.array(fn_group, np.int32),
                  f"fc_{k}_collect_to": np.arange(nAA, dtype=np.int32), f"fc_{k}_collect_from": frm.copy(),
                  f"fc_{k}_norm_out_factor": np.full((nAA, 1, 1), 1.0 / math.sqrt(2.0))})
    # ---- AAA = AA1 x A1 -> invariants, l1 >= l2 >= l3 = L
    gidx = {g: k for k, g in enumerate(groups)}
    terms, nout = [], 0
    for l1 in range(lmax + 1):
        for l2 in range(l1 + 1):
            for l3 in range(l2 + 1):
                if (l3, l1, l2) not in gidx:
                    continue
                g = gidx[(l3, l1, l2)]
                for M in range(-l3, l3 + 1):
                    terms.append((nout, g_first[g] + M + l3, l3 * (l3 + 1) + M, 1.0 / (2 * l3 + 1)))
                nout += 1
    l, r, o, c = _prod_arrays(terms)
    nAAA = nout
    s.update(prod_AAA_left_ind=l, prod_AAA_right_ind=r, prod_AAA_m_sum_ind=o, prod_AAA_cg_coeff=c,
             prod_AAA_n_output_funcs=np.array([nAAA], np.int64), prod_AAA_n_cg_terms=np.array([c.size], np.int64),
             prod_AAA_lmax=np.array([0], np.int64), prod_AAA_Lmax=np.array([0], np.int64))
    # ---- AAAA = AA2 x AA2 -> invariants: right group ascending in (l3, l4, L), left group >= right group in
    # (l1, l2), equal L; linearly dependent invariants dropped (single-channel numerical rank test)
    nAAAA = 0
    if order4:
        rng = np.random.default_rng(seed_indep)
        nsamp = 400
        Arand = rng.standard_normal((nsamp, nlm))
        AAr = np.zeros((nsamp, nAA))
        pl, pr, po, pc = s["prod_AA_left_ind"], s["prod_AA_right_ind"], s["prod_AA_m_sum_ind"], s["prod_AA_cg_coeff"]
        np.add.at(AAr, (slice(None), po), pc[None, :] * Arand[:, pl] * Arand[:, pr])
        order_r = sorted(range(len(groups)), key=lambda g: (groups[g][1], groups[g][2], groups[g][0]))
        basis = np.zeros((nsamp, 0))
        terms = []
        for gr in order_r:
            L = groups[gr][0]
            for gl in sorted(range(len(groups)), key=lambda g: (groups[g][1], groups[g][2])):
                if groups[gl][0] != L or (groups[gl][1], groups[gl][2]) < (groups[gr][1], groups[gr][2]):
                    continue
                if lmax <= 4:
                    if (L, groups[gl][1:], groups[gr][1:]) in _AAAA_SKIP:
                        continue
                else:
                    v = (AAr[:, g_first[gl]:g_first[gl] + 2 * L + 1] *
                         AAr[:, g_first[gr]:g_first[gr] + 2 * L + 1]).sum(1)
                    v = v / np.linalg.norm(v)
                    trial = np.concatenate([basis, v[:, None]], 1)
                    sv = np.linalg.svd(trial, compute_uv=False)
                    if sv[-1] < 1e-8 * sv[0]:
                        continue
                    basis = trial
                for M in range(-L, L + 1):
                    terms.append((nAAAA, g_first[gl] + M + L, g_first[gr] + M + L, 1.0 / (2 * L + 1)))
                nAAAA += 1
        l, r, o, c = _prod_arrays(terms)
        s.update(prod_AAAA_left_ind=l, prod_AAAA_right_ind=r, prod_AAAA_m_sum_ind=o, prod_AAAA_cg_coeff=c,
                 prod_AAAA_n_output_funcs=np.array([nAAAA], np.int64),
                 prod_AAAA_n_cg_terms=np.array([c.size], np.int64),
                 prod_AAAA_lmax=np.array([0], np.int64), prod_AAAA_Lmax=np.array([0], np.int64))
    # ---- rho reduce: invariants of each source
    nL0 = sum(1 for g in groups if g[0] == 0)

    def red(src, idx):
        idx = np.asarray(idx, dtype=np.int32)
        s[f"rho_collect_ind_{src}"] = idx
        s[f"rho_w_l_tile_{src}"] = np.arange(idx.size, dtype=np.int32)
        s[f"rho_total_sum_ind_{src}"] = np.zeros((idx.size, 1), np.int32)
        s[f"rho_w_shape_{src}"] = np.array([idx.size], np.int64)

    red("A", [0])
    red("AA", np.arange(nL0))
    red("AAA", np.arange(nAAA))
    if order4:
        red("AAAA", np.arange(nAAAA))
    s["_groups"] = groups
    return s


def random_model_1l(*, lmax=4, n_elements=1, element_names=("W",), embedding_size=32, nradbase=8, nradmax=32,
                    fc_width=None, hidden=64, rho_n_out=17, energy_hidden=64, rcut=6.0, radial_basis_p=16,
                    inv_avg_n_neigh=1.0 / 58.0, order4=True, seed=20260101):
    """A GRACE-1L-shaped model with weights W ~ N(0, 1) and norm scalars 1/sqrt(n_in) (i.e. N(0, 1/fan_in)),
    chem_embedding ~ N(0, 1), zero shifts, output_scale 1, SiLU everywhere; returns the dict that `save_model`
    writes as kokkos.npz."""
    rng = np.random.default_rng(seed)
    fc_width = nradmax if fc_width is None else fc_width
    nl = lmax + 1
    s = structure_1l(lmax, order4=order4)
    groups = s.pop("_groups")
    i64 = lambda v: np.array([v], dtype=np.int64)
    f64 = lambda v: np.array([v], dtype=np.float64)
    N = lambda *shape: rng.standard_normal(shape)
    d = {"grace_model_kind": np.array([b"GRACE-1L"], dtype="|S8"), "grace_format_version": i64(1),
         "n_elements": i64(n_elements), "element_names": np.array([n.encode() for n in element_names], dtype="|S2"),
         "embedding_size": i64(embedding_size), "nradbase": i64(nradbase), "rcut": f64(rcut),
         "radial_basis_p": i64(radial_basis_p), "has_bond_specific_cutoff": i64(0), "lmax": i64(lmax),
         "nradmax": i64(nradmax), "mlp_rad_has_chem_emb": i64(0), "chem_embedding": N(n_elements, embedding_size)}
    dims = [nradbase, hidden, hidden, nradmax * nl]
    for i in range(3):
        d[f"mlp_rad_W{i}"] = N(dims[i], dims[i + 1])
        d[f"mlp_rad_norm{i}"] = f64(1.0 / math.sqrt(dims[i]))
    d["mlp_rad_n_layers"] = i64(3)
    d["A_inv_avg_n_neigh"] = np.array(inv_avg_n_neigh)
    d["A_lin_transform_W"] = N(embedding_size, nradmax)
    d["A_lin_transform_norm"] = f64(1.0 / math.sqrt(embedding_size))
    ntile_aa = len(groups)
    for k, n_in_left, ntile in ([("A1", nradmax, nl), ("AA1", fc_width, ntile_aa)] +
                                ([("AA2", fc_width, ntile_aa)] if order4 else [])):
        d[f"fc_{k}_w_left"] = N(fc_width, n_in_left, ntile)
        d[f"fc_{k}_norm_left"] = np.array(1.0 / math.sqrt(n_in_left))
        d[f"fc_{k}_w_right"] = N(fc_width, nradmax, ntile)
        d[f"fc_{k}_norm_right"] = np.array(1.0 / math.sqrt(nradmax))
        d[f"fc_{k}_n_out"] = i64(fc_width)
        d[f"fc_{k}_left_coefs"] = i64(1)
    for src, n_in in [("A", nradmax), ("AA", fc_width), ("AAA", fc_width)] + ([("AAAA", fc_width)] if order4 else []):
        w_shape = int(s[f"rho_w_shape_{src}"][0])
        d[f"rho_reduce_{src}_W"] = N(n_elements, rho_n_out, n_in, w_shape)
        d[f"rho_reduce_{src}_norm"] = np.array(1.0 / math.sqrt(n_in))
        d[f"rho_n_in_{src}"] = i64(n_in)
    d["rho_n_out"] = i64(rho_n_out)
    d["rho_is_central_atom_type_dependent"] = i64(1)
    d["rho_number_of_atom_types"] = i64(n_elements)
    d["rho_instruction_names"] = np.array([b"A", b"AA", b"AAA"] + ([b"AAAA"] if order4 else []), dtype="|S8")
    d["energy_mlp_W0"] = N(rho_n_out - 1, energy_hidden)
    d["energy_mlp_norm0"] = f64(1.0 / math.sqrt(rho_n_out - 1))
    d["energy_mlp_W1"] = N(energy_hidden, 1)
    d["energy_mlp_norm1"] = f64(1.0 / math.sqrt(energy_hidden))
    d["energy_mlp_n_layers"] = i64(2)
    d["energy_mlp_activation"] = i64(0)
    d["shift_values"] = np.zeros(n_elements)
    d.update(s)
    return d


def add_uq_head(d, blocks, *, rp_dim=12, max_clusters=3, seed=20260111):
    """Adds a random uqv6 UQ head to a model dict (the keys libgrace/src/uq_head.cpp:11-76 reads): random projection
    R [d_basis, rp_dim] of the invariant basis (per block, the collected functions of that reduce's sources times their
    channels, libgrace/include/grace/uq.h:31-48), per element 1 .. max_clusters GMM clusters with centroids, symmetric
    positive definite precision matrices and interpolation thresholds over the rp_dim + n_density features, n_density =
    2 for one basis block and 1 + the number of blocks otherwise.  blocks: [(reduce prefix, source names)]."""
    rng = np.random.default_rng(seed)
    i64 = lambda v: np.array([v], dtype=np.int64)
    d_basis = 0
    for pre, names in blocks:
        srcs = [k for k in names if f"{pre}_collect_ind_{k}" in d]
        d_basis += sum(int(np.asarray(d[f"{pre}_n_in_{k}"]).ravel()[0]) * len(d[f"{pre}_collect_ind_{k}"]) for k in srcs)
    nd = 2 if len(blocks) == 1 else 1 + len(blocks)
    E, K, D = int(np.asarray(d["n_elements"]).ravel()[0]), max_clusters, rp_dim + nd
    d["uq_schema_version"] = i64(6)
    d["uq_n_elements"] = i64(E)
    d["uq_max_clusters"] = i64(K)
    d["uq_rp_dim"] = i64(rp_dim)
    d["uq_feature_dim"] = i64(D)
    d["uq_rp_normalize"] = i64(1)
    d["uq_rp_add_density_channel"] = i64(1)
    d["uq_rp_density_scale"] = np.array([1.0])
    d["uq_feature_transform"] = i64(0)
    d["uq_rp_matrix"] = rng.standard_normal((d_basis, rp_dim)) / math.sqrt(rp_dim)
    cen = rng.standard_normal((E, K, D)) * 0.4
    cen[:, :, rp_dim:] = rng.normal(1.0, 1.0, (E, K, nd))
    d["uq_centroids"] = cen
    a = rng.standard_normal((E, K, D, D))
    d["uq_inv_cov"] = a @ np.swapaxes(a, -1, -2) / D + np.eye(D)
    d["uq_n_clusters"] = rng.integers(1, K + 1, size=E).astype(np.int32)
    d["uq_interp_thresholds"] = rng.uniform(0.5, 3.0, (E, K))
    return d


def add_uq_head_1l(d, **kw):
    """GRACE-1L: one basis block, the sources of the rho reduce (libgrace/src/model_1l.cpp:216-271)"""
    return add_uq_head(d, [("rho", ("A", "AA", "AAA", "AAAA"))], **kw)


def add_uq_head_3l(d, **kw):
    """GRACE-3L: one block per layer, the inputs of rho1, rho2, rho3 in their instruction order (libgrace/src/model_3l.cpp:
    453-463); four density channels"""
    names = lambda k: tuple(n.decode() if isinstance(n, bytes) else str(n) for n in np.asarray(d[f"rho{k}_instruction_names"]).ravel())
    return add_uq_head(d, [(f"rho{k}", names(k)) for k in (1, 2, 3)], **kw)


def add_uq_head_2l(d, **kw):
    """GRACE-2L: blocks [I2 over B .. BBBB, rho over A .. AAAA] (libgrace/src/model_2l.cpp:404-478)"""
    return add_uq_head(d, [("I2", ("B", "BB", "BBB", "BBBB")), ("rho", ("A", "AA", "AAA", "AAAA"))], **kw)


# ---------------------------------------------------------------------------------------------------------------
# GRACE-2L: structure arrays and random models
# ---------------------------------------------------------------------------------------------------------------
def _rotation(rng):
    q = rng.standard_normal(4)
    a, b, c, d = q / np.linalg.norm(q)
    return np.array([[a * a + b * b - c * c - d * d, 2 * (b * c - a * d), 2 * (b * d + a * c)],
                     [2 * (b * c + a * d), a * a - b * b + c * c - d * d, 2 * (c * d - a * b)],
                     [2 * (b * d - a * c), 2 * (c * d + a * b), a * a - b * b - c * c + d * d]])


_CG_CACHE = {}


def real_cg(l1, l2, L):
    """Real Clebsch-Gordan tensor T[2l1+1, 2l2+1, 2L+1] of the real harmonics above, for any parity of l1 + l2 + L:
    the one-dimensional space of rotation-invariant tensors, found numerically from the rotation matrices of the
    harmonics.  Even couplings (l1 + l2 + L even) are normalised as coupling_tables (Y x Y -> Y); odd couplings to
    sum_{m1 m2} T[m1, m2, M]^2 = 1 with the sign that makes, at m2 = +l2, the entry of the largest m1 (smallest M)
    positive (the vector product a x b for l1 = l2 = L = 1)."""
    key = (l1, l2, L)
    if key in _CG_CACHE:
        return _CG_CACHE[key]
    if (l1 + l2 + L) % 2 == 0:
        T = coupling_tables(max(l1, l2, L))[key]
        _CG_CACHE[key] = T
        return T
    rng = np.random.default_rng(7)
    u = rng.standard_normal((200, 3))
    u /= np.linalg.norm(u, axis=1)[:, None]
    n1, n2, n3 = 2 * l1 + 1, 2 * l2 + 1, 2 * L + 1

    def wigner(l, R):
        Y = real_sh_np(u, l)[:, l * l:(l + 1) ** 2]
        YR = real_sh_np(u @ R.T, l)[:, l * l:(l + 1) ** 2]
        return np.linalg.lstsq(Y, YR, rcond=None)[0].T

    rows = []
    for _ in range(3):
        R = _rotation(rng)
        K = np.einsum("am,bn,cM->abcmnM", wigner(l1, R), wigner(l2, R), wigner(L, R)).reshape(n1 * n2 * n3, -1)
        rows.append(K - np.eye(n1 * n2 * n3))
    sv, vt = np.linalg.svd(np.concatenate(rows, 0))[1:]
    if not (sv[-1] < 1e-9 and sv[-2] > 1e-6):
        raise ValueError(f"no unique coupling {key}")
    T = vt[-1].reshape(n1, n2, n3)
    T[np.abs(T) < 1e-10] = 0.0
    T /= math.sqrt((T[:, :, 0] ** 2).sum())
    for m1 in range(n1 - 1, -1, -1):
        nz = np.nonzero(T[m1, n2 - 1, :])[0]
        if nz.size:
            if T[m1, n2 - 1, nz[0]] < 0:
                T = -T
            break
    _CG_CACHE[key] = T
    return T


def structure_2l(lmax):
    """Structure arrays of a GRACE-2L model with body order 3 per layer (no AAAA / BBBB stage) and Lmax = lmax in both
    layers.  Irreducible pieces carry (L, parity); lists of functions are ordered by (L, parity) with odd parity
    first, collect lists of the equivariant reduces by (parity, L).

    layer 1: A, A1, AA, AA1 as structure_1l; AAA = AA1 x A -> the invariants of structure_1l followed by the vectors
             (L = 1, odd parity) of the AA groups (l1, l2, L') x A(l3), l3 = L' +- 1, in (l1, l2, L', l3) order, without
             the groups l2 = 0 < l1 and the stretched self couplings L' = 2 l1 (the selection read off the exported
             lmax 2 and lmax 3 models); I1 and I carry (0, +) and (1, -): 4 functions.
    layer 2: YI = every coupling Y_l x I_l' -> L <= lmax, both parities; B0 = the natural-parity functions;
             B = all (L, parity) present; B1 one weight tile per piece; BB = B1 x B1 over the first piece of every L
             (pairs l1 >= l2, every L <= lmax, vanishing antisymmetric self couplings left out);
             BB1 takes its right input from the B piece of equal (L, parity);
             BBB = BB1 x B -> invariants, one per unordered triple (l1, l2, L) and coupling.
    """
    s = structure_1l(lmax, order4=False)
    groups = s["_groups"]
    nl = lmax + 1
    nlm = nl * nl
    g_first = np.cumsum([0] + [2 * g[0] + 1 for g in groups])
    nAA = int(g_first[-1])
    gidx = {(g[1], g[2], g[0]): k for k, g in enumerate(groups)}         # (l1, l2, L) -> group
    # ---- AAA vectors
    l0, r0, o0, c0 = (s[f"prod_AAA_{k}"] for k in ("left_ind", "right_ind", "m_sum_ind", "cg_coeff"))
    nAAA0 = int(s["prod_AAA_n_output_funcs"][0])
    terms = [(int(o), int(l), int(r), float(c)) for o, l, r, c in zip(o0, l0, r0, c0)]
    nout = nAAA0
    for (l1, l2, Lp) in sorted(gidx):
        if (l2 == 0 and l1 > 0) or (l1 == l2 and l1 > 0 and Lp == l1 + l2):
            continue
        g = gidx[(l1, l2, Lp)]
        for l3 in (Lp - 1, Lp + 1):
            if l3 < 0 or l3 > lmax:
                continue
            T = real_cg(Lp, l3, 1)
            for M in range(3):
                for a in range(2 * Lp + 1):
                    for b in range(2 * l3 + 1):
                        if T[a, b, M] != 0.0:
                            terms.append((nout + M, int(g_first[g]) + a, l3 * l3 + b, float(T[a, b, M])))
            nout += 3
    nAAA = nout
    l, r, o, c = _prod_arrays(terms)
    s.update(prod_AAA_left_ind=l, prod_AAA_right_ind=r, prod_AAA_m_sum_ind=o, prod_AAA_cg_coeff=c,
             prod_AAA_n_output_funcs=np.array([nAAA], np.int64), prod_AAA_n_cg_terms=np.array([c.size], np.int64),
             prod_AAA_lmax=np.array([1], np.int64), prod_AAA_Lmax=np.array([1], np.int64))

    def reduce_arrays(pfx, src, conns):
        """conns: list of (collect function, output function, group key); tiles number the groups in order."""
        tiles, t = [], -1
        last = None
        for _, _, key in conns:
            if key != last:
                t += 1
                last = key
            tiles.append(t)
        s[f"{pfx}_collect_ind_{src}"] = np.array([q[0] for q in conns], np.int32)
        s[f"{pfx}_w_l_tile_{src}"] = np.array(tiles, np.int32)
        s[f"{pfx}_total_sum_ind_{src}"] = np.array([q[1] for q in conns], np.int32).reshape(-1, 1)
        s[f"{pfx}_w_shape_{src}"] = np.array([t + 1], np.int64)

    # ---- I1 (0, +), (1, -) from A, AA, AAA; I from I1; rho (invariants) as structure_1l
    reduce_arrays("I1", "A", [(1 + m, 1 + m, "l1") for m in range(3)] + [(0, 0, "l0")])
    vec = [(int(g_first[k]) + m, 1 + m, ("g", k)) for k, g in enumerate(groups) if g[0] == 1 for m in range(3)]
    inv = [(int(g_first[k]), 0, ("g", k)) for k, g in enumerate(groups) if g[0] == 0]
    reduce_arrays("I1", "AA", vec + inv)
    reduce_arrays("I1", "AAA", [(q, 1 + (q - nAAA0) % 3, ("v", (q - nAAA0) // 3)) for q in range(nAAA0, nAAA)] +
                  [(q, 0, ("i", q)) for q in range(nAAA0)])
    reduce_arrays("I", "I1", [(1 + m, 1 + m, "l1") for m in range(3)] + [(0, 0, "l0")])
    # ---- YI: Y_l x I_l'
    I_pieces = [(0, +1, 0), (1, -1, 1)]                                   # (l', parity, first function)
    yi_groups = []                                                        # (L, parity, l, l')
    for l in range(nl):
        for (lp, pp, _) in I_pieces:
            for L in range(abs(l - lp), min(lmax, l + lp) + 1):
                yi_groups.append((L, (-1) ** l * pp, l, lp))
    yi_groups.sort(key=lambda g: (g[0], g[1], g[2], g[3]))
    yi_first = np.cumsum([0] + [2 * g[0] + 1 for g in yi_groups])
    lr, yo, yc = [], [], []
    for k, (L, p, l, lp) in enumerate(yi_groups):
        T = real_cg(l, lp, L)
        i0 = 0 if lp == 0 else 1
        for M in range(2 * L + 1):
            for a in range(2 * l + 1):
                for b in range(2 * lp + 1):
                    if T[a, b, M] != 0.0:
                        lr.append((l * l + a, i0 + b))
                        yo.append(int(yi_first[k]) + M)
                        yc.append(float(T[a, b, M]))
    s.update(YI_lr_inds=np.array(lr, np.int32), YI_m_sum_ind=np.array(yo, np.int32), YI_cg_coeff=np.array(yc),
             YI_n_output_funcs=np.array([int(yi_first[-1])], np.int64), YI_n_cg_terms=np.array([len(yc)], np.int64),
             YI_Lmax=np.array([lmax], np.int64))
    # ---- B pieces (L, parity) and the reduce from YI and B0
    pieces = sorted({(g[0], g[1]) for g in yi_groups} | {(l, (-1) ** l) for l in range(nl)})
    b_first = dict(zip(pieces, np.cumsum([0] + [2 * P[0] + 1 for P in pieces])[:-1]))
    nB = sum(2 * P[0] + 1 for P in pieces)
    order = sorted(range(len(yi_groups)), key=lambda k: (yi_groups[k][1], yi_groups[k][0], k))
    reduce_arrays("B", "YI", [(int(yi_first[k]) + M, int(b_first[yi_groups[k][:2]]) + M, ("g", k))
                              for k in order for M in range(2 * yi_groups[k][0] + 1)])
    lorder = sorted(range(nl), key=lambda l: ((-1) ** l, l))
    reduce_arrays("B", "B0", [(l * l + M, int(b_first[(l, (-1) ** l)]) + M, ("l", l)) for l in lorder
                              for M in range(2 * l + 1)])
    # ---- FC B1: one tile per piece
    tile = np.concatenate([np.full(2 * P[0] + 1, k, np.int32) for k, P in enumerate(pieces)])
    s.update(fc_B1_w_tile_left=tile, fc_B1_w_tile_right=tile.copy(), fc_B1_collect_to=np.arange(nB, dtype=np.int32),
             fc_B1_collect_from=np.arange(nB, dtype=np.int32),
             fc_B1_norm_out_factor=np.full((nB, 1, 1), 1.0 / math.sqrt(2.0)))
    # ---- BB = B1 x B1 over the first piece of every L
    first_piece = {}
    for P in pieces:
        first_piece.setdefault(P[0], P)
    bb_groups = []                                                        # (L, parity, l1, l2)
    for l1 in range(nl):
        for l2 in range(l1 + 1):
            for L in range(l1 - l2, min(lmax, l1 + l2) + 1):
                if l1 == l2 and (l1 + l2 + L) % 2:
                    continue
                p = first_piece[l1][1] * first_piece[l2][1]
                if (L, p) in b_first:
                    bb_groups.append((L, p, l1, l2))
    bb_groups.sort()
    bb_first = np.cumsum([0] + [2 * g[0] + 1 for g in bb_groups])
    nBB = int(bb_first[-1])
    terms = []
    for k, (L, p, l1, l2) in enumerate(bb_groups):
        T = real_cg(l1, l2, L)
        f1, f2 = int(b_first[first_piece[l1]]), int(b_first[first_piece[l2]])
        for M in range(2 * L + 1):
            acc = {}
            for a in range(2 * l1 + 1):
                for b in range(2 * l2 + 1):
                    v = T[a, b, M]
                    if v == 0.0:
                        continue
                    x, y = f1 + a, f2 + b
                    if l1 == l2 and x < y:
                        x, y = y, x
                    acc[(x, y)] = acc.get((x, y), 0.0) + v
            for (x, y), v in acc.items():
                if abs(v) > 1e-12:
                    o = int(bb_first[k]) + M
                    terms.append((o, x, y, v, (o, y, x) if l1 == l2 else (o, x, y)))
    l, r, o, c = _prod_arrays(terms)
    s.update(prod_BB_left_ind=l, prod_BB_right_ind=r, prod_BB_m_sum_ind=o, prod_BB_cg_coeff=c,
             prod_BB_n_output_funcs=np.array([nBB], np.int64), prod_BB_n_cg_terms=np.array([c.size], np.int64),
             prod_BB_lmax=np.array([lmax], np.int64), prod_BB_Lmax=np.array([lmax], np.int64))
    tile = np.concatenate([np.full(2 * g[0] + 1, k, np.int32) for k, g in enumerate(bb_groups)])
    frm = np.concatenate([int(b_first[(g[0], g[1])]) + np.arange(2 * g[0] + 1) for g in bb_groups]).astype(np.int32)
    s.update(fc_BB1_w_tile_left=tile, fc_BB1_w_tile_right=tile.copy(), fc_BB1_collect_to=np.arange(nBB, dtype=np.int32),
             fc_BB1_collect_from=frm, fc_BB1_norm_out_factor=np.full((nBB, 1, 1), 1.0 / math.sqrt(2.0)))
    # ---- BBB = BB1 x B -> invariants: one per unordered triple and coupling parity, even-parity BB groups only
    seen, terms, nBBB = set(), [], 0
    for k in sorted(range(len(bb_groups)), key=lambda k: (bb_groups[k][2], bb_groups[k][3], bb_groups[k][0])):
        L, p, l1, l2 = bb_groups[k]
        if p != 1 or (L, 1) not in b_first:
            continue
        key = (tuple(sorted((l1, l2, L))), (l1 + l2 + L) % 2)
        canonical = (l1 + l2 + L) % 2 == 1 or L <= l2
        if key in seen or not canonical:
            continue
        seen.add(key)
        for M in range(2 * L + 1):
            terms.append((nBBB, int(bb_first[k]) + M, int(b_first[(L, 1)]) + M, 1.0 / (2 * L + 1)))
        nBBB += 1
    l, r, o, c = _prod_arrays(terms)
    s.update(prod_BBB_left_ind=l, prod_BBB_right_ind=r, prod_BBB_m_sum_ind=o, prod_BBB_cg_coeff=c,
             prod_BBB_n_output_funcs=np.array([nBBB], np.int64), prod_BBB_n_cg_terms=np.array([c.size], np.int64),
             prod_BBB_lmax=np.array([0], np.int64), prod_BBB_Lmax=np.array([0], np.int64))
    # ---- I2: invariants of B, BB, BBB
    reduce_arrays("I2", "B", [(0, 0, "b")])
    reduce_arrays("I2", "BB", [(int(bb_first[k]), 0, ("g", k)) for k, g in enumerate(bb_groups) if g[0] == 0])
    reduce_arrays("I2", "BBB", [(q, 0, ("i", q)) for q in range(nBBB)])
    s["_groups"] = groups
    s["_sizes"] = dict(nAA=nAA, nAAA=nAAA, nI=4, nYI=int(yi_first[-1]), nB=nB, nBB=nBB, nBBB=nBBB,
                       nt_AA=len(groups), nt_B=len(pieces), nt_BB=len(bb_groups))
    return s


def random_model_2l(*, lmax=4, n_elements=4, element_names=("Al", "Co", "Ni", "Ti"), embedding_size=32, nradbase=8,
                    c1=32, cr=32, c2=32, i1_width=16, hidden=64, rho_n_out=17, energy_hidden=64, rcut=6.0,
                    radial_basis_p=16, inv_avg_n_neigh=1.0 / 78.0, seed=20260103):
    """A GRACE-2L-shaped model (body order 3 per layer) with weights ~ N(0, 1) and norm scalars 1/sqrt(n_in):
    c1 layer-1 radial / FC channels, cr layer-2 radial channels (= message width), c2 layer-2 FC channels.
    Keys as the reference loader reads them, libgrace/src/model_2l.cpp:28-420."""
    rng = np.random.default_rng(seed)
    nl = lmax + 1
    s = structure_2l(lmax)
    s.pop("_groups")
    z = s.pop("_sizes")
    i64 = lambda v: np.array([v], dtype=np.int64)
    f64 = lambda v: np.array([v], dtype=np.float64)
    N = lambda *shape: rng.standard_normal(shape)
    d = {"grace_model_kind": np.array([b"GRACE-2L"], dtype="|S8"), "grace_format_version": i64(1),
         "n_elements": i64(n_elements), "element_names": np.array([n.encode() for n in element_names], dtype="|S2"),
         "embedding_size": i64(embedding_size), "nradbase": i64(nradbase), "rcut": f64(rcut),
         "radial_basis_p": i64(radial_basis_p), "has_bond_specific_cutoff": i64(0), "lmax": i64(lmax),
         "chem_embedding": N(n_elements, embedding_size)}
    for pfx, c in (("mlp_rad_R", c1), ("mlp_rad_R1", cr)):
        dims = [nradbase, hidden, hidden, c * nl]
        for i in range(3):
            d[f"{pfx}_W{i}"] = N(dims[i], dims[i + 1])
            d[f"{pfx}_norm{i}"] = f64(1.0 / math.sqrt(dims[i]))
        d[f"{pfx}_n_layers"] = i64(3)
        d[f"{pfx}_n_rad_max"] = i64(c)
        d[f"{pfx}_has_chem_emb"] = i64(0)
    for pfx, c in (("A", c1), ("B0", cr)):
        d[f"{pfx}_inv_avg_n_neigh"] = np.array(inv_avg_n_neigh)
        d[f"{pfx}_lin_transform_W"] = N(embedding_size, c)
        d[f"{pfx}_lin_transform_norm"] = f64(1.0 / math.sqrt(embedding_size))
    d["YI_inv_avg_n_neigh"] = np.array(inv_avg_n_neigh)
    d["YI_n_rad_max"] = i64(cr)
    for k, c, ntile in (("A1", c1, nl), ("AA1", c1, z["nt_AA"]), ("B1", c2, z["nt_B"]), ("BB1", c2, z["nt_BB"])):
        d[f"fc_{k}_w_left"] = N(c, c, ntile)
        d[f"fc_{k}_norm_left"] = np.array(1.0 / math.sqrt(c))
        d[f"fc_{k}_w_right"] = N(c, c, ntile)
        d[f"fc_{k}_norm_right"] = np.array(1.0 / math.sqrt(c))
        d[f"fc_{k}_n_out"] = i64(c)
        d[f"fc_{k}_left_coefs"] = i64(1)

    def reduce_w(pfx, srcs, n_out, n_in, elem, nfuncs):
        for src in srcs:
            w_shape = int(s[f"{pfx}_w_shape_{src}"][0])
            d[f"{pfx}_reduce_{src}_W"] = N(n_elements, n_out, n_in[src], w_shape) if elem else N(n_out, n_in[src], w_shape)
            d[f"{pfx}_reduce_{src}_norm"] = np.array(1.0 / math.sqrt(n_in[src]))
            d[f"{pfx}_n_in_{src}"] = i64(n_in[src])
        d[f"{pfx}_n_out"] = i64(n_out)
        d[f"{pfx}_n_funcs"] = i64(nfuncs)
        d[f"{pfx}_is_central_atom_type_dependent"] = i64(1 if elem else 0)
        d[f"{pfx}_instruction_names"] = np.array([x.encode() for x in srcs], dtype="|S8")

    l1 = {"A": c1, "AA": c1, "AAA": c1}
    reduce_w("I1", ["A", "AA", "AAA"], i1_width, l1, True, 4)
    reduce_w("rho", ["A", "AA", "AAA"], rho_n_out, l1, True, 1)
    reduce_w("I", ["I1"], cr, {"I1": i1_width}, False, 4)
    reduce_w("B", ["YI", "B0"], c2, {"YI": cr, "B0": cr}, False, z["nB"])
    reduce_w("I2", ["B", "BB", "BBB"], rho_n_out, {"B": c2, "BB": c2, "BBB": c2}, True, 1)
    d["I_nl_LN_scale"] = 1.0 + 0.1 * N(rho_n_out - 1)
    d["I_nl_LN_type"] = i64(1)
    d["I_nl_LN_n_out"] = i64(rho_n_out)
    d["I_0_LN_scale"] = 1.0 + 0.1 * N(rho_n_out)
    d["I_0_LN_type"] = i64(0)
    d["I_0_LN_n_out"] = i64(rho_n_out)
    d["energy_mlp_W0"] = N(rho_n_out - 1, energy_hidden)
    d["energy_mlp_norm0"] = f64(1.0 / math.sqrt(rho_n_out - 1))
    d["energy_mlp_W1"] = N(energy_hidden, 1)
    d["energy_mlp_norm1"] = f64(1.0 / math.sqrt(energy_hidden))
    d["energy_mlp_n_layers"] = i64(2)
    d["energy_mlp_activation"] = i64(1)
    d["shift_values"] = np.zeros(n_elements)
    d.update(s)
    return d


# ---------------------------------------------------------------------------------------------------------------
# GRACE-3L: structure arrays and random weights
# ---------------------------------------------------------------------------------------------------------------
def _irrep_offsets(irreps):
    return np.concatenate([[0], np.cumsum([2 * l + 1 for l, _ in irreps])]).astype(np.int64)


def _couplings(left, right, out, self_product):
    """Coupling paths (ia, ib, ic) of irreps (l, s) (s = 1: pseudo-tensor): triangle rule, and the product is a
    pseudo-tensor when exactly one of {one factor pseudo, l_a + l_b + l_c odd} holds twice over, i.e.
    s_c = s_a xor s_b xor parity(l_a + l_b + l_c).  A self product keeps ia >= ib."""
    paths = []
    for ia, (la, sa) in enumerate(left):
        for ib, (lb, sb) in enumerate(right):
            if self_product and ib > ia:
                continue
            for ic, (lc, sc) in enumerate(out):
                if abs(la - lb) <= lc <= la + lb and sc == (sa ^ sb ^ ((la + lb + lc) & 1)):
                    paths.append((ia, ib, ic))
    return paths


def _coupled_functions(left, right, out, paths):
    """Functions (path, M) in path order, their CG terms (left fn, right fn, fn, value) and destination (irrep
    function of `out`)."""
    lo, ro, oo = _irrep_offsets(left), _irrep_offsets(right), _irrep_offsets(out)
    terms, fn_path, fn_dst, fn_l = [], [], [], []
    for ip, (ia, ib, ic) in enumerate(paths):
        la, lb, lc = left[ia][0], right[ib][0], out[ic][0]
        T = real_cg(la, lb, lc)
        for M in range(2 * lc + 1):
            f = len(fn_path)
            fn_path.append(ip)
            fn_dst.append(int(oo[ic]) + M)
            fn_l.append(lc)
            for m1, m2 in zip(*np.nonzero(T[:, :, M])):
                terms.append((int(lo[ia]) + int(m1), int(ro[ib]) + int(m2), f, float(T[m1, m2, M])))
    return terms, np.array(fn_path, np.int32), np.array(fn_dst, np.int32), np.array(fn_l, np.int32)


def structure_3l(lmax, lmsg=None, pseudo_message=True, elem_dep=False):
    """Structure arrays (no weights) of a GRACE-3L model, keys as libgrace/src/model_3l.cpp:165-464 reads them.

    Irreps are (l, s), s = 1 for pseudo-tensors.  Per layer K = A1, A2, A3 the lm features X are the natural irreps
    l <= lmax (the scalar SPBF in layer 1, the reduce K_red of the equivariant SPBF in layers 2-3); the product
    reduces K_2_red, K_3_red, K_4_red carry the natural irreps l <= lmax and, in layer 2 when `pseudo_message`, the
    pseudo irreps too; the message eq1 holds the natural irreps l <= lmsg, eq2 those and (pseudo_message) their
    pseudo partners.  Every coupling the triangle and parity rules allow is one path with its own weight tile.
    `elem_dep`: the eq reduces and the reduces of the equivariant SPBFs carry one weight set per element of the
    central atom (the rho reduces always do).  Returns the arrays and '_sizes'."""
    lmsg = lmax if lmsg is None else lmsg
    nl = lmax + 1
    nlm = nl * nl
    X = [(l, 0) for l in range(nl)]
    nat_msg = [(l, 0) for l in range(lmsg + 1)]
    s, sizes = {}, {}
    i64 = lambda v: np.array([v], dtype=np.int64)
    i32a = lambda v: np.asarray(v, dtype=np.int32)
    lm_l = np.repeat(np.arange(nl), 2 * np.arange(nl) + 1).astype(np.int32)

    def cpl(name, left, right, out, self_product):
        paths = _couplings(left, right, out, self_product)
        terms, fn_path, fn_dst, fn_l = _coupled_functions(left, right, out, paths)
        s[f"{name}_nfunc"] = i64(len(fn_path))
        s[f"{name}_n_groups_left"] = i64(len(left))
        s[f"{name}_n_groups_right"] = i64(len(right))
        s[f"{name}_group_left"] = i32a(np.repeat(np.arange(len(left)), [2 * l + 1 for l, _ in left]))
        s[f"{name}_group_right"] = i32a(np.repeat(np.arange(len(right)), [2 * l + 1 for l, _ in right]))
        s[f"{name}_left_ind"] = i32a([t[0] for t in terms])
        s[f"{name}_right_ind"] = i32a([t[1] for t in terms])
        s[f"{name}_m_sum_ind"] = i32a([t[2] for t in terms])
        s[f"{name}_cg"] = np.array([t[3] for t in terms], dtype=np.float64)
        s[f"{name}_out_l"] = fn_l
        sizes[name] = dict(nfunc=len(fn_path), npaths=len(paths), ngl=len(left), ngr=len(right), nterms=len(terms))
        return paths, fn_path, fn_dst

    def reduce_instr(red, src, collect, tile, dst, w_shape):
        s[f"{red}_collect_ind_{src}"] = i32a(collect)
        s[f"{red}_w_l_tile_{src}"] = i32a(tile)
        s[f"{red}_total_sum_ind_{src}"] = i32a(dst).reshape(-1, 1)
        s[f"{red}_w_shape_{src}"] = i64(max(int(w_shape), 1))

    def product_reduce(red, prod, paths, fn_path, fn_dst, out):
        nfo = int(_irrep_offsets(out)[-1])
        reduce_instr(red, prod, np.arange(len(fn_path)), fn_path, fn_dst, len(paths))
        cnt = np.zeros(nfo)
        np.add.at(cnt, fn_dst, 1.0)
        s[f"{red}_norm_map"] = 1.0 / np.sqrt(np.maximum(cnt, 1.0))
        s[f"{red}_n_funcs"] = i64(nfo)
        s[f"{red}_only_invar"] = i64(0)
        s[f"{red}_is_central_atom_type_dependent"] = i64(0)
        s[f"{red}_instruction_names"] = np.array([prod.encode()], dtype="|S8")
        sizes[red] = dict(nfunc=nfo, w_shape={prod: max(len(paths), 1)})

    def fc(name, left):
        """out[f] = nof[f] (left[f] + W[l] X[lm]) for the natural functions f of `left`; the others pass."""
        lo = _irrep_offsets(left)
        nleft = int(lo[-1])
        frm, to, tile = [], [], []
        for i, (l, sp) in enumerate(left):
            if sp == 0 and l <= lmax:
                for M in range(2 * l + 1):
                    frm.append(l * l + M)
                    to.append(int(lo[i]) + M)
                    tile.append(l)
        nof = np.ones(nleft)
        nof[to] = 1.0 / math.sqrt(2.0)
        s[f"fc_{name}_w_tile_left"] = np.zeros(nleft, np.int32)
        s[f"fc_{name}_w_tile_right"] = i32a(tile)
        s[f"fc_{name}_collect_from"] = i32a(frm)
        s[f"fc_{name}_collect_to"] = i32a(to)
        s[f"fc_{name}_norm_out_factor"] = nof.reshape(-1, 1, 1)
        s[f"fc_{name}_left_coefs"] = i64(0)

    def collect_reduce(red, sources, out, invariant, elem):
        """eq / rho: from each source the functions whose irrep is in `out` (the invariants for rho), one weight tile
        per source irrep."""
        oo = _irrep_offsets(out)
        names = []
        for src, irr in sources:
            so = _irrep_offsets(irr)
            col, tile, dst = [], [], []
            for i, ir in enumerate(irr):
                if ir in out:
                    k = out.index(ir)
                    for M in range(2 * ir[0] + 1):
                        col.append(int(so[i]) + M)
                        tile.append(i)
                        dst.append(0 if invariant else int(oo[k]) + M)
            reduce_instr(red, src, col, tile, dst, len(irr))
            names.append(src)
            sizes.setdefault(red, dict(w_shape={}))["w_shape"][src] = len(irr)
        nfo = int(oo[-1])
        s[f"{red}_n_funcs"] = i64(nfo)
        s[f"{red}_only_invar"] = i64(1 if invariant else 0)
        s[f"{red}_is_central_atom_type_dependent"] = i64(1 if elem else 0)
        s[f"{red}_instruction_names"] = np.array([n.encode() for n in names], dtype="|S8")
        if not invariant:
            s[f"{red}_norm_map"] = np.full(nfo, 0.5)
        sizes[red]["nfunc"] = 1 if invariant else nfo

    message = None
    spbf, prods, reds, fcs, eqn, rmsn = [], [], [], [], [], []
    for k in (1, 2, 3):
        K = f"A{k}"
        spbf.append(K)
        s[f"{K}_equivariant"] = i64(0 if k == 1 else 1)
        s[f"{K}_lmax"] = i64(lmax)
        s[f"{K}_Lmax"] = i64(lmax)
        s[f"{K}_l_tile"] = lm_l.copy()
        Xn = K
        if k > 1:
            ylm = [(l, 0) for l in range(nl)]
            paths = _couplings(ylm, message, X, False)
            terms, fn_path, fn_dst, _ = _coupled_functions(ylm, message, X, paths)
            nlmi = int(_irrep_offsets(message)[-1])
            W = np.zeros((nlm * nlmi, len(fn_path)))
            for a, b, f, v in terms:
                W[a * nlmi + b, f] = v
            s[f"{K}_cg_W"] = W
            s[f"{K}_nfunc"] = i64(len(fn_path))
            s[f"{K}_n_lm_ind"] = i64(nlmi)
            mo = _irrep_offsets(message)
            mask = np.zeros(nlmi)
            mask[int(mo[message.index((0, 0))])] = 1.0
            s[f"{K}_chem_l0_mask"] = mask
            sizes[K] = dict(nfunc=len(fn_path), npaths=len(paths), nlmi=nlmi)
            red = K + "_red"
            reduce_instr(red, K, np.arange(len(fn_path)), fn_path, fn_dst, len(paths))
            cnt = np.zeros(nlm)
            np.add.at(cnt, fn_dst, 1.0)
            s[f"{red}_norm_map"] = 1.0 / np.sqrt(np.maximum(cnt, 1.0))
            s[f"{red}_n_funcs"] = i64(nlm)
            s[f"{red}_only_invar"] = i64(0)
            s[f"{red}_is_central_atom_type_dependent"] = i64(1 if elem_dep else 0)
            s[f"{red}_instruction_names"] = np.array([K.encode()], dtype="|S8")
            sizes[red] = dict(nfunc=nlm, w_shape={K: len(paths)})
            reds.append(red)
            Xn = red
        else:
            sizes[K] = dict(nfunc=nlm)
        T = list(X) + ([(l, 1) for l in range(nl)] if (k == 2 and pseudo_message) else [])
        p2 = cpl(K + "_2", X, X, T, True)
        product_reduce(K + "_2_red", K + "_2", *p2, T)
        fc(K + "_2a", T)
        p3 = cpl(K + "_3", T, X, T, False)
        product_reduce(K + "_3_red", K + "_3", *p3, T)
        fc(K + "_2b", T)
        p4 = cpl(K + "_4", T, T, T, True)
        product_reduce(K + "_4_red", K + "_4", *p4, T)
        prods += [K + "_2", K + "_3", K + "_4"]
        reds += [K + "_2_red", K + "_3_red", K + "_4_red"]
        fcs += [K + "_2a", K + "_2b"]
        sources = [(Xn, X), (K + "_2_red", T), (K + "_3_red", T), (K + "_4_red", T)]
        if k < 3:
            message = list(nat_msg) + ([(l, 1) for l in range(lmsg + 1)] if (k == 2 and pseudo_message) else [])
            collect_reduce(f"eq{k}", sources, message, False, elem_dep)
            reds.append(f"eq{k}")
            mo = _irrep_offsets(message)
            M = int(mo[-1])
            e = f"eq{k}_norm"
            s[f"{e}_expand_index"] = i32a(np.repeat(np.arange(len(message)), [2 * l + 1 for l, _ in message]))
            s[f"{e}_degree_weights"] = np.repeat([1.0 / ((2 * l + 1) * len(message)) for l, _ in message],
                                                 [2 * l + 1 for l, _ in message])
            mask = np.zeros(M)
            mask[int(mo[message.index((0, 0))])] = 1.0
            s[f"{e}_l0_mask"] = mask
            s[f"{e}_eps"] = np.array([1e-8])
            s[f"{e}_center_l0"] = i64(1)
            eqn.append(e)
            sizes[e] = dict(n_groups=len(message), M=M)
        collect_reduce(f"rho{k}", sources, [(0, 0)], True, True)
        reds.append(f"rho{k}")
        rmsn.append(f"rho{k}_norm")
    enc = lambda names: np.array([n.encode() for n in names], dtype="|S12")
    s.update(spbf_names=enc(spbf), prod_names=enc(prods), reduce_names=enc(reds), fc_names=enc(fcs),
             eqnorm_names=enc(eqn), rmsnorm_names=enc(rmsn), out1_origins=enc(rmsn))
    s["_sizes"] = sizes
    return s


def random_model_3l(*, lmax=4, lmsg=None, pseudo_message=True, elem_dep=False, n_elements=8, element_names=None, embedding_size=32,
                    nradbase=8, channels=64, hidden=128, rho_n_out=32, energy_hidden=64, rcut=6.0, p=5,
                    inv_avg_n_neigh=1.0 / 72.0, rms_type=1, seed=20260104):
    """A GRACE-3L-shaped model (three layers: scalar SPBF, then two equivariant SPBFs coupling the normalised
    message of the layer before; cp_l products up to body order 4 per layer) with weights ~ N(0, 1) and norm
    scalars 1/sqrt(n_in).  `channels` = radial channels = cp_l rank of every layer.  Keys as the reference loader
    reads them, libgrace/src/model_3l.cpp:165-464."""
    rng = np.random.default_rng(seed)
    nl = lmax + 1
    s = structure_3l(lmax, lmsg, pseudo_message, elem_dep)
    z = s.pop("_sizes")
    C = channels
    i64 = lambda v: np.array([v], dtype=np.int64)
    f64 = lambda v: np.array([v], dtype=np.float64)
    N = lambda *shape: rng.standard_normal(shape)
    if element_names is None:
        table = ("H He Li Be B C N O F Ne Na Mg Al Si P S Cl Ar K Ca Sc Ti V Cr Mn Fe Co Ni Cu Zn Ga Ge As Se Br Kr Rb Sr "
                 "Y Zr Nb Mo Tc Ru Rh Pd Ag Cd In Sn Sb Te I Xe Cs Ba La Ce Pr Nd Pm Sm Eu Gd Tb Dy Ho Er Tm Yb Lu Hf Ta "
                 "W Re Os Ir Pt Au Hg Tl Pb Bi Ac Th Pa U Np Pu").split()
        element_names = table[:n_elements]
    d = {"grace_model_kind": np.array([b"GRACE-3L"], dtype="|S8"), "grace_format_version": i64(1),
         "n_elements": i64(n_elements), "element_names": np.array([n.encode() for n in element_names], dtype="|S2"),
         "embedding_size": i64(embedding_size), "nradbase": i64(nradbase), "rcut": f64(rcut),
         "has_bond_specific_cutoff": i64(0), "chem_embedding": N(n_elements, embedding_size),
         "shift_values": np.zeros(n_elements), "output_scale": f64(1.0)}
    for k in (1, 2, 3):
        K = f"A{k}"
        d[f"{K}_n_rad_max"] = i64(C)
        d[f"{K}_n_rad_basis"] = i64(nradbase)
        d[f"{K}_p"] = i64(p)
        d[f"{K}_rcut"] = f64(rcut)
        d[f"{K}_inv_avg_n_neigh"] = f64(inv_avg_n_neigh)
        dims = [nradbase + 2 * embedding_size, hidden, hidden, C * nl]
        for i in range(3):
            d[f"{K}_mlp_W{i}"] = N(dims[i], dims[i + 1])
            d[f"{K}_mlp_norm{i}"] = f64(1.0 / math.sqrt(dims[i]))
            if i < 2:
                d[f"{K}_mlp_b{i}"] = N(dims[i + 1])
        d[f"{K}_mlp_n_layers"] = i64(3)
        if k == 1:
            d[f"{K}_lin_transform_W"] = N(embedding_size, C)
            d[f"{K}_lin_transform_norm"] = f64(1.0 / math.sqrt(embedding_size))
        else:
            d[f"{K}_chem_linear_W"] = N(embedding_size, C)
            d[f"{K}_chem_linear_norm"] = f64(1.0 / math.sqrt(embedding_size))
        for q in ("2", "3", "4"):
            P = f"{K}_{q}"
            d[f"{P}_rank"] = i64(C)
            d[f"{P}_n_left"] = i64(C)
            d[f"{P}_n_right"] = i64(C)
            d[f"{P}_U"] = N(z[P]["ngl"], C, C)
            d[f"{P}_V"] = N(z[P]["ngr"], C, C)
            d[f"{P}_norm_u"] = f64(1.0 / math.sqrt(C))
            d[f"{P}_norm_v"] = f64(1.0 / math.sqrt(C))
        for f in ("2a", "2b"):
            d[f"fc_{K}_{f}_n_out"] = i64(C)
            d[f"fc_{K}_{f}_w_right"] = N(C, C, nl)
            d[f"fc_{K}_{f}_norm_right"] = f64(1.0 / math.sqrt(C))
    for red, info in z.items():
        if "w_shape" not in info:
            continue
        elem = bool(int(s[f"{red}_is_central_atom_type_dependent"][0]))
        n_out = rho_n_out if red.startswith("rho") else C
        for src, w_shape in info["w_shape"].items():
            d[f"{red}_reduce_{src}_W"] = N(n_elements, n_out, C, w_shape) if elem else N(n_out, C, w_shape)
            d[f"{red}_reduce_{src}_norm"] = f64(1.0 / math.sqrt(C))
            d[f"{red}_n_in_{src}"] = i64(C)
        d[f"{red}_n_out"] = i64(n_out)
    for k in (1, 2):
        e = f"eq{k}_norm"
        d[f"{e}_affine_weight"] = 1.0 + 0.1 * N(z[e]["n_groups"], C)
    for k in (1, 2, 3):
        r = f"rho{k}_norm"
        d[f"{r}_scale"] = 1.0 + 0.1 * N(rho_n_out - rms_type)
        d[f"{r}_type"] = i64(rms_type)
        d[f"{r}_n_out"] = i64(rho_n_out)
    d["energy_mlp_origin_n_out"] = i64(rho_n_out)
    d["energy_mlp_n_origins"] = i64(3)
    d["energy_mlp_W0"] = N(rho_n_out - 1, energy_hidden)
    d["energy_mlp_norm0"] = f64(1.0 / math.sqrt(rho_n_out - 1))
    d["energy_mlp_W1"] = N(energy_hidden, 1)
    d["energy_mlp_norm1"] = f64(1.0 / math.sqrt(energy_hidden))
    d["energy_mlp_n_layers"] = i64(2)
    d["energy_mlp_activation"] = i64(0)
    d.update(s)
    return d


def save_model(path, d):
    """Uncompressed .npz, as np.savez (the reference loader rejects compressed members)."""
    np.savez(path, **{k: v for k, v in d.items() if not k.startswith("_")})


# ---------------------------------------------------------------------------------------------------------------
# structures
# ---------------------------------------------------------------------------------------------------------------
def _supercell(basis, a, reps):
    reps = (reps, reps, reps) if np.isscalar(reps) else tuple(reps)
    basis = np.asarray(basis, dtype=np.float64)
    g = np.stack(np.meshgrid(np.arange(reps[0]), np.arange(reps[1]), np.arange(reps[2]), indexing="ij"), -1)
    pos = (g.reshape(-1, 1, 3) + basis[None, :, :]).reshape(-1, 3) * a
    cell = np.diag([a * reps[0], a * reps[1], a * reps[2]]).astype(np.float64)
    return pos, cell


def bcc_supercell(a, reps):
    """positions [2 r^3, 3], cell [3, 3] of a cubic bcc supercell."""
    return _supercell([[0, 0, 0], [0.5, 0.5, 0.5]], a, reps)


def fcc_supercell(a, reps):
    return _supercell([[0, 0, 0], [0.5, 0.5, 0], [0.5, 0, 0.5], [0, 0.5, 0.5]], a, reps)


def jitter(pos, sigma, seed):
    return pos + np.random.default_rng(seed).normal(0.0, sigma, pos.shape)
