"""CPU oracle for the GRACE energy + forces + virial hot path (TEST INFRASTRUCTURE, not product code).

This file restates, in plain numpy fp64, the algorithm of the reference CPU drivers.  Only the tests, the smoke
check and the CPU-baseline leg of the benchmark may import it; the shipped library never does.

Every function cites the reference file:line it follows (paths relative to the reference checkout):

* real spherical harmonics and gradient ........ libgrace/include/grace/fused_cpu.h:686-798   (sh_coefs, sh_block)
* Chebyshev x envelope radial basis ............. libgrace/include/grace/radial_x.h:11-26      (radial_basis_x)
* radial MLP, value + tangent ................... libgrace/include/grace/radial_x.h:29-60      (mlp_x)
* bond filter / geometry ........................ libgrace/include/grace/bonds.h:120-162       (BondGather<CsrBonds>)
* species weight z .............................. libgrace/src/fused_1l.cpp:150-162
* A basis ....................................... libgrace/include/grace/fused_cpu.h:947-982   (atom_scatter)
* FC ............................................ libgrace/include/grace/fused_cpu.h:1102-1175 (build_fc), :349-364
* CG product .................................... libgrace/include/grace/fused_cpu.h:1177-1198 (build_prod), :409-475
* reduce ........................................ libgrace/include/grace/fused_cpu.h:1202-1273 (build_red), :637-649
* energy readout ................................ libgrace/src/fused_1l.cpp:378-427            (energy_atom)
* bond force, virial ............................ libgrace/include/grace/fused_cpu.h:1027-1050 (bond_force),
                                                  libgrace/src/fused_1l.cpp:46-51,351-371
* dead AAAA stage of max_order-3 files .......... libgrace/src/max_order3.h:84-134 (here: the stage is skipped)
* UQ head (uqv6: basis, projection, GMM) ........ libgrace/include/grace/fused_cpu.h:1275-1412, src/fused_1l.cpp:594-636

The reference evaluates the network in fp32 with cubic-Hermite tables of the radial MLP; this restatement evaluates
the same formulas directly in fp64 (no tables), which is what the reference's own TensorFlow fp64 goldens
(tests/fixtures/ref_tf/order3_tf.npz) pin to ~1e-7.

Pinning status (see tests/test_oracle_*.py):
* GRACE-1L end to end (radial basis, MLP, SH, A, FC, CG product, reduce, readout, forces, virial): pinned by the
  TF-fp64 goldens of grace_1l_order3 / legacy_1l_order3 on W54, WMo54, W2tri, by finite differences of E, and by the
  compiled reference (oracle/_ref) for the AAAA stage (grace_1l_w48) and the synthetic benchmark models.
* UQ head of GRACE-1L (gamma, sigma, cluster): no fixture of the reference carries a UQ head; pinned by the compiled
  reference on generated heads (its projection runs in fp32: gamma to 1e-4 relative) and by a brute-force restatement
  of the GMM in the test.
* GRACE-2L: see grace_oracle_2l.py.
"""
from __future__ import annotations

import numpy as np

__all__ = ["load_npz", "Model1L", "real_sh", "radial_basis", "mlp_value_tangent", "compute_1l", "virial_to_stress"]


def load_npz(path):
    """kokkos.npz -> dict of numpy arrays (numpy's own reader: independent of the product's C reader)."""
    with np.load(path, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def _scalar(d, key, default=None):
    if key not in d:
        if default is None:
            raise KeyError(key)
        return default
    return d[key].reshape(-1)[0]


# ---------------------------------------------------------------------------------------------------------------
# spherical harmonics: fused_cpu.h:686-798
# ---------------------------------------------------------------------------------------------------------------
def _sh_coefs(lmax):
    """fused_cpu.h:686-704: a, b over (l, m < l-1), c, d over l."""
    a, b, c, d = {}, {}, {}, {}
    for l in range(2, lmax + 1):
        for mm in range(0, l - 1):
            l2, m2, lm1 = float(l * l), float(mm * mm), float(l - 1)
            a[(l, mm)] = np.sqrt((4.0 * l2 - 1.0) / (l2 - m2))
            b[(l, mm)] = -np.sqrt((lm1 * lm1 - m2) / (4.0 * lm1 * lm1 - 1.0))
        c[l] = -np.sqrt(1.0 + 0.5 / l)
        d[l] = np.sqrt(2.0 * l + 1.0)
    return a, b, c, d


def real_sh(u, lmax):
    """Real 4pi-normalised spherical harmonics Y[nb, nlm] (index l(l+1)+m) of unit vectors u[nb, 3] and the gradient
    G[nb, nlm, 3] of their polynomial extension with respect to (x, y, z).  fused_cpu.h:712-798."""
    u = np.asarray(u, dtype=np.float64)
    nb = u.shape[0]
    rx, ry, rz = u[:, 0], u[:, 1], u[:, 2]
    nlm = (lmax + 1) ** 2
    a, b, c, d = _sh_coefs(lmax)
    plm, dplm = {}, {}
    plm[(0, 0)] = np.ones(nb)
    dplm[(0, 0)] = np.zeros(nb)
    if lmax > 0:
        plm[(1, 0)] = np.sqrt(3.0) * rz
        dplm[(1, 0)] = np.full(nb, np.sqrt(3.0))
        plm[(1, 1)] = np.full(nb, -np.sqrt(1.5))
        dplm[(1, 1)] = np.zeros(nb)
        for l in range(2, lmax + 1):
            for mm in range(0, l - 1):
                ca, cb = a[(l, mm)], b[(l, mm)]
                plm[(l, mm)] = ca * (rz * plm[(l - 1, mm)] + cb * plm[(l - 2, mm)])
                dplm[(l, mm)] = ca * (plm[(l - 1, mm)] + rz * dplm[(l - 1, mm)] + cb * dplm[(l - 2, mm)])
            prev, dprev = plm[(l - 1, l - 1)], dplm[(l - 1, l - 1)]
            plm[(l, l - 1)] = d[l] * prev * rz
            plm[(l, l)] = c[l] * prev
            dplm[(l, l - 1)] = d[l] * (dprev * rz + prev)
            dplm[(l, l)] = c[l] * dprev
    Y = np.zeros((nb, nlm))
    G = np.zeros((nb, nlm, 3))
    sq2 = np.sqrt(2.0)
    for l in range(lmax + 1):
        cidx = l * (l + 1)
        Y[:, cidx] = plm[(l, 0)]
        G[:, cidx, 2] = dplm[(l, 0)]
        # (x + i y)^m and its x, y derivatives, by recurrence
        pr, pi = rx.copy(), ry.copy()
        prx, pry = np.ones(nb), np.zeros(nb)
        pix, piy = np.zeros(nb), np.ones(nb)
        for mm in range(1, l + 1):
            sg = sq2 if mm % 2 == 0 else -sq2
            pv, dpv = plm[(l, mm)], dplm[(l, mm)]
            Y[:, cidx + mm] = sg * pr * pv
            Y[:, cidx - mm] = sg * pi * pv
            G[:, cidx + mm, 0] = sg * prx * pv
            G[:, cidx + mm, 1] = sg * pry * pv
            G[:, cidx + mm, 2] = sg * pr * dpv
            G[:, cidx - mm, 0] = sg * pix * pv
            G[:, cidx - mm, 1] = sg * piy * pv
            G[:, cidx - mm, 2] = sg * pi * dpv
            nrx = prx * rx + pr - pix * ry
            nry = pry * rx - piy * ry - pi
            nix = prx * ry + pix * rx + pi
            niy = pry * ry + pr + piy * rx
            prx, pry, pix, piy = nrx, nry, nix, niy
            pr, pi = pr * rx - pi * ry, pr * ry + pi * rx
    return Y, G


# ---------------------------------------------------------------------------------------------------------------
# radial functions: radial_x.h
# ---------------------------------------------------------------------------------------------------------------
def radial_basis(x, p, nrb):
    """g[nb, nrb] = T_k(2x-1) fcut_p(x), k = 1..nrb, and dg/dx.  radial_x.h:11-26."""
    x = np.asarray(x, dtype=np.float64)
    xp = x ** p
    xp1 = xp * x
    xp2 = xp1 * x
    fc = 1.0 - 0.5 * (p + 1) * (p + 2) * xp + p * (p + 2) * xp1 - 0.5 * p * (p + 1) * xp2
    dfc = 0.5 * p * (p + 1) * (p + 2) * (-(x ** (p - 1)) + 2.0 * xp - xp1)
    t = 2.0 * x - 1.0
    Tp, Tc = np.ones_like(x), t.copy()
    dTp, dTc = np.zeros_like(x), np.full_like(x, 2.0)
    g = np.empty(x.shape + (nrb,))
    dg = np.empty_like(g)
    for k in range(nrb):
        g[..., k] = Tc * fc
        dg[..., k] = dTc * fc + Tc * dfc
        Tn = 2.0 * t * Tc - Tp
        dTn = 2.0 * (2.0 * Tc + t * dTc) - dTp
        Tp, dTp, Tc, dTc = Tc, dTc, Tn, dTn
    return g, dg


def mlp_value_tangent(layers, h, dh, act):
    """Radial MLP: s = norm (W^T h); hidden layers SiLU (act 0) or tanh (act 1), linear output; forward-mode
    tangent.  layers = [(W[n_in, n_out], norm)].  radial_x.h:29-60."""
    n = len(layers)
    for il, (W, norm) in enumerate(layers):
        s = (h @ W) * norm
        ds = (dh @ W) * norm
        if il < n - 1:
            if act == 1:
                s = np.tanh(s)
                ds = ds * (1.0 - s * s)
            else:
                sg = 1.0 / (1.0 + np.exp(-s))
                ds = sg * (1.0 + s * (1.0 - sg)) * ds
                s = s * sg
        h, dh = s, ds
    return h, dh


# ---------------------------------------------------------------------------------------------------------------
# model container (what the oracle needs from a GRACE-1L kokkos.npz; src/model_1l.cpp:18-273)
# ---------------------------------------------------------------------------------------------------------------
class _FC:
    def __init__(self, d, pfx):
        self.wl = np.asarray(d[pfx + "_w_left"], dtype=np.float64)      # [n_out, n_in, tiles]
        self.wr = np.asarray(d[pfx + "_w_right"], dtype=np.float64)
        self.tile_l = d[pfx + "_w_tile_left"].astype(np.int64).ravel()
        self.tile_r = d[pfx + "_w_tile_right"].astype(np.int64).ravel()
        self.to = d[pfx + "_collect_to"].astype(np.int64).ravel()
        self.frm = d[pfx + "_collect_from"].astype(np.int64).ravel()
        self.nof = np.asarray(d[pfx + "_norm_out_factor"], dtype=np.float64).ravel()
        self.norm_l = float(_scalar(d, pfx + "_norm_left", 1.0))
        self.norm_r = float(_scalar(d, pfx + "_norm_right", 1.0))
        self.n_out = int(_scalar(d, pfx + "_n_out"))
        # gather matrix right-connection -> output function
        self.nf = self.tile_l.size
        self.S = np.zeros((self.nf, self.to.size))
        self.S[self.to, np.arange(self.to.size)] = 1.0

    def fwd(self, Xl, Xr):
        """out[a,f,k] = nof[f] (norm_l sum_n Wl[k,n,tile_l f] Xl[a,f,n] + norm_r sum_{c->f} sum_n Wr[k,n,tile c]
        Xr[a,from c,n]).  fused_cpu.h:349-356 + build_fc."""
        left = np.einsum("knf,afn->afk", self.wl[:, :, self.tile_l], Xl, optimize=True) * self.norm_l
        rc = np.einsum("knc,acn->ack", self.wr[:, :, self.tile_r], Xr[:, self.frm, :], optimize=True) * self.norm_r
        right = np.einsum("fc,ack->afk", self.S, rc, optimize=True)
        return (left + right) * self.nof[None, :, None]

    def bwd(self, gout, gXl, gXr):
        """adds into gXl, gXr.  fused_cpu.h:358-364."""
        g = gout * self.nof[None, :, None]
        gXl += np.einsum("knf,afk->afn", self.wl[:, :, self.tile_l], g, optimize=True) * self.norm_l
        gc = g[:, self.to, :]                                                        # [a, c, k]
        gr = np.einsum("knc,ack->acn", self.wr[:, :, self.tile_r], gc, optimize=True) * self.norm_r
        np.add.at(gXr, (slice(None), self.frm, slice(None)), gr)


class _Prod:
    def __init__(self, d, pfx):
        self.l = d[pfx + "_left_ind"].astype(np.int64).ravel()
        self.r = d[pfx + "_right_ind"].astype(np.int64).ravel()
        self.o = d[pfx + "_m_sum_ind"].astype(np.int64).ravel()
        self.c = np.asarray(d[pfx + "_cg_coeff"], dtype=np.float64).ravel()
        self.nout = int(_scalar(d, pfx + "_n_output_funcs"))
        self.S = np.zeros((self.nout, self.c.size))
        self.S[self.o, np.arange(self.c.size)] = self.c

    def fwd(self, L, R):
        """out[a,o,k] = sum_t c_t L[a,l_t,k] R[a,r_t,k].  fused_cpu.h:409-427."""
        return np.einsum("ot,atk->aok", self.S, L[:, self.l, :] * R[:, self.r, :], optimize=True)

    def bwd(self, L, R, g, gL, gR):
        """gL[l_t] += c_t g[o_t] R[r_t], gR[r_t] += c_t g[o_t] L[l_t].  fused_cpu.h:429-452."""
        gt = g[:, self.o, :] * self.c[None, :, None]
        np.add.at(gL, (slice(None), self.l, slice(None)), gt * R[:, self.r, :])
        np.add.at(gR, (slice(None), self.r, slice(None)), gt * L[:, self.l, :])


class _Reduce:
    def __init__(self, d, pfx, src):
        self.W = np.asarray(d[f"{pfx}_reduce_{src}_W"], dtype=np.float64)          # [nel, n_out, n_in, w_shape]
        self.norm = float(_scalar(d, f"{pfx}_reduce_{src}_norm", 1.0))
        self.ci = d[f"{pfx}_collect_ind_{src}"].astype(np.int64).ravel()
        self.tile = d[f"{pfx}_w_l_tile_{src}"].astype(np.int64).ravel()

    def fwd(self, mu, X):
        """rho[a,k] = norm sum_c sum_n W[mu_a,k,n,tile c] X[a,ci c,n].  fused_cpu.h:637-643 + build_red."""
        Wc = self.W[:, :, :, self.tile]                                            # [nel, k, n, c]
        return np.einsum("aknc,acn->ak", Wc[mu], X[:, self.ci, :], optimize=True) * self.norm

    def bwd(self, mu, grho, gX):
        Wc = self.W[:, :, :, self.tile]
        g = np.einsum("aknc,ak->acn", Wc[mu], grho, optimize=True) * self.norm
        np.add.at(gX, (slice(None), self.ci, slice(None)), g)


class Model1L:
    """GRACE-1L model arrays as the oracle uses them (keys of src/model_1l.cpp:18-273)."""

    def __init__(self, path_or_dict):
        d = load_npz(path_or_dict) if isinstance(path_or_dict, str) else path_or_dict
        self.d = d
        self.n_elements = int(_scalar(d, "n_elements"))
        self.emb = int(_scalar(d, "embedding_size"))
        self.lmax = int(_scalar(d, "lmax"))
        self.nl = self.lmax + 1
        self.nlm = self.nl ** 2
        self.nrb = int(_scalar(d, "nradbase"))
        self.C = int(_scalar(d, "nradmax"))
        self.p = int(_scalar(d, "radial_basis_p", 16))
        self.rcut = float(_scalar(d, "rcut", 6.0))
        self.names = [s.decode() for s in d["element_names"]] if "element_names" in d else []
        if int(_scalar(d, "has_bond_specific_cutoff", 0)):
            self.cut = np.asarray(d["bond_cutoff_map"], dtype=np.float64).reshape(self.n_elements, self.n_elements)
        else:
            self.cut = np.full((self.n_elements, self.n_elements), self.rcut)
        nlay = int(_scalar(d, "mlp_rad_n_layers", 3))
        self.rad = [(np.asarray(d[f"mlp_rad_W{i}"], dtype=np.float64), float(_scalar(d, f"mlp_rad_norm{i}", 1.0)))
                    for i in range(nlay)]
        self.rad_act = int(_scalar(d, "radial_activation", 0))
        ce = np.asarray(d["chem_embedding"], dtype=np.float64)
        # z[mu, n] = (A_lin_W^T emb[mu]) norm inv_avg_n_neigh : src/fused_1l.cpp:150-162
        self.z = (ce @ np.asarray(d["A_lin_transform_W"], dtype=np.float64)) * \
            float(_scalar(d, "A_lin_transform_norm", 1.0)) * float(_scalar(d, "A_inv_avg_n_neigh", 1.0))
        self.fcA1 = _FC(d, "fc_A1")
        self.fcAA1 = _FC(d, "fc_AA1")
        self.pAA = _Prod(d, "prod_AA")
        self.pAAA = _Prod(d, "prod_AAA")
        self.order4 = "prod_AAAA_n_cg_terms" in d          # max_order3.h: absent stage contributes nothing
        if self.order4:
            self.fcAA2 = _FC(d, "fc_AA2")
            self.pAAAA = _Prod(d, "prod_AAAA")
        self.aaa_right_a = bool(int(_scalar(d, "AAA_right_A", 0)))
        self.nrho = int(_scalar(d, "rho_n_out"))
        self.red = {s: _Reduce(d, "rho", s) for s in (["A", "AA", "AAA"] + (["AAAA"] if self.order4 else []))}
        nel = int(_scalar(d, "energy_mlp_n_layers", 2))
        self.emlp = [(np.asarray(d[f"energy_mlp_W{i}"], dtype=np.float64).copy(),
                      float(_scalar(d, f"energy_mlp_norm{i}", 1.0))) for i in range(nel)]
        self.e_act = int(_scalar(d, "energy_mlp_activation", 0))
        self.e_ln = "energy_mlp_scale" in d                # src/npz3.h:330-338: scale folded into layer 0
        if self.e_ln:
            s = np.asarray(d["energy_mlp_scale"], dtype=np.float64).ravel()
            self.emlp[0] = (self.emlp[0][0] * s[:, None], self.emlp[0][1])
        self.shift = np.asarray(d["shift_values"], dtype=np.float64).ravel() if "shift_values" in d \
            else np.zeros(self.n_elements)
        self.out_scale = float(_scalar(d, "output_scale", 1.0))
        self.has_uq = int(_scalar(d, "uq_schema_version", 0)) == 6
        if self.has_uq:                                     # the uqv6 head: libgrace/src/uq_head.cpp:11-76
            self.uq_rp = int(_scalar(d, "uq_rp_dim"))
            self.uq_D = int(_scalar(d, "uq_feature_dim"))
            self.uq_K = int(_scalar(d, "uq_max_clusters"))
            self.uq_scale = float(_scalar(d, "uq_rp_density_scale", 1.0))
            self.uq_R = np.asarray(d["uq_rp_matrix"], dtype=np.float64).reshape(-1, self.uq_rp)
            self.uq_cen = np.asarray(d["uq_centroids"], dtype=np.float64).reshape(self.n_elements, self.uq_K, self.uq_D)
            self.uq_icov = np.asarray(d["uq_inv_cov"], dtype=np.float64).reshape(self.n_elements, self.uq_K, self.uq_D, self.uq_D)
            self.uq_ncl = np.asarray(d["uq_n_clusters"]).astype(np.int64).ravel()
            self.uq_thr = np.asarray(d["uq_interp_thresholds"], dtype=np.float64).reshape(self.n_elements, self.uq_K)

    def uq_features(self, t):
        """phi [atoms, rp_dim + n_density] = concat((B / |B|) R, log |B| density_scale ...)."""
        parts = []
        for src in ["A", "AA", "AAA"] + (["AAAA"] if self.order4 else []):
            X = t[src][:, self.red[src].ci, :]                                     # [a, c, n]
            parts.append(np.transpose(X, (0, 2, 1)).reshape(X.shape[0], -1))
        B = np.concatenate(parts, axis=1)
        nrm = np.sqrt((B * B).sum(1))
        f = np.empty((B.shape[0], self.uq_D))
        f[:, :self.uq_rp] = (B @ self.uq_R) / (nrm + 1.0e-12)[:, None]
        f[:, self.uq_rp:] = (np.log(nrm + 1.0e-12) * self.uq_scale)[:, None]
        return f

    def uq(self, mu, t):
        """gamma, sigma, cluster of every atom from the forward tensors (uqv6, gamma only).
        Basis: per source of the rho reduce, X_s[ci_s[c]][n] flattened n-outer, c-inner (fused_cpu.h:1290-1312,
        libgrace/include/grace/uq.h:1-9); projection, normalisation, log-norm density channels, nearest centroid,
        Mahalanobis distance: fused_cpu.h:1375-1412, src/fused_1l.cpp:616-636."""
        f = self.uq_features(t)
        na = f.shape[0]
        gamma, sigma, cluster = np.zeros(na), np.zeros(na), np.zeros(na)
        for a in range(na):
            m = mu[a]
            d2 = ((f[a][None, :] - self.uq_cen[m, :self.uq_ncl[m]]) ** 2).sum(1)
            k = int(np.argmin(d2))                                                 # the first of equal distances
            dl = f[a] - self.uq_cen[m, k]
            sigma[a] = np.sqrt(dl @ self.uq_icov[m, k] @ dl + 1.0e-8)
            gamma[a] = sigma[a] / max(self.uq_thr[m, k], 1.0e-10)
            cluster[a] = k
        return gamma, sigma, cluster

    # ---- per-atom dense chain -------------------------------------------------------------------------------
    def dense_forward(self, mu, A):
        """A[a, nlm, C] -> rho[a, nrho] and the tensors the reverse needs.  src/fused_1l.cpp:260-300."""
        t = {"A": A}
        t["A1"] = self.fcA1.fwd(A, A)
        t["AA"] = self.pAA.fwd(t["A1"], t["A1"])
        t["AA1"] = self.fcAA1.fwd(t["AA"], A)
        Ar = A if self.aaa_right_a else t["A1"]
        t["AAA"] = self.pAAA.fwd(t["AA1"], Ar)
        rho = self.red["A"].fwd(mu, A) + self.red["AA"].fwd(mu, t["AA"]) + self.red["AAA"].fwd(mu, t["AAA"])
        if self.order4:
            t["AA2"] = self.fcAA2.fwd(t["AA"], A)
            t["AAAA"] = self.pAAAA.fwd(t["AA2"], t["AA2"])
            rho = rho + self.red["AAAA"].fwd(mu, t["AAAA"])
        return rho, t

    def dense_backward(self, mu, t, grho):
        """dE/drho -> dE/dA.  src/fused_1l.cpp:306-349."""
        A = t["A"]
        gA = np.zeros_like(A)
        gA1 = np.zeros_like(t["A1"])
        gAA = np.zeros_like(t["AA"])
        gAA1 = np.zeros_like(t["AA1"])
        gAAA = np.zeros_like(t["AAA"])
        self.red["A"].bwd(mu, grho, gA)
        self.red["AA"].bwd(mu, grho, gAA)
        self.red["AAA"].bwd(mu, grho, gAAA)
        if self.order4:
            gAAAA = np.zeros_like(t["AAAA"])
            gAA2 = np.zeros_like(t["AA2"])
            self.red["AAAA"].bwd(mu, grho, gAAAA)
            self.pAAAA.bwd(t["AA2"], t["AA2"], gAAAA, gAA2, gAA2)
            self.fcAA2.bwd(gAA2, gAA, gA)
        if self.aaa_right_a:
            self.pAAA.bwd(t["AA1"], A, gAAA, gAA1, gA)
        else:
            self.pAAA.bwd(t["AA1"], t["A1"], gAAA, gAA1, gA1)
        self.fcAA1.bwd(gAA1, gAA, gA)
        self.pAA.bwd(t["A1"], t["A1"], gAA, gA1, gA1)
        self.fcA1.bwd(gA1, gA, gA)
        return gA

    def energy_atoms(self, mu, rho):
        """E_i = (MLP(rho[1:]) + rho[0]) output_scale + shift[mu_i] and dE/drho.  src/fused_1l.cpp:378-427;
        legacy RMS layer norm fused_cpu.h:666-682."""
        x = rho[:, 1:].copy()
        n = x.shape[1]
        if self.e_ln:
            x0 = x.copy()
            q = 1.0 / np.sqrt((x0 * x0).sum(1) / n + 1e-16)
            x = x0 * q[:, None]
        acts, pres = [x], []
        nlay = len(self.emlp)
        for L, (W, norm) in enumerate(self.emlp):
            pre = (acts[-1] @ W) * norm
            pres.append(pre)
            if L < nlay - 1:
                acts.append(np.tanh(pre) if self.e_act == 1 else pre / (1.0 + np.exp(-pre)))
            else:
                acts.append(pre)
        E = (acts[-1][:, 0] + rho[:, 0]) * self.out_scale + self.shift[mu]
        g = np.full((rho.shape[0], 1), self.out_scale)
        for L in range(nlay - 1, -1, -1):
            W, norm = self.emlp[L]
            if L < nlay - 1:
                v = pres[L]
                if self.e_act == 1:
                    tt = acts[L + 1]
                    g = g * (1.0 - tt * tt)
                else:
                    sg = 1.0 / (1.0 + np.exp(-v))
                    g = g * (sg * (1.0 + v * (1.0 - sg)))
            g = (g @ W.T) * norm
        if self.e_ln:
            tdot = (g * x0).sum(1)
            g = q[:, None] * (g - x0 * (tdot * q * q / n)[:, None])
        grho = np.empty_like(rho)
        grho[:, 0] = self.out_scale
        grho[:, 1:] = g
        return E, grho

    spline = 0    # > 0: the radial functions from cubic tables of that many intervals, as the reference's engines take them

    def radial_exact(self, x):
        g, dg = radial_basis(x, self.p, self.nrb)
        return mlp_value_tangent(self.rad, g, dg, self.rad_act)

    def radial(self, x):
        """R[nb, C, nl], dR/dx  (MLP output index o = n nl + l: src/fused_1l.cpp:123)."""
        R, dR = self.radial_exact(x) if self.spline <= 0 else spline_radial(self, "_tab", self.radial_exact, self.spline, x)
        return R.reshape(-1, self.C, self.nl), dR.reshape(-1, self.C, self.nl)


def spline_radial(owner, slot, exact, N, x):
    """Radial functions and d/dx from the reference's tables, in fp64 (the reference stores fp32 coefficients): N intervals
    over x in [0, 1], per interval the cubic through value and derivative of the MLP at both ends
    (Grace1LFused::build_splines, src/fused_1l.cpp:102-129: c = {f0, d0, -3 f0 - 2 d0 + 3 f1 - d1, 2 f0 + d0 - 2 f1 + d1}
    with d = f' / N), evaluated as spline_eval (libgrace/include/grace/fused_cpu.h:1052-1074): k = min(int(x N), N - 1),
    t = x N - k, R = c0 + t (c1 + t (c2 + t c3)), dR/dx = N (c1 + t (2 c2 + 3 c3 t)).  The table is kept on `owner`."""
    tab = getattr(owner, slot, None)
    if tab is None or tab[0] != N:
        F, D = exact(np.arange(N + 1) / N)
        tab = (N, F, D / N)
        setattr(owner, slot, tab)
    _, F, Dh = tab
    s = np.asarray(x, dtype=np.float64) * N
    k = np.clip(s.astype(np.int64), 0, N - 1)
    t = (s - k)[:, None]
    f0, f1, d0, d1 = F[k], F[k + 1], Dh[k], Dh[k + 1]
    c2 = -3.0 * f0 - 2.0 * d0 + 3.0 * f1 - d1
    c3 = 2.0 * f0 + d0 - 2.0 * f1 + d1
    return f0 + t * (d0 + t * (c2 + t * c3)), (d0 + t * (2.0 * c2 + t * 3.0 * c3)) * N


class ZeroBondError(ValueError):
    """bonds.h:49-62: two atoms at the same position."""


def compute_1l(model: Model1L, mu, offset, j, rij, *, chunk=512, want_forces=True, uq=False):
    """One GRACE-1L energy + forces + virial call on a CSR bond list.

    mu[n]      model element of every atom (all mapped)
    offset[n+1], j[nb], rij[nb,3]   bonds of central atom i are offset[i]:offset[i+1], r_ij = x_j - x_i (+ S cell)

    Returns dict(energy, energies[n], forces[n,3], virial[6] = (xx yy zz xy xz yz)).
    Driver skeleton: src/fused_1l.cpp:474-582; bond filter bonds.h:120-162 (keep r^2 < rc^2, error on r = 0).
    """
    mu = np.asarray(mu, dtype=np.int64)
    offset = np.asarray(offset, dtype=np.int64)
    j = np.asarray(j, dtype=np.int64)
    rij = np.asarray(rij, dtype=np.float64).reshape(-1, 3)
    n = mu.size
    lm_l = np.repeat(np.arange(model.nl), 2 * np.arange(model.nl) + 1)           # l of each lm
    energies = np.zeros(n)
    forces = np.zeros((n, 3))
    virial = np.zeros(6)
    virials = np.zeros((n, 6))
    lower = np.zeros((n, 3))    # yx zx zy of the centroid form (cvatom of the GPU engines: kk/grace_1l_kk_impl.h:1344-1362)
    uqv = [np.zeros(n), np.zeros(n), np.zeros(n)] if uq else None
    feats = np.zeros((n, model.uq_D)) if uq else None
    for a0 in range(0, n, chunk):
        a1 = min(n, a0 + chunk)
        na = a1 - a0
        b0, b1 = offset[a0], offset[a1]
        bi = np.repeat(np.arange(a0, a1), np.diff(offset[a0:a1 + 1]))            # central atom of each bond
        bj = j[b0:b1]
        d = rij[b0:b1]
        rsq = d[:, 0] * d[:, 0] + d[:, 1] * d[:, 1] + d[:, 2] * d[:, 2]
        rc = model.cut[mu[bi], mu[bj]]
        keep = rsq < rc * rc
        if np.any(keep & (rsq == 0.0)):
            q = np.nonzero(keep & (rsq == 0.0))[0][0]
            raise ZeroBondError(f"two atoms at the same position (a bond of length 0 between atoms {bi[q]} and "
                                f"{bj[q]} of the neighbour list): not a physical structure")
        bi, bj, d, rsq, rc = bi[keep], bj[keep], d[keep], rsq[keep], rc[keep]
        r = np.sqrt(rsq)
        rh = d * (1.0 / r)[:, None]
        Y, G = real_sh(rh, model.lmax)
        R, dR = model.radial(r / rc)                                             # [nb, C, nl]
        zb = model.z[mu[bj]]                                                     # [nb, C]
        # A[lm][n] = sum_b Y_lm R_{n,l(lm)} z[n] : fused_cpu.h:947-982
        Rz = R * zb[:, :, None]
        contrib = Y[:, :, None] * np.transpose(Rz, (0, 2, 1))[:, lm_l, :]       # [nb, nlm, C]
        A = np.zeros((na, model.nlm, model.C))
        np.add.at(A, bi - a0, contrib)
        rho, t = model.dense_forward(mu[a0:a1], A)
        E, grho = model.energy_atoms(mu[a0:a1], rho)
        energies[a0:a1] = E
        if uq:
            for dst, val in zip(uqv, model.uq(mu[a0:a1], t)):
                dst[a0:a1] = val
            feats[a0:a1] = model.uq_features(t)
        if not want_forces:
            continue
        gA = model.dense_backward(mu[a0:a1], t, grho)
        gAb = gA[bi - a0]                                                        # [nb, nlm, C]
        # fused_cpu.h:836-860: gY[lm] = gA[lm].(R_l z), gR[l] = z sum_{lm in l} Y gA[lm]
        gY = np.einsum("bqn,bqn->bq", gAb, np.transpose(Rz, (0, 2, 1))[:, lm_l, :])
        YgA = Y[:, :, None] * gAb                                                # [nb, nlm, C]
        gR = np.zeros((bi.size, model.nl, model.C))
        np.add.at(gR, (slice(None), lm_l, slice(None)), YgA)
        gR *= zb[:, None, :]
        dEdx = np.einsum("bln,bnl->b", gR, dR)
        # fused_cpu.h:1036-1050: fv = dEdx/rc rhat + (g - (g.rhat) rhat)/r,  g = sum_lm gY G
        gv = np.einsum("bq,bqd->bd", gY, G)
        gr = (gv * rh).sum(1)
        fv = (dEdx / rc)[:, None] * rh + (gv - gr[:, None] * rh) / r[:, None]
        np.add.at(forces, bi, fv)                                                # fused_cpu.h:1089-1095
        np.add.at(forces, bj, -fv)
        dl = -rh * r[:, None]                                                    # src/fused_1l.cpp:46-51
        v6 = bond_virials(dl, fv)
        virial += v6.sum(0)
        np.add.at(virials, bi, 0.5 * v6)                                         # add_vatom, fused_cpu.h:1075-1087: half to each atom
        np.add.at(virials, bj, 0.5 * v6)
        l3 = 0.5 * np.stack([dl[:, 1] * fv[:, 0], dl[:, 2] * fv[:, 0], dl[:, 2] * fv[:, 1]], axis=1)    # v6 v7 v8 of kk/grace_1l_kk_impl.h:1346
        np.add.at(lower, bi, l3)
        np.add.at(lower, bj, l3)
    out = {"energy": float(energies.sum()), "energies": energies, "forces": forces, "virial": virial, "virials": virials,
           "centroid_virials": np.concatenate([virials, lower], axis=1)}
    if uq:
        out.update(gamma=uqv[0], atomic_sigma=uqv[1], gmm_cluster=uqv[2], uq_features=feats)
    return out


def bond_virials(dl, fv):
    """[nb, 6] = (xx yy zz xy xz yz) of dl (x) fv per bond, dl = x_i - x_j, fv = force on i (src/fused_1l.cpp:46-51)"""
    return np.stack([dl[:, 0] * fv[:, 0], dl[:, 1] * fv[:, 1], dl[:, 2] * fv[:, 2], dl[:, 0] * fv[:, 1], dl[:, 0] * fv[:, 2],
                     dl[:, 1] * fv[:, 2]], axis=1)


def virial_to_stress(virial, volume):
    """ASE Voigt stress (xx yy zz yz xz xy) from the virial (xx yy zz xy xz yz):
    python/grace_runtime/calculator.py:155-157."""
    v = np.asarray(virial, dtype=np.float64)
    return -v[[0, 1, 2, 5, 4, 3]] / volume
