"""CPU oracle for the GRACE-2L energy + forces + virial path (TEST INFRASTRUCTURE, not product code).

Plain numpy fp64 restatement of the reference's two-layer CPU driver.  Only the tests, the smoke check and the
CPU-baseline leg of the benchmark may import it; the shipped library never does.

Reference followed (paths relative to the reference checkout):

* model arrays ................................... libgrace/src/model_2l.cpp:28-420          (load_arrays)
* layer 1 forward (A .. AAAA, I1, rho, I) ........ libgrace/src/fused_2l.cpp:404-452          (layer1_forward)
* equivariant reduce with total_sum_ind .......... libgrace/include/grace/fused_cpu.h:1202-1273 (build_red), :637-649
* message pairs (y, I), YI coupling .............. libgrace/src/fused_2l.cpp:228-276
* layer 2 forward, energy, layer-2 reverse ....... libgrace/src/fused_2l.cpp:621-781          (layer2)
* neighbour gather Y R1 I_j ...................... libgrace/include/grace/fused_cpu.h:984-1025 (atom_yi)
* its reverse, dE/dI_j scatter ................... libgrace/include/grace/fused_cpu.h:903-942  (bond_yi_bwd_g, _commit)
* readout with the two RMSNorms .................. libgrace/src/fused_2l.cpp:548-615          (energy_atom)
* layer 1 reverse ................................ libgrace/src/fused_2l.cpp:458-542          (layer1_backward)
* phases P1 .. P5 ................................ libgrace/src/fused_2l.cpp:849-1099         (compute)
* UQ head (uqv6, gamma only): keys, basis blocks .. libgrace/src/model_2l.cpp:404-478, src/fused_2l.cpp:1156-1186,
  GMM ............................................ libgrace/include/grace/fused_cpu.h:1375-1412

Pinning status: end to end (energy, per-atom energies, forces, stress) against the reference's TensorFlow fp64
goldens of grace_2l_order3 / legacy_2l_order3 on W54, WMo54, W2tri (tests/fixtures/ref_tf/order3_tf.npz), by finite
differences of the energy, and against the compiled reference (oracle/_ref) for models with the BBBB / AAAA stages and
the synthetic benchmark models.  UQ head (uq_features, uq): against the compiled reference on a generated head attached
to the fixture model grace_2l_small (cluster indices exactly, gamma and sigma to 1e-4: its projection is fp32), live and
as committed goldens, and by what the definition fixes (tests/test_uq.py).
"""
from __future__ import annotations

import numpy as np

from .grace_oracle import (ZeroBondError, _FC, _Prod, _scalar, load_npz, mlp_value_tangent, radial_basis, real_sh, spline_radial)

__all__ = ["Model2L", "compute_2l"]


class _ReduceEq:
    """Reduce with per-connection output function fo = total_sum_ind (equivariant) or one output function (scalar).
    out[a, fo_c, k] += norm sum_n W[(mu_a,) k, n, tile_c] X[a, ci_c, n].  fused_cpu.h:1202-1273 + :637-649."""

    def __init__(self, d, pfx, src, elem, scalar):
        W = np.asarray(d[f"{pfx}_reduce_{src}_W"], dtype=np.float64)
        self.elem = elem
        self.W = W if elem else W[None]                                            # [nel | 1, k, n, w_shape]
        self.norm = float(_scalar(d, f"{pfx}_reduce_{src}_norm", 1.0))
        self.ci = d[f"{pfx}_collect_ind_{src}"].astype(np.int64).ravel()
        self.tile = d[f"{pfx}_w_l_tile_{src}"].astype(np.int64).ravel()
        self.fo = np.zeros_like(self.ci) if scalar else d[f"{pfx}_total_sum_ind_{src}"].astype(np.int64).ravel()

    def fwd(self, mu, X, out):
        Wc = self.W[:, :, :, self.tile]                                            # [nel, k, n, c]
        idx = mu if self.elem else np.zeros_like(mu)
        v = np.einsum("aknc,acn->ack", Wc[idx], X[:, self.ci, :], optimize=True) * self.norm
        np.add.at(out, (slice(None), self.fo, slice(None)), v)

    def bwd(self, mu, gout, gX):
        Wc = self.W[:, :, :, self.tile]
        idx = mu if self.elem else np.zeros_like(mu)
        g = np.einsum("aknc,ack->acn", Wc[idx], gout[:, self.fo, :], optimize=True) * self.norm
        np.add.at(gX, (slice(None), self.ci, slice(None)), g)


def _mlp(d, pfx):
    n = int(_scalar(d, pfx + "_n_layers", 3))
    return [(np.asarray(d[f"{pfx}_W{i}"], dtype=np.float64), float(_scalar(d, f"{pfx}_norm{i}", 1.0))) for i in range(n)]


class Model2L:
    """GRACE-2L model arrays (keys of src/model_2l.cpp:28-420)."""

    def __init__(self, path_or_dict):
        d = load_npz(path_or_dict) if isinstance(path_or_dict, str) else path_or_dict
        self.d = d
        self.n_elements = int(_scalar(d, "n_elements"))
        self.lmax = int(_scalar(d, "lmax"))
        self.nl = self.lmax + 1
        self.nlm = self.nl ** 2
        self.nrb = int(_scalar(d, "nradbase"))
        self.p = int(_scalar(d, "radial_basis_p", 16))
        self.rcut = float(_scalar(d, "rcut", 6.0))
        self.names = [s.decode() for s in d["element_names"]] if "element_names" in d else []
        if int(_scalar(d, "has_bond_specific_cutoff", 0)):
            self.cut = np.asarray(d["bond_cutoff_map"], dtype=np.float64).reshape(self.n_elements, self.n_elements)
        else:
            self.cut = np.full((self.n_elements, self.n_elements), self.rcut)
        self.C1 = int(_scalar(d, "mlp_rad_R_n_rad_max"))
        self.CR = int(_scalar(d, "mlp_rad_R1_n_rad_max"))
        self.rad1 = _mlp(d, "mlp_rad_R")
        self.rad2 = _mlp(d, "mlp_rad_R1")
        self.rad_act = int(_scalar(d, "radial_activation", 0))
        ce = np.asarray(d["chem_embedding"], dtype=np.float64)
        # fused_2l.cpp:176-192
        self.zA = (ce @ np.asarray(d["A_lin_transform_W"], dtype=np.float64)) * \
            float(_scalar(d, "A_lin_transform_norm", 1.0)) * float(_scalar(d, "A_inv_avg_n_neigh", 1.0))
        self.zB0 = (ce @ np.asarray(d["B0_lin_transform_W"], dtype=np.float64)) * \
            float(_scalar(d, "B0_lin_transform_norm", 1.0)) * float(_scalar(d, "B0_inv_avg_n_neigh", 1.0))
        self.order4 = "prod_AAAA_n_cg_terms" in d       # max_order3.h: absent AAAA / BBBB stages contribute nothing
        self.fcA1, self.fcAA1 = _FC(d, "fc_A1"), _FC(d, "fc_AA1")
        self.pAA, self.pAAA = _Prod(d, "prod_AA"), _Prod(d, "prod_AAA")
        self.fcB1, self.fcBB1 = _FC(d, "fc_B1"), _FC(d, "fc_BB1")
        self.pBB, self.pBBB = _Prod(d, "prod_BB"), _Prod(d, "prod_BBB")
        if self.order4:
            self.fcAA2, self.pAAAA = _FC(d, "fc_AA2"), _Prod(d, "prod_AAAA")
            self.fcBB2, self.pBBBB = _FC(d, "fc_BB2"), _Prod(d, "prod_BBBB")
        s1 = ["A", "AA", "AAA"] + (["AAAA"] if self.order4 else [])
        s2 = ["B", "BB", "BBB"] + (["BBBB"] if self.order4 else [])
        self.nI1, self.I1_n_out = int(_scalar(d, "I1_n_funcs")), int(_scalar(d, "I1_n_out"))
        self.nI = int(_scalar(d, "I_n_funcs"))
        self.nB, self.C2 = int(_scalar(d, "B_n_funcs")), int(_scalar(d, "B_n_out"))
        self.nrho = int(_scalar(d, "rho_n_out"))
        self.rI1 = {s: _ReduceEq(d, "I1", s, True, False) for s in s1}
        self.rRho = {s: _ReduceEq(d, "rho", s, True, True) for s in s1}
        self.rI = _ReduceEq(d, "I", "I1", False, False)
        self.rB = {s: _ReduceEq(d, "B", s, False, False) for s in ("YI", "B0")}
        self.rI2 = {s: _ReduceEq(d, "I2", s, True, True) for s in s2}
        # YI coupling: unique (y, I) pairs, terms (pair, o, c)   fused_2l.cpp:228-276
        lr = d["YI_lr_inds"].astype(np.int64).reshape(-1, 2)
        self.yi_o = d["YI_m_sum_ind"].astype(np.int64).ravel()
        self.yi_c = np.asarray(d["YI_cg_coeff"], dtype=np.float64).ravel()
        self.nYI = int(_scalar(d, "YI_n_output_funcs"))
        self.yi_inv = float(_scalar(d, "YI_inv_avg_n_neigh", 1.0))
        pairs = sorted({(int(y), int(i)) for y, i in lr})
        pid = {p: q for q, p in enumerate(pairs)}
        self.yp_y = np.array([p[0] for p in pairs], dtype=np.int64)
        self.yp_i = np.array([p[1] for p in pairs], dtype=np.int64)
        self.yp_l = np.floor(np.sqrt(self.yp_y + 1e-9)).astype(np.int64)
        self.yt_pair = np.array([pid[(int(y), int(i))] for y, i in lr], dtype=np.int64)
        self.uq_setup(d)
        self.SYI = np.zeros((self.nYI, len(pairs)))                                 # YI[o] = sum_p SYI[o, p] YIp[p]
        np.add.at(self.SYI, (self.yi_o, self.yt_pair), self.yi_c * self.yi_inv)
        # readout
        self.rms = bool(int(_scalar(d, "energy_rms_norm", 1)))
        if self.rms:
            self.lnI = np.asarray(d["I_nl_LN_scale"], dtype=np.float64).ravel()
            self.ln0 = np.asarray(d["I_0_LN_scale"], dtype=np.float64).ravel()
        else:
            self.lnI, self.ln0 = np.ones(self.nrho - 1), np.ones(self.nrho)
        self.emlp = [(W.copy(), n) for W, n in _mlp(d, "energy_mlp")] if "energy_mlp_n_layers" in d else \
            [(np.asarray(d[f"energy_mlp_W{i}"], dtype=np.float64).copy(), float(_scalar(d, f"energy_mlp_norm{i}", 1.0)))
             for i in range(2)]
        self.e_act = int(_scalar(d, "energy_mlp_activation", 1))
        self.e_ln = "energy_mlp_scale" in d
        if self.e_ln:
            s = np.asarray(d["energy_mlp_scale"], dtype=np.float64).ravel()
            self.emlp[0] = (self.emlp[0][0] * s[:, None], self.emlp[0][1])
        self.shift = np.asarray(d["shift_values"], dtype=np.float64).ravel() if "shift_values" in d \
            else np.zeros(self.n_elements)
        self.out_scale = float(_scalar(d, "output_scale", 1.0))

    def uq_setup(self, d):
        """the uqv6 UQ head (libgrace/src/model_2l.cpp:404-478): blocks [I2 over B .. BBBB, rho over A .. AAAA]"""
        self.has_uq = int(_scalar(d, "uq_schema_version", 0)) == 6
        if not self.has_uq:
            return
        ne = int(_scalar(d, "n_elements"))
        self.uq_rp, self.uq_D, self.uq_K = int(_scalar(d, "uq_rp_dim")), int(_scalar(d, "uq_feature_dim")), int(_scalar(d, "uq_max_clusters"))
        self.uq_scale = float(_scalar(d, "uq_rp_density_scale", 1.0))
        self.uq_R = np.asarray(d["uq_rp_matrix"], dtype=np.float64).reshape(-1, self.uq_rp)
        self.uq_cen = np.asarray(d["uq_centroids"], dtype=np.float64).reshape(ne, self.uq_K, self.uq_D)
        self.uq_icov = np.asarray(d["uq_inv_cov"], dtype=np.float64).reshape(ne, self.uq_K, self.uq_D, self.uq_D)
        self.uq_ncl = np.asarray(d["uq_n_clusters"]).astype(np.int64).ravel()
        self.uq_thr = np.asarray(d["uq_interp_thresholds"], dtype=np.float64).reshape(ne, self.uq_K)

    def uq_features(self, t1, t2):
        """phi = ((B / |B|) R, log |B|, log |B_I2|, log |B_rho|) density_scale; B = [I2 block, rho block], each the collected
        functions of its reduce's sources, n-outer and c-inner (libgrace/include/grace/uq.h:1-9, src/fused_2l.cpp:1156-1186)."""
        blocks = []
        for reds, t in ((self.rI2, t2), (self.rRho, t1)):
            parts = []
            for src, r in reds.items():
                X = t[src][:, r.ci, :]
                parts.append(np.transpose(X, (0, 2, 1)).reshape(X.shape[0], -1))
            blocks.append(np.concatenate(parts, axis=1))
        B = np.concatenate(blocks, axis=1)
        nrm = np.sqrt((B * B).sum(1))
        f = np.empty((B.shape[0], self.uq_D))
        f[:, :self.uq_rp] = (B @ self.uq_R) / (nrm + 1.0e-12)[:, None]
        f[:, self.uq_rp] = np.log(nrm + 1.0e-12) * self.uq_scale
        for b, blk in enumerate(blocks):
            f[:, self.uq_rp + 1 + b] = np.log(np.sqrt((blk * blk).sum(1)) + 1.0e-12) * self.uq_scale
        return f

    def uq(self, mu, f):
        """nearest centroid of the element, Mahalanobis distance, gamma (libgrace/include/grace/fused_cpu.h:1375-1412)"""
        na = f.shape[0]
        gamma, sigma, cluster = np.zeros(na), np.zeros(na), np.zeros(na)
        for a in range(na):
            m = mu[a]
            d2 = ((f[a][None, :] - self.uq_cen[m, :self.uq_ncl[m]]) ** 2).sum(1)
            k = int(np.argmin(d2))
            dl = f[a] - self.uq_cen[m, k]
            sigma[a] = np.sqrt(dl @ self.uq_icov[m, k] @ dl + 1.0e-8)
            gamma[a] = sigma[a] / max(self.uq_thr[m, k], 1.0e-10)
            cluster[a] = k
        return gamma, sigma, cluster

    spline = 0    # > 0: the radial functions of both layers from cubic tables of that many intervals (grace_oracle.spline_radial)

    def radial(self, which, x):
        layers, C = (self.rad1, self.C1) if which == 1 else (self.rad2, self.CR)

        def exact(xs):
            g, dg = radial_basis(xs, self.p, self.nrb)
            return mlp_value_tangent(layers, g, dg, self.rad_act)
        R, dR = exact(x) if self.spline <= 0 else spline_radial(self, f"_tab{which}", exact, self.spline, x)
        return R.reshape(-1, C, self.nl), dR.reshape(-1, C, self.nl)

    # ---- layer 1 dense chain: fused_2l.cpp:404-452 ------------------------------------------------------------
    def layer1_forward(self, mu, A):
        t = {"A": A}
        t["A1"] = self.fcA1.fwd(A, A)
        t["AA"] = self.pAA.fwd(t["A1"], t["A1"])
        t["AA1"] = self.fcAA1.fwd(t["AA"], A)
        t["AAA"] = self.pAAA.fwd(t["AA1"], A)
        if self.order4:
            t["AA2"] = self.fcAA2.fwd(t["AA"], A)
            t["AAAA"] = self.pAAAA.fwd(t["AA2"], t["AA2"])
        na = A.shape[0]
        I1 = np.zeros((na, self.nI1, self.I1_n_out))
        rho = np.zeros((na, 1, self.nrho))
        for s in self.rI1:
            self.rI1[s].fwd(mu, t[s], I1)
            self.rRho[s].fwd(mu, t[s], rho)
        Iv = np.zeros((na, self.nI, self.CR))
        self.rI.fwd(mu, I1, Iv)
        t["I1"] = I1
        return Iv, rho[:, 0, :], t

    def layer1_backward(self, mu, t, gI, grho):
        """dE/dI, dE/drho of the chunk's atoms -> dE/dA.  fused_2l.cpp:458-509."""
        A = t["A"]
        gI1 = np.zeros_like(t["I1"])
        self.rI.bwd(mu, gI, gI1)
        g = {k: np.zeros_like(t[k]) for k in t if k != "I1"}
        grho3 = grho[:, None, :]
        for s in self.rI1:
            self.rI1[s].bwd(mu, gI1, g[s])
            self.rRho[s].bwd(mu, grho3, g[s])
        if self.order4:
            self.pAAAA.bwd(t["AA2"], t["AA2"], g["AAAA"], g["AA2"], g["AA2"])
            self.fcAA2.bwd(g["AA2"], g["AA"], g["A"])
        self.pAAA.bwd(t["AA1"], A, g["AAA"], g["AA1"], g["A"])
        self.fcAA1.bwd(g["AA1"], g["AA"], g["A"])
        self.pAA.bwd(t["A1"], t["A1"], g["AA"], g["A1"], g["A1"])
        self.fcA1.bwd(g["A1"], g["A"], g["A"])
        return g["A"]

    # ---- layer 2 dense chain: fused_2l.cpp:655-760 ------------------------------------------------------------
    def layer2_forward(self, mu, YIp, B0):
        t = {"B0": B0, "YIp": YIp}
        YI = np.einsum("op,apn->aon", self.SYI, YIp, optimize=True)
        na = B0.shape[0]
        B = np.zeros((na, self.nB, self.C2))
        self.rB["YI"].fwd(mu, YI, B)
        self.rB["B0"].fwd(mu, B0, B)
        t["B"] = B
        t["B1"] = self.fcB1.fwd(B, B)
        t["BB"] = self.pBB.fwd(t["B1"], t["B1"])
        t["BB1"] = self.fcBB1.fwd(t["BB"], B)
        t["BBB"] = self.pBBB.fwd(t["BB1"], B)
        if self.order4:
            t["BB2"] = self.fcBB2.fwd(t["BB"], B)
            t["BBBB"] = self.pBBBB.fwd(t["BB2"], t["BB2"])
        I2 = np.zeros((na, 1, self.nrho))
        for s in self.rI2:
            self.rI2[s].fwd(mu, t[s], I2)
        return I2[:, 0, :], t

    def layer2_backward(self, mu, t, gI2):
        B = t["B"]
        g = {k: np.zeros_like(t[k]) for k in ("B", "B1", "BB", "BB1", "BBB")}
        if self.order4:
            g["BB2"], g["BBBB"] = np.zeros_like(t["BB2"]), np.zeros_like(t["BBBB"])
        for s in self.rI2:
            self.rI2[s].bwd(mu, gI2[:, None, :], g[s])
        if self.order4:
            self.pBBBB.bwd(t["BB2"], t["BB2"], g["BBBB"], g["BB2"], g["BB2"])
            self.fcBB2.bwd(g["BB2"], g["BB"], g["B"])
        self.pBBB.bwd(t["BB1"], B, g["BBB"], g["BB1"], g["B"])
        self.fcBB1.bwd(g["BB1"], g["BB"], g["B"])
        self.pBB.bwd(t["B1"], t["B1"], g["BB"], g["B1"], g["B1"])
        self.fcB1.bwd(g["B1"], g["B"], g["B"])
        na = B.shape[0]
        gYI = np.zeros((na, self.nYI, self.CR))
        gB0 = np.zeros_like(t["B0"])
        self.rB["YI"].bwd(mu, g["B"], gYI)
        self.rB["B0"].bwd(mu, g["B"], gB0)
        gYIp = np.einsum("op,aon->apn", self.SYI, gYI, optimize=True)
        return gYIp, gB0

    # ---- readout: fused_2l.cpp:548-615 -----------------------------------------------------------------------
    def energy_atoms(self, mu, rho, I2):
        eps = 1e-10                                                                  # model_2l.h:156
        nr = self.nrho
        if self.rms:
            s1 = np.sqrt((rho[:, 1:] ** 2).sum(1) / (nr - 1) + eps)
            s0 = np.sqrt((I2 ** 2).sum(1) / nr + eps)
        else:
            s1 = np.ones(rho.shape[0])
            s0 = np.ones(rho.shape[0])
        x = rho[:, 1:] / s1[:, None] * self.lnI[None, :] + I2[:, 1:] / s0[:, None] * self.ln0[None, 1:]
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
        E = (acts[-1][:, 0] + rho[:, 0] + I2[:, 0] / s0 * self.ln0[0]) * self.out_scale + self.shift[mu]
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
        t1 = (g * self.lnI[None, :] * rho[:, 1:]).sum(1) if self.rms else np.zeros(rho.shape[0])
        grho[:, 1:] = g * self.lnI[None, :] / s1[:, None] - rho[:, 1:] * (t1 / ((nr - 1) * s1 ** 3))[:, None]
        gy = np.empty_like(I2)
        gy[:, 0] = self.out_scale
        gy[:, 1:] = g
        t0 = (gy * self.ln0[None, :] * I2).sum(1) if self.rms else np.zeros(rho.shape[0])
        gI2 = gy * self.ln0[None, :] / s0[:, None] - I2 * (t0 / (nr * s0 ** 3))[:, None]
        return E, grho, gI2


def _bond_force(dEdx, gY, G, rh, r, rc):
    """fused_cpu.h:1036-1050: fv = dEdx/rc rhat + (g - (g.rhat) rhat)/r,  g = sum_lm gY G."""
    gv = np.einsum("bq,bqd->bd", gY, G)
    gr = (gv * rh).sum(1)
    return (dEdx / rc)[:, None] * rh + (gv - gr[:, None] * rh) / r[:, None]


def _add_vatom(virials, bi, bj, rh, r, fv):
    """add_vatom, libgrace/include/grace/fused_cpu.h:1075-1087: half of the bond's (x_i - x_j) (x) f_i to each of its atoms"""
    dl = -rh * r[:, None]
    v6 = 0.5 * np.stack([dl[:, 0] * fv[:, 0], dl[:, 1] * fv[:, 1], dl[:, 2] * fv[:, 2], dl[:, 0] * fv[:, 1], dl[:, 0] * fv[:, 2],
                         dl[:, 1] * fv[:, 2]], axis=1)
    np.add.at(virials, bi, v6)
    np.add.at(virials, bj, v6)


def _virial(rh, r, fv):
    dl = -rh * r[:, None]
    return np.array([(dl[:, 0] * fv[:, 0]).sum(), (dl[:, 1] * fv[:, 1]).sum(), (dl[:, 2] * fv[:, 2]).sum(),
                     (dl[:, 0] * fv[:, 1]).sum(), (dl[:, 0] * fv[:, 2]).sum(), (dl[:, 1] * fv[:, 2]).sum()])


def compute_2l(model: Model2L, mu, offset, j, rij, *, chunk=128, want_forces=True, uq=False):
    """One GRACE-2L energy + forces + virial call on a CSR bond list of a closed system (every j is a central atom:
    the periodic images are folded onto their owners, as the reference's CSR path does).

    Arguments and result as compute_1l.  Phases of src/fused_2l.cpp:849-1099: P1 layer 1 forward -> I, rho of every
    atom; P3 layer 2 + energy + layer-2 reverse (forces of the layer-2 bonds, dE/dI_j summed per neighbour);
    P5 layer 1 reverse with dE/dI and dE/drho."""
    mu = np.asarray(mu, dtype=np.int64)
    offset = np.asarray(offset, dtype=np.int64)
    j = np.asarray(j, dtype=np.int64)
    rij = np.asarray(rij, dtype=np.float64).reshape(-1, 3)
    n = mu.size
    nl, nlm = model.nl, model.nlm
    lm_l = np.repeat(np.arange(nl), 2 * np.arange(nl) + 1)
    energies = np.zeros(n)
    forces = np.zeros((n, 3))
    virial = np.zeros(6)
    virials = np.zeros((len(mu), 6))

    def bonds(a0, a1):
        b0, b1 = offset[a0], offset[a1]
        bi = np.repeat(np.arange(a0, a1), np.diff(offset[a0:a1 + 1]))
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
        return bi, bj, r, rc, rh, Y, G

    chunks = [(a0, min(n, a0 + chunk)) for a0 in range(0, n, chunk)]
    I_glob = np.zeros((n, model.nI, model.CR))
    rho_glob = np.zeros((n, model.nrho))
    state = []
    # ---- P1
    for a0, a1 in chunks:
        bi, bj, r, rc, rh, Y, G = bonds(a0, a1)
        R, _ = model.radial(1, r / rc)
        Rz = np.transpose(R * model.zA[mu[bj]][:, :, None], (0, 2, 1))[:, lm_l, :]     # [nb, nlm, C1]
        A = np.zeros((a1 - a0, nlm, model.C1))
        np.add.at(A, bi - a0, Y[:, :, None] * Rz)
        Iv, rho, t = model.layer1_forward(mu[a0:a1], A)
        I_glob[a0:a1] = Iv
        rho_glob[a0:a1] = rho
        state.append(t)
    # ---- P3
    feats = np.zeros((n, model.uq_D)) if uq else None
    gI_sum = np.zeros_like(I_glob)
    grho_glob = np.zeros_like(rho_glob)
    for a0, a1 in chunks:
        bi, bj, r, rc, rh, Y, G = bonds(a0, a1)
        R1, dR1 = model.radial(2, r / rc)                                              # [nb, CR, nl]
        R1t = np.transpose(R1, (0, 2, 1))                                              # [nb, nl, CR]
        zb = model.zB0[mu[bj]]
        B0 = np.zeros((a1 - a0, nlm, model.CR))
        np.add.at(B0, bi - a0, Y[:, :, None] * (R1t * zb[:, None, :])[:, lm_l, :])
        Ij = I_glob[bj]                                                                # [nb, nI, CR]
        RI = R1t[:, model.yp_l, :] * Ij[:, model.yp_i, :]                              # [nb, npair, CR]
        YIp = np.zeros((a1 - a0, model.yp_y.size, model.CR))
        np.add.at(YIp, bi - a0, Y[:, model.yp_y, None] * RI)
        I2, t2 = model.layer2_forward(mu[a0:a1], YIp, B0)
        E, grho, gI2 = model.energy_atoms(mu[a0:a1], rho_glob[a0:a1], I2)
        energies[a0:a1] = E
        if uq:
            feats[a0:a1] = model.uq_features(state[chunks.index((a0, a1))], t2)
        if not want_forces:
            continue
        grho_glob[a0:a1] = grho
        gYIp, gB0 = model.layer2_backward(mu[a0:a1], t2, gI2)
        gB0b = gB0[bi - a0]                                                            # [nb, nlm, CR]
        gPb = gYIp[bi - a0]                                                            # [nb, npair, CR]
        # B0 part: as the layer-1 bond reverse with z = zB0
        gY = np.einsum("bqn,bqn->bq", gB0b, (R1t * zb[:, None, :])[:, lm_l, :])
        gR = np.zeros((bi.size, nl, model.CR))
        np.add.at(gR, (slice(None), lm_l, slice(None)), Y[:, :, None] * gB0b)
        gR *= zb[:, None, :]
        # YI part: fused_cpu.h:903-932
        np.add.at(gY, (slice(None), model.yp_y), (gPb * RI).sum(2))
        YgP = Y[:, model.yp_y, None] * gPb                                             # [nb, npair, CR]
        np.add.at(gR, (slice(None), model.yp_l, slice(None)), YgP * Ij[:, model.yp_i, :])
        gIj = np.zeros_like(Ij)
        np.add.at(gIj, (slice(None), model.yp_i, slice(None)), YgP * R1t[:, model.yp_l, :])
        np.add.at(gI_sum, bj, gIj)
        dEdx = np.einsum("bln,bnl->b", gR, dR1)
        fv = _bond_force(dEdx, gY, G, rh, r, rc)
        np.add.at(forces, bi, fv)
        np.add.at(forces, bj, -fv)
        virial += _virial(rh, r, fv)
        _add_vatom(virials, bi, bj, rh, r, fv)                                         # src/fused_2l.cpp:778
    if want_forces:
        # ---- P5
        for (a0, a1), t in zip(chunks, state):
            bi, bj, r, rc, rh, Y, G = bonds(a0, a1)
            R, dR = model.radial(1, r / rc)
            zb = model.zA[mu[bj]]
            Rz = np.transpose(R * zb[:, :, None], (0, 2, 1))[:, lm_l, :]
            gA = model.layer1_backward(mu[a0:a1], t, gI_sum[a0:a1], grho_glob[a0:a1])
            gAb = gA[bi - a0]
            gY = np.einsum("bqn,bqn->bq", gAb, Rz)
            gR = np.zeros((bi.size, nl, model.C1))
            np.add.at(gR, (slice(None), lm_l, slice(None)), Y[:, :, None] * gAb)
            gR *= zb[:, None, :]
            dEdx = np.einsum("bln,bnl->b", gR, dR)
            fv = _bond_force(dEdx, gY, G, rh, r, rc)
            np.add.at(forces, bi, fv)
            np.add.at(forces, bj, -fv)
            virial += _virial(rh, r, fv)
            _add_vatom(virials, bi, bj, rh, r, fv)                                     # src/fused_2l.cpp:539
    out = {"energy": float(energies.sum()), "energies": energies, "forces": forces, "virial": virial, "virials": virials}
    if uq:
        g, sg, cl = model.uq(mu, feats)
        out.update(gamma=g, atomic_sigma=sg, gmm_cluster=cl, uq_features=feats)
    return out
