"""CPU oracle for the GRACE-3L energy + forces + virial path (TEST INFRASTRUCTURE, not product code).

fp64 restatement of the forward pass of the reference's three-layer CPU driver on torch CPU tensors; forces and
the virial come from reverse-mode differentiation of that forward pass with respect to the bond vectors (the
reference codes the same adjoints by hand).  Only the tests, the smoke check and the CPU-baseline leg of the
benchmark may import it; the shipped library never does.

Reference followed (paths relative to the reference checkout):

* model arrays, layer dataflow ................... libgrace/src/model_3l.cpp:36-154 (validate_layers), :165-464
* radial MLP on [T_k(2x-1), emb_i, emb_j] ........ libgrace/src/fused_3l.cpp:299-346  (radial_mlp_x)
* envelope, species factor, o = c (lmax+1) + l ... libgrace/src/fused_3l.cpp:441-521, :1085-1146
* scalar SPBF (layer 1) .......................... libgrace/src/fused_3l.cpp:1239-1253
* equivariant SPBF (layers 2, 3) ................. libgrace/src/fused_3l.cpp:1049-1083 (bond_vectors), :1254-1275
* contraction over (src, dst, tile) connections .. libgrace/include/grace/fused_3l_cpu.h:84-221
* cp_l couple .................................... libgrace/include/grace/fused_3l_cpu.h:223-321
* reduces, FCRight2Left, layer chain ............. libgrace/src/fused_3l.cpp:890-1010
* EquivariantRMSNorm, InvariantLayerRMSNorm ...... libgrace/include/grace/fused_3l_cpu.h:335-444
* readout ........................................ libgrace/src/fused_3l.cpp:1300-1360
* bond force from dE/dx and dE/dY, virial ........ libgrace/src/fused_3l.cpp:1030-1047, :117-123
* UQ head (uqv6, gamma only): basis blocks ....... libgrace/src/fused_3l.cpp:845-866, :1156-1201 (uq_layer),
  GMM ............................................ libgrace/include/grace/fused_cpu.h:1385-1416 (uq_gmm)

Pinning status: there is no GRACE-3L model file, golden vector or fixture in the reference checkout (its 3L tests
need a registry model that is downloaded), so this oracle is pinned against the COMPILED REFERENCE (oracle/_ref) on
generated random-weight models (energy, per-atom energies, forces, virial, at the reference's fp32 + spline
accuracy), by finite differences of the energy, and by rotation / translation / permutation invariance.  The UQ head
(uq_block, uq): against the compiled reference on a generated head (cluster indices exactly, gamma and sigma to 1e-4:
the reference projects in fp32), live and as committed goldens, and by what the definition fixes (tests/test_uq.py).
"""
from __future__ import annotations

import numpy as np
import torch

from .grace_oracle import ZeroBondError, _scalar, load_npz, real_sh

__all__ = ["Model3L", "compute_3l"]

_T = lambda a: torch.as_tensor(np.ascontiguousarray(a), dtype=torch.float64)
_I = lambda a: torch.as_tensor(np.ascontiguousarray(a).astype(np.int64).ravel())


def _names(d, key):
    return [x.decode() if isinstance(x, bytes) else str(x) for x in np.atleast_1d(d[key])] if key in d else []


class _SH(torch.autograd.Function):
    """Y_lm(u) with the gradient of the polynomial extension: fused_cpu.h:686-798."""

    @staticmethod
    def forward(ctx, u, lmax):
        Y, G = real_sh(u.detach().numpy(), lmax)
        ctx.save_for_backward(_T(G))
        return _T(Y)

    @staticmethod
    def backward(ctx, gY):
        (G,) = ctx.saved_tensors
        return torch.einsum("bq,bqd->bd", gY, G), None


class _Contract:
    """out[a, dst_c, k] += sum_n W[(mu_a,) k, n, tile_c] X[a, src_c, n] norm.  fused_3l_cpu.h:84-221."""

    def __init__(self, W, norm, src, dst, tile, elem):
        self.W = _T(W) * float(norm)
        self.src, self.dst, self.tile, self.elem = _I(src), _I(dst), _I(tile), elem

    def apply(self, X, out, mu):
        if self.src.numel() == 0:
            return out
        if self.elem:
            Wc = self.W[:, :, :, self.tile][mu]                       # [a, k, n, c]
            v = torch.einsum("aknc,acn->ack", Wc, X[:, self.src, :])
        else:
            Wc = self.W[:, :, self.tile]                              # [k, n, c]
            v = torch.einsum("knc,acn->ack", Wc, X[:, self.src, :])
        return out.index_add(1, self.dst, v)


class _Reduce:
    def __init__(self, d, name, n_elements):
        self.name = name
        self.n_out = int(_scalar(d, name + "_n_out"))
        self.n_funcs = int(_scalar(d, name + "_n_funcs"))
        self.only_invar = bool(_scalar(d, name + "_only_invar", 0))
        self.elem = bool(_scalar(d, name + "_is_central_atom_type_dependent", 0))
        self.nfo = 1 if self.only_invar else self.n_funcs
        self.inputs = _names(d, name + "_instruction_names")
        self.ins = []
        for cn in self.inputs:
            ci = d[f"{name}_collect_ind_{cn}"]
            dst = np.zeros_like(ci) if self.only_invar else d[f"{name}_total_sum_ind_{cn}"]
            self.ins.append(_Contract(d[f"{name}_reduce_{cn}_W"], _scalar(d, f"{name}_reduce_{cn}_norm", 1.0), ci, dst,
                                      d[f"{name}_w_l_tile_{cn}"], self.elem))
        self.norm_map = _T(d[name + "_norm_map"]).reshape(-1) if name + "_norm_map" in d else None

    def apply(self, T, mu):
        na = mu.numel()
        out = torch.zeros((na, self.nfo, self.n_out), dtype=torch.float64)
        for cn, c in zip(self.inputs, self.ins):
            out = c.apply(T[cn], out, mu)
        if self.norm_map is not None:
            out = out * self.norm_map[None, :, None]
        return out


class _CPL:
    """cp_l: Lp = norm_u U[g(f)] X_left[f], Rp = norm_v V[g(f)] X_right[f], out[o] = sum_t cg Lp[l_t] Rp[r_t]."""

    def __init__(self, d, name):
        self.U = _T(d[name + "_U"]) * float(_scalar(d, name + "_norm_u", 1.0))     # [g, rank, n_left]
        self.V = _T(d[name + "_V"]) * float(_scalar(d, name + "_norm_v", 1.0))
        self.gl, self.gr = _I(d[name + "_group_left"]), _I(d[name + "_group_right"])
        self.li, self.ri, self.oi = _I(d[name + "_left_ind"]), _I(d[name + "_right_ind"]), _I(d[name + "_m_sum_ind"])
        self.cg = _T(d[name + "_cg"]).reshape(-1)
        self.nfunc = int(_scalar(d, name + "_nfunc"))
        self.rank = int(_scalar(d, name + "_rank"))

    def apply(self, XL, XR):
        Lp = torch.einsum("fkn,afn->afk", self.U[self.gl], XL)
        Rp = torch.einsum("fkn,afn->afk", self.V[self.gr], XR)
        out = torch.zeros((XL.shape[0], self.nfunc, self.rank), dtype=torch.float64)
        return out.index_add(1, self.oi, self.cg[None, :, None] * Lp[:, self.li, :] * Rp[:, self.ri, :])


class _FC:
    """FCRight2Left with left_coefs = 0: out[f] = nof[f] (left[f] + sum_conn W[tile]^T right[from])."""

    def __init__(self, d, name):
        p = "fc_" + name
        if int(_scalar(d, p + "_left_coefs", 0)):
            raise ValueError("FC " + name + ": left_coefs = 1 is not a GRACE-3L export")
        self.nof = _T(d[p + "_norm_out_factor"]).reshape(-1)
        self.right = _Contract(d[p + "_w_right"], _scalar(d, p + "_norm_right", 1.0), d[p + "_collect_from"],
                               d[p + "_collect_to"], d[p + "_w_tile_right"], False)

    def apply(self, left, right):
        return self.right.apply(right, left, None) * self.nof[None, :, None]


class Model3L:
    """kokkos.npz of a GRACE-3L model as the reference engine resolves it by name."""

    def __init__(self, path_or_dict):
        d = load_npz(path_or_dict) if isinstance(path_or_dict, str) else path_or_dict
        self.d = d
        self.n_elements = int(_scalar(d, "n_elements"))
        self.ne = int(_scalar(d, "embedding_size", 64))
        self.nrb = int(_scalar(d, "nradbase", 10))
        self.lmax = int(_scalar(d, "lmax", _scalar(d, "A1_lmax", 4)))
        self.nl = self.lmax + 1
        self.nlm = self.nl ** 2
        self.rcut = float(_scalar(d, "rcut", 6.0))
        self.cut = np.full((self.n_elements, self.n_elements), self.rcut)
        if "bond_cutoff_map" in d and int(_scalar(d, "has_bond_specific_cutoff", 0)):
            self.cut = np.asarray(d["bond_cutoff_map"], dtype=np.float64).reshape(self.n_elements, self.n_elements)
        self.emb = _T(d["chem_embedding"])
        self.shift = _T(d["shift_values"]).reshape(-1)
        self.oscale = float(_scalar(d, "output_scale", 1.0))
        self.layers = []
        for k in (1, 2, 3):
            K = f"A{k}"
            L = {"K": K, "equiv": bool(_scalar(d, K + "_equivariant", 0)), "C": int(_scalar(d, K + "_n_rad_max")),
                 "p": int(_scalar(d, K + "_p", 5)), "inv_avg": float(_scalar(d, K + "_inv_avg_n_neigh", 1.0)),
                 "lt": _I(d[K + "_l_tile"])}
            nlay = int(_scalar(d, K + "_mlp_n_layers"))
            L["mlp"] = [(_T(d[f"{K}_mlp_W{i}"]), float(_scalar(d, f"{K}_mlp_norm{i}", 1.0)),
                         _T(d[f"{K}_mlp_b{i}"]).reshape(-1) if f"{K}_mlp_b{i}" in d else None) for i in range(nlay)]
            if not L["equiv"]:
                ztr = self.emb @ _T(d[K + "_lin_transform_W"]) * float(_scalar(d, K + "_lin_transform_norm", 1.0))
                L["fac"] = ztr * L["inv_avg"]
            else:
                L["fac"] = torch.full((self.n_elements, L["C"]), L["inv_avg"], dtype=torch.float64)
                L["zproj"] = self.emb @ _T(d[K + "_chem_linear_W"]) * float(_scalar(d, K + "_chem_linear_norm", 1.0))
                L["mask"] = _T(d[K + "_chem_l0_mask"]).reshape(-1)
                L["nlmi"] = int(_scalar(d, K + "_n_lm_ind"))
                L["cgW"] = _T(d[K + "_cg_W"])                                     # [nlm * nlmi, nfunc]
                L["redA"] = _Reduce(d, K + "_red", self.n_elements)
            for q in ("2", "3", "4"):
                L["p" + q] = _CPL(d, f"{K}_{q}")
                L["r" + q] = _Reduce(d, f"{K}_{q}_red", self.n_elements)
            L["fa"], L["fb"] = _FC(d, K + "_2a"), _FC(d, K + "_2b")
            if k < 3:
                L["eq"] = _Reduce(d, f"eq{k}", self.n_elements)
                e = f"eq{k}_norm"
                L["eqn"] = {"aff": _T(d[e + "_affine_weight"]), "dw": _T(d[e + "_degree_weights"]).reshape(-1),
                            "mask": _T(d[e + "_l0_mask"]).reshape(-1), "e": _I(d[e + "_expand_index"]),
                            "eps": float(_scalar(d, e + "_eps", 1e-8)), "center": bool(_scalar(d, e + "_center_l0", 1))}
            L["rho"] = _Reduce(d, f"rho{k}", self.n_elements)
            r = f"rho{k}_norm"
            L["rhon"] = {"scale": _T(d[r + "_scale"]).reshape(-1), "type": int(_scalar(d, r + "_type", 0))}
            self.layers.append(L)
        nlay = int(_scalar(d, "energy_mlp_n_layers"))
        self.emlp = [(_T(d[f"energy_mlp_W{i}"]), float(_scalar(d, f"energy_mlp_norm{i}", 1.0))) for i in range(nlay)]
        self.eact = int(_scalar(d, "energy_mlp_activation", 0))
        # the uqv6 UQ head (libgrace/src/uq_head.cpp:11-76, model_3l.cpp:453-463)
        self.has_uq = int(_scalar(d, "uq_schema_version", 0)) == 6
        if self.has_uq:
            ne = self.n_elements
            self.uq_rp, self.uq_D, self.uq_K = int(_scalar(d, "uq_rp_dim")), int(_scalar(d, "uq_feature_dim")), int(_scalar(d, "uq_max_clusters"))
            self.uq_scale = float(_scalar(d, "uq_rp_density_scale", 1.0))
            self.uq_R = np.asarray(d["uq_rp_matrix"], dtype=np.float64).reshape(-1, self.uq_rp)
            self.uq_cen = np.asarray(d["uq_centroids"], dtype=np.float64).reshape(ne, self.uq_K, self.uq_D)
            self.uq_icov = np.asarray(d["uq_inv_cov"], dtype=np.float64).reshape(ne, self.uq_K, self.uq_D, self.uq_D)
            self.uq_ncl = np.asarray(d["uq_n_clusters"]).astype(np.int64).ravel()
            self.uq_thr = np.asarray(d["uq_interp_thresholds"], dtype=np.float64).reshape(ne, self.uq_K)

    def uq_block(self, L, T):
        """the rows of one layer's basis block: the inputs of its rho reduce in the model's instruction order, per input
        channel-outer and collected-function-inner (libgrace/src/fused_3l.cpp:1167-1181)"""
        parts = []
        for cn, c in zip(L["rho"].inputs, L["rho"].ins):
            X = T[cn].detach().numpy()[:, np.asarray(self.d[f"{L['rho'].name}_collect_ind_{cn}"]).astype(np.int64).ravel(), :]
            parts.append(np.transpose(X, (0, 2, 1)).reshape(X.shape[0], -1))
        return np.concatenate(parts, axis=1)

    def uq(self, mu, blocks):
        """phi = ((B / |B|) R, log |B|, log |B_rho1|, log |B_rho2|, log |B_rho3|) density_scale (the first uq_D - uq_rp
        density channels), nearest centroid of the element (first of equal distances), sigma = sqrt(delta^T S delta +
        1e-8), gamma = sigma / max(threshold, 1e-10)  (fused_3l.cpp:1191-1199, fused_cpu.h:1385-1416)"""
        B = np.concatenate(blocks, axis=1)
        nrm = np.sqrt((B * B).sum(1))
        dens = [nrm] + [np.sqrt((b * b).sum(1)) for b in blocks]
        f = np.empty((B.shape[0], self.uq_D))
        f[:, :self.uq_rp] = (B @ self.uq_R) / (nrm + 1.0e-12)[:, None]
        for p in range(self.uq_D - self.uq_rp):
            f[:, self.uq_rp + p] = np.log(dens[p] + 1.0e-12) * self.uq_scale
        na = f.shape[0]
        gamma, sigma, cluster = np.zeros(na), np.zeros(na), np.zeros(na)
        for a in range(na):
            m = int(mu[a])
            d2 = ((f[a][None, :] - self.uq_cen[m, :self.uq_ncl[m]]) ** 2).sum(1)
            k = int(np.argmin(d2))
            dl = f[a] - self.uq_cen[m, k]
            sigma[a] = np.sqrt(dl @ self.uq_icov[m, k] @ dl + 1.0e-8)
            gamma[a] = sigma[a] / max(self.uq_thr[m, k], 1.0e-10)
            cluster[a] = k
        return gamma, sigma, cluster, f

    # ---- radial functions from the reference's tables (libgrace/src/fused_3l.cpp:491-533, evaluated as
    # spline_eval, libgrace/include/grace/fused_cpu.h:1052-1074), in fp64 (the reference stores fp32 coefficients): one table
    # per ordered pair of species and per layer, N_k intervals over x in [0, 1] (spline_n_3l, libgrace/include/grace/
    # system.h:95-103: spline / 2 for layers 1 and 2, at least 16; spline for layer 3), per interval the cubic through value
    # and derivative of the exact function at both ends.  self.spline = 0 (the default): the exact function.
    spline = 0

    def radial(self, L, x, mi, mj):
        if not self.spline:
            return self.radial_exact(L, x, mi, mj)
        k = self.layers.index(L)
        N = max(16, self.spline // 2) if k < 2 else self.spline
        R = torch.zeros((x.shape[0], self.nl, L["C"]), dtype=torch.float64)
        pairs = torch.unique(torch.stack([mi, mj], 1), dim=0) if x.shape[0] else []
        for a, b in [(int(p[0]), int(p[1])) for p in pairs]:
            key = (k, N, a, b)
            tabs = self.__dict__.setdefault("_tables", {})
            if key not in tabs:
                knots = torch.arange(N + 1, dtype=torch.float64) / N
                ia, ib = torch.full((N + 1,), a, dtype=torch.int64), torch.full((N + 1,), b, dtype=torch.int64)
                # every row of the exact function depends on its own x only: the tangent along (1, 1, ...) is d/dx row by row
                F, D = torch.func.jvp(lambda xx: self.radial_exact(L, xx, ia, ib), (knots,), (torch.ones_like(knots),))
                tabs[key] = (F.detach(), D.detach() / N)
            F, Dh = tabs[key]
            sel = torch.nonzero((mi == a) & (mj == b))[:, 0]
            sx = x[sel] * N
            kk = torch.clamp(sx.detach().to(torch.int64), 0, N - 1)
            t = (sx - kk)[:, None, None]
            f0, f1, d0, d1 = F[kk], F[kk + 1], Dh[kk], Dh[kk + 1]
            c2 = -3.0 * f0 - 2.0 * d0 + 3.0 * f1 - d1
            c3 = 2.0 * f0 + d0 - 2.0 * f1 + d1
            R = R.index_add(0, sel, f0 + t * (d0 + t * (c2 + t * c3)))
        return R

    # ---- radial functions R[b, l, c] of layer k: MLP([T_1..T_nrb(2x - 1), emb_i, emb_j]) env(x) fac[mu_j]
    def radial_exact(self, L, x, mi, mj):
        t = 2.0 * x - 1.0
        Tp, Tc, cols = torch.ones_like(t), t, []
        for _ in range(self.nrb):
            cols.append(Tc)
            Tp, Tc = Tc, 2.0 * t * Tc - Tp
        h = torch.cat([torch.stack(cols, 1), self.emb[mi], self.emb[mj]], 1)
        for i, (W, nrm, b) in enumerate(L["mlp"]):
            h = (h @ W) * nrm
            if i < len(L["mlp"]) - 1:
                if b is not None:
                    h = h + nrm * b
                h = h * torch.sigmoid(h)
        p = L["p"]
        env = 1.0 - 0.5 * (p + 1) * (p + 2) * x ** p + p * (p + 2) * x ** (p + 1) - 0.5 * p * (p + 1) * x ** (p + 2)
        R = h.reshape(-1, L["C"], self.nl).transpose(1, 2)                        # [b, l, c]
        return R * env[:, None, None] * L["fac"][mj][:, None, :]

    def chain(self, L, T, mu):
        """Layer chain after the SPBF: fused_3l.cpp:970-990; T holds the tensors by model name."""
        K = L["K"]
        X = T[K + "_red"] if L["equiv"] else T[K]
        T[K + "_2"] = L["p2"].apply(X, X)
        R2 = T[K + "_2_red"] = L["r2"].apply(T, mu)
        FA = L["fa"].apply(R2, X)
        T[K + "_3"] = L["p3"].apply(FA, X)
        T[K + "_3_red"] = L["r3"].apply(T, mu)
        FB = L["fb"].apply(R2, X)
        T[K + "_4"] = L["p4"].apply(FB, FB)
        T[K + "_4_red"] = L["r4"].apply(T, mu)
        I = None
        if "eq" in L:
            EQ = L["eq"].apply(T, mu)
            E = L["eqn"]
            C = EQ.shape[2]
            xc = EQ - (E["mask"][None, :, None] * EQ.mean(2, keepdim=True) if E["center"] else 0.0)
            S = (E["dw"][None, :, None] * xc * xc).sum((1, 2))
            r = 1.0 / torch.sqrt(S / C + E["eps"])
            I = xc * r[:, None, None] * E["aff"][E["e"]][None]
        rho = L["rho"].apply(T, mu)[:, 0, :]
        n0 = 1 if L["rhon"]["type"] == 1 else 0
        xs = rho[:, n0:]
        r = 1.0 / torch.sqrt((xs * xs).mean(1) + 1e-10)
        rn = torch.cat([rho[:, :n0], xs * r[:, None] * L["rhon"]["scale"][None]], 1)
        return I, rn

    def readout(self, h, mu):
        lin = h[:, 0]
        s = (h[:, 1:] @ self.emlp[0][0]) * self.emlp[0][1]
        act = torch.tanh(s) if self.eact == 1 else s * torch.sigmoid(s)
        e = (act @ self.emlp[1][0])[:, 0] * self.emlp[1][1]
        return (e + lin) * self.oscale + self.shift[mu]


def compute_3l(model: Model3L, mu, offset, j, rij, *, want_forces=True, bond_chunk=20000, debug=None, uq=False):
    """One GRACE-3L energy + forces + virial call on a CSR bond list (arguments and results as compute_1l).
    Driver skeleton: src/fused_3l.cpp:1550-1637; bond filter bonds.h:120-162.  `debug`: dict that receives the
    per-layer tensors (numpy) by model name."""
    mu_np = np.asarray(mu, dtype=np.int64)
    offset = np.asarray(offset, dtype=np.int64)
    j_np = np.asarray(j, dtype=np.int64)
    rij_np = np.asarray(rij, dtype=np.float64).reshape(-1, 3)
    n = mu_np.size
    bi = np.repeat(np.arange(n), np.diff(offset))
    rsq = (rij_np * rij_np).sum(1) if rij_np.size else np.zeros(0)
    rsq = rij_np[:, 0] * rij_np[:, 0] + rij_np[:, 1] * rij_np[:, 1] + rij_np[:, 2] * rij_np[:, 2]
    rc_np = model.cut[mu_np[bi], mu_np[j_np]]
    keep = rsq < rc_np * rc_np
    if np.any(keep & (rsq == 0.0)):
        q = np.nonzero(keep & (rsq == 0.0))[0][0]
        raise ZeroBondError(f"two atoms at the same position (a bond of length 0 between atoms {bi[q]} and "
                            f"{j_np[q]} of the neighbour list): not a physical structure")
    bi_t, bj_t = _I(bi[keep]), _I(j_np[keep])
    mu_t = _I(mu_np)
    d = _T(rij_np[keep]).requires_grad_(want_forces)
    rc = _T(rc_np[keep])
    r = torch.sqrt((d * d).sum(1))
    u = d / r[:, None]
    Y = _SH.apply(u, model.lmax)
    x = r / rc
    mi, mj = mu_t[bi_t], mu_t[bj_t]
    I_prev, h = None, 0.0
    uq_blocks = []
    if uq and not model.has_uq:
        raise ValueError("GRACE-3L: the model has no UQ head")
    for L in model.layers:
        R = model.radial(L, x, mi, mj)                                            # [b, l, c]
        Uy = Y[:, :, None] * R[:, L["lt"], :]                                     # [b, nlm, c]
        T = {}
        if not L["equiv"]:
            T[L["K"]] = torch.zeros((n, model.nlm, L["C"]), dtype=torch.float64).index_add(0, bi_t, Uy)
        else:
            nlmi = L["nlmi"]
            Mall = I_prev + L["mask"][None, :, None] * L["zproj"][mu_t][:, None, :]      # [n, nlmi, c]
            P = torch.zeros((n, model.nlm, nlmi, L["C"]), dtype=torch.float64)
            for b0 in range(0, bi_t.numel(), bond_chunk):
                sl = slice(b0, b0 + bond_chunk)
                P = P.index_add(0, bi_t[sl], Uy[sl][:, :, None, :] * Mall[bj_t[sl]][:, None, :, :])
            T[L["K"]] = torch.einsum("pf,apc->afc", L["cgW"], P.reshape(n, model.nlm * nlmi, L["C"]))
            T[L["K"] + "_red"] = L["redA"].apply(T, mu_t)
        I_prev, rn = model.chain(L, T, mu_t)
        h = h + rn
        if uq:
            uq_blocks.append(model.uq_block(L, T))
        if debug is not None:
            for key, v in T.items():
                debug[key] = v.detach().numpy()
            debug[L["K"] + "_R"] = R.detach().numpy()
            debug[L["K"] + "_rhon"] = rn.detach().numpy()
            if I_prev is not None:
                debug[L["K"] + "_I"] = I_prev.detach().numpy()
    E = model.readout(h, mu_t)
    out = {"energy": float(E.detach().sum()), "energies": E.detach().numpy().copy()}
    if uq:
        out["gamma"], out["atomic_sigma"], out["gmm_cluster"], out["uq_features"] = model.uq(mu_np, uq_blocks)
    if not want_forces:
        return out
    (g,) = torch.autograd.grad(E.sum(), d)
    g = g.numpy()
    forces = np.zeros((n, 3))
    np.add.at(forces, bi[keep], g)              # the force on i of bond (i, j) is dE/d r_ij (r_ij = x_j - x_i)
    np.add.at(forces, j_np[keep], -g)
    dl = -rij_np[keep]
    out["forces"] = forces
    out["virial"] = np.array([(dl[:, 0] * g[:, 0]).sum(), (dl[:, 1] * g[:, 1]).sum(), (dl[:, 2] * g[:, 2]).sum(),
                              (dl[:, 0] * g[:, 1]).sum(), (dl[:, 0] * g[:, 2]).sum(), (dl[:, 1] * g[:, 2]).sum()])
    # per-atom virials: half of each bond's (x_i - x_j) (x) f_i to each of its atoms (add_vatom, libgrace/include/grace/
    # fused_cpu.h:1075-1087, called per layer in src/fused_3l.cpp:1424; the halves are linear in the bond force, so the
    # total bond force g gives the sum over the layers)
    v6 = 0.5 * np.stack([dl[:, 0] * g[:, 0], dl[:, 1] * g[:, 1], dl[:, 2] * g[:, 2], dl[:, 0] * g[:, 1], dl[:, 0] * g[:, 2],
                         dl[:, 1] * g[:, 2]], axis=1)
    virials = np.zeros((n, 6))
    np.add.at(virials, bi[keep], v6)
    np.add.at(virials, j_np[keep], v6)
    out["virials"] = virials
    return out
