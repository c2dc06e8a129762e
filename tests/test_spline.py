"""Radial tables of the oracles (grace_oracle.spline_radial): the reference's engines take the radial functions of a bond
from cubic tables (FusedSettings::spline_n = 1024, libgrace/include/grace/system.h:78; tables libgrace/src/fused_1l.cpp:
102-129, evaluation libgrace/include/grace/fused_cpu.h:1052-1074).  No GPU.  Pinned by what the construction fixes: the
table reproduces the MLP and its derivative at the knots, value and derivative are continuous across knots, the error
falls as the fourth power of the interval (the derivative's as the third), and a call with tables of 1024 intervals is
within the reference's gate of the call without."""
import numpy as np
import pytest

import cases
from oracle import grace_oracle as g1
from oracle import grace_oracle_2l as g2
from oracle import grace_oracle_3l as g3


def _models(model_dir):
    yield g1.Model1L(cases.model_file(model_dir, "mix2")), (lambda m, x: m.radial(x))
    m2 = g2.Model2L(cases.model_file(model_dir, "l2mix"))
    yield m2, (lambda m, x: m.radial(1, x))
    yield m2, (lambda m, x: m.radial(2, x))


def test_tables_reproduce_the_mlp_at_the_knots_and_converge_at_fourth_order(model_dir):
    rng = np.random.default_rng(0)
    x = np.sort(rng.uniform(0.02, 0.999, 4000))
    for m, rad in _models(model_dir):
        m.spline = 0
        R0, dR0 = rad(m, x)
        err, derr = {}, {}
        for N in (256, 1024):
            m.spline = N
            knots = np.arange(1, N) / N
            Rk, dRk = rad(m, knots)
            m.spline = 0
            Re, dRe = rad(m, knots)
            m.spline = N
            assert np.abs(Rk - Re).max() < 1e-13 * max(1.0, np.abs(Re).max())
            assert np.abs(dRk - dRe).max() < 1e-10 * max(1.0, np.abs(dRe).max())
            below, _ = rad(m, knots - 1e-12)                       # continuity across a knot
            assert np.abs(below - Rk).max() < 1e-9 * max(1.0, np.abs(Re).max())
            R, dR = rad(m, x)
            err[N], derr[N] = np.abs(R - R0).max(), np.abs(dR - dR0).max()
        m.spline = 0
        assert 120.0 < err[256] / err[1024] < 500.0            # 4^4 = 256
        assert 30.0 < derr[256] / derr[1024] < 130.0           # 4^3 = 64


@pytest.mark.parametrize("model,struct,rc", [("mix2", "alloy54", 5.0), ("l2mix", "alloy54", 5.0)])
def test_a_call_with_tables_is_within_the_gate_of_the_call_without(model_dir, gold, model, struct, rc):
    layers = cases.LAYERS[model]
    m = (g1.Model1L if layers == 1 else g2.Model2L)(cases.model_file(model_dir, model))
    compute = g1.compute_1l if layers == 1 else g2.compute_2l
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    tag = f"e2e/{model}/{struct}"
    key = f"nl/{struct}@{float(gold[tag + '/rc_list']):g}"
    perm, offset, j, image, shifts = (gold[f"{key}/{k}"] for k in ("perm", "offset", "j", "image", "shifts"))
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    exact = compute(m, types[perm] - 1, offset, j, rij)
    m.spline = 1024
    tab = compute(m, types[perm] - 1, offset, j, rij)
    m.spline = 0
    n = len(pos)
    assert 0 < abs(tab["energy"] - exact["energy"]) / n < 1e-7                         # gate: 1e-6 eV/atom
    assert np.abs(tab["forces"] - exact["forces"]).max() < 1e-5                         # the gate; 2.3e-6 on the 2L case
    assert np.abs(tab["virial"] - exact["virial"]).max() < 1e-5 * max(1.0, np.abs(exact["virial"]).max())
    # and as close to the compiled reference (fp32, tables of 1024 intervals) as the call without tables is
    ref_e = float(gold[tag + "/energy"])
    assert abs(tab["energy"] - ref_e) / n < 1e-6


def _radial_3l(m, k, x, a, b):
    """R [n, l, c] and dR/dx of layer k for bonds of the species pair (a, b) at reduced lengths x, from the 3L oracle"""
    import torch
    xt = torch.tensor(np.asarray(x, dtype=np.float64), requires_grad=True)
    mi, mj = torch.full((len(x),), a, dtype=torch.int64), torch.full((len(x),), b, dtype=torch.int64)
    R = m.radial(m.layers[k], xt, mi, mj)
    w = torch.tensor(np.random.default_rng(5).uniform(0.5, 1.5, tuple(R.shape[1:])))
    (g,) = torch.autograd.grad((R * w).sum(), xt)                   # one weighted sum of derivatives per bond
    return R.detach().numpy(), g.numpy()


def test_3l_tables_per_species_pair(model_dir):
    """GRACE-3L (libgrace/src/fused_3l.cpp:491-533): one table per ordered species pair and layer, spline / 2 intervals for
    layers 1 and 2 and spline for layer 3 (libgrace/include/grace/system.h:98-102).  Knot values and derivatives are the
    exact function's, the interval count per layer shows in where the knots are, pairs (a, b) and (b, a) have their own
    tables, the error falls as the fourth power."""
    m = g3.Model3L(cases.model_file(model_dir, "l3mix"))
    rng = np.random.default_rng(1)
    x = np.sort(rng.uniform(0.02, 0.999, 1500))
    for k in range(3):
        for a, b in ((0, 1), (1, 0), (1, 1)):
            m.spline = 0
            R0, g0 = _radial_3l(m, k, x, a, b)
            err = {}
            for S in (256, 1024):
                N = S if k == 2 else S // 2
                knots = np.arange(1, N) / N
                m.spline = 0
                Re, ge = _radial_3l(m, k, knots, a, b)
                m.spline = S
                Rk, gk = _radial_3l(m, k, knots, a, b)
                assert np.abs(Rk - Re).max() < 1e-13 * max(1.0, np.abs(Re).max())
                assert np.abs(gk - ge).max() < 1e-10 * max(1.0, np.abs(ge).max())
                below, _ = _radial_3l(m, k, knots - 1e-12, a, b)
                assert np.abs(below - Rk).max() < 1e-9 * max(1.0, np.abs(Re).max())
                R, _ = _radial_3l(m, k, x, a, b)
                err[S] = np.abs(R - R0).max()
                if k < 2:                                                # at the knots of a table of S intervals that are not
                    mid = (2 * np.arange(N) + 1) / S                     # knots of S / 2 the table differs from the function
                    Rm, _ = _radial_3l(m, k, mid, a, b)
                    m.spline = 0
                    Rme, _ = _radial_3l(m, k, mid, a, b)
                    assert np.abs(Rm - Rme).max() > 1e-14 * max(1.0, np.abs(Rme).max())
            m.spline = 0
            assert 120.0 < err[256] / err[1024] < 500.0
    m.spline = 1024                                                      # the two orders of a mixed pair differ
    Rab, _ = _radial_3l(m, 0, x[:50], 0, 1)
    Rba, _ = _radial_3l(m, 0, x[:50], 1, 0)
    assert np.abs(Rab - Rba).max() > 1e-6
    m.spline = 8                                                         # layers 1 and 2 never below 16 intervals
    R16, _ = _radial_3l(m, 0, np.arange(1, 16) / 16, 0, 1)
    m.spline = 0
    Re, _ = _radial_3l(m, 0, np.arange(1, 16) / 16, 0, 1)
    assert np.abs(R16 - Re).max() < 1e-13 * max(1.0, np.abs(Re).max())


def test_3l_call_with_tables_is_within_the_gate(model_dir, gold):
    m = g3.Model3L(cases.model_file(model_dir, "l3mix"))
    pos, cell, pbc, types = cases.structure_alloy54()
    tag = "e2e/l3mix/alloy54"
    key = f"nl/alloy54@{float(gold[tag + '/rc_list']):g}"
    perm, offset, j, image, shifts = (gold[f"{key}/{k}"] for k in ("perm", "offset", "j", "image", "shifts"))
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    exact = g3.compute_3l(m, types[perm] - 1, offset, j, rij)
    m.spline = 1024
    tab = g3.compute_3l(m, types[perm] - 1, offset, j, rij)
    m.spline = 0
    n = len(pos)
    assert 0 < abs(tab["energy"] - exact["energy"]) / n < 1e-6
    assert np.abs(tab["forces"] - exact["forces"]).max() < 1e-5 * max(1.0, np.abs(exact["forces"]).max())
    assert np.abs(tab["virial"] - exact["virial"]).max() < 1e-5 * max(1.0, np.abs(exact["virial"]).max())
    ref_e = float(gold[tag + "/energy"])                                 # the compiled reference: fp32 with its default tables
    assert abs(tab["energy"] - ref_e) / n < 1e-5
