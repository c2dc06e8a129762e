"""The generated product kernels (grace_runtime_amd/csrc/jit_prod.hpp) compiled for the host and compared with a direct
evaluation of their term lists: forward values and both operand adjoints, overwrite and accumulate, for the
block-structured generator of the long cp_l couples (reference behaviour: couple_row_fwd / couple_row_bwd,
libgrace/include/grace/fused_3l_cpu.h:232-276) and for the all-in-registers generator of the shorter products.  The
source is the text the engine hands to hiprtc; here the launch bookkeeping is defined away and the column loop runs on
the CPU."""
import ctypes
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

HOST_PREFIX = """
#define __global__
#define __launch_bounds__(x)
struct D3 { unsigned x; };
static D3 blockIdx, blockDim, threadIdx;
"""
HOST_SUFFIX = """
extern "C" void run_fwd(const T *L, const T *R, T *O, int natoms)
{
  blockDim.x = 1; threadIdx.x = 0;
  for (unsigned c = 0; c < (unsigned) natoms * C; c++) { blockIdx.x = c; prod_fwd(L, R, O, natoms, 1); }
}
extern "C" void run_bwd(const T *L, const T *R, const T *G, T *gL, T *gR, int accL, int accR, int natoms)
{
  blockDim.x = 1; threadIdx.x = 0;
  for (unsigned c = 0; c < (unsigned) natoms * C; c++) { blockIdx.x = c; prod_bwd(L, R, G, gL, gR, accL, accR, natoms, 1); }
}
"""


def jit_source_exe():
    exe = os.path.join(ROOT, "tests", "build", "jit_source")
    srcs = [os.path.join(ROOT, "tests", "jit_source.cpp"), os.path.join(ROOT, "grace_runtime_amd", "csrc", "jit_prod.hpp")]
    if not os.path.exists(exe) or any(os.path.getmtime(exe) < os.path.getmtime(s) for s in srcs):
        sys.path.insert(0, ROOT)
        import __graft_entry__
        exe = __graft_entry__.build_jit_source()
    return exe


def host_library(tmp_path, kind, terms, group_l, group_r, nout, channels, precision):
    """generated source of the term list -> shared library with run_fwd / run_bwd"""
    l, r, o, c = terms
    tf = tmp_path / "terms.txt"
    with open(tf, "w") as f:
        f.write(f"{len(l)} {len(group_l)} {len(group_r)} {nout}\n")
        f.write(" ".join(str(int(g)) for g in group_l) + "\n" + " ".join(str(int(g)) for g in group_r) + "\n")
        for t in range(len(l)):
            f.write(f"{int(l[t])} {int(r[t])} {int(o[t])} {float(c[t])!r}\n")
    res = subprocess.run([jit_source_exe(), kind, str(tf), str(channels), str(precision)], capture_output=True, text=True)
    if res.returncode != 0:
        return None
    # the empty asm statements with register constraints of the GPU are barriers for its compiler only
    body = "\n".join(line for line in res.stdout.splitlines() if '"+v"' not in line)
    cpp = tmp_path / "gen.cpp"
    cpp.write_text(HOST_PREFIX + body + HOST_SUFFIX)
    so = tmp_path / "gen.so"
    subprocess.run(["g++", "-O0", "-shared", "-fPIC", "-ffp-contract=off", str(cpp), "-o", str(so)], check=True)
    return ctypes.CDLL(str(so))


def direct(terms, L, R, G, nout):
    """out[a][o][k] = sum_t c L[a][l][k] R[a][r][k] and the adjoints of L and R for the output adjoint G (float64)"""
    l, r, o, c = terms
    out = np.zeros((L.shape[0], nout, L.shape[2]))
    gL = np.zeros(L.shape)
    gR = np.zeros(R.shape)
    for t in range(len(l)):
        out[:, o[t]] += c[t] * L[:, l[t]] * R[:, r[t]]
        gL[:, l[t]] += c[t] * G[:, o[t]] * R[:, r[t]]
        gR[:, r[t]] += c[t] * G[:, o[t]] * L[:, l[t]]
    return out, gL, gR


def run_case(tmp_path, kind, terms, group_l, group_r, nout, precision, channels=4, natoms=3, seed=1):
    lib = host_library(tmp_path, kind, terms, group_l, group_r, nout, channels, precision)
    assert lib is not None, "the generator refused the term list"
    dt = np.float64 if precision == 64 else np.float32
    tol = 1e-12 if precision == 64 else 2e-5
    rng = np.random.default_rng(seed)
    nfl, nfr = len(group_l), len(group_r)
    L = rng.standard_normal((natoms, nfl, channels)).astype(dt)
    R = rng.standard_normal((natoms, nfr, channels)).astype(dt)
    G = rng.standard_normal((natoms, nout, channels)).astype(dt)
    ref_out, ref_gL, ref_gR = direct(terms, L.astype(np.float64), R.astype(np.float64), G.astype(np.float64), nout)
    ptr = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    out = np.full((natoms, nout, channels), np.nan, dt)
    lib.run_fwd(ptr(L), ptr(R), ptr(out), natoms)
    scale = max(1.0, np.abs(ref_out).max())
    if kind == "blocked":
        assert np.abs(out - ref_out).max() < tol * scale       # every output row written, outputs without terms are zero
    else:                                                       # outputs without terms are not live: never written
        live = np.zeros(nout, bool)
        live[terms[2]] = True
        assert np.abs(out[:, live] - ref_out[:, live]).max() < tol * scale
        assert np.isnan(out[:, ~live]).all()
    for acc in ((0, 1) if kind == "blocked" else (1,)):        # the engines run the register generator accumulating only
        gL = rng.standard_normal(L.shape).astype(dt) if acc else np.full(L.shape, np.nan, dt)
        gR = rng.standard_normal(R.shape).astype(dt) if acc else np.full(R.shape, np.nan, dt)
        exp_gL = ref_gL + (gL if acc else 0.0)
        exp_gR = ref_gR + (gR if acc else 0.0)
        lib.run_bwd(ptr(L), ptr(R), ptr(G), ptr(gL), ptr(gR), acc, acc, natoms)
        scale = max(1.0, np.abs(ref_gL).max(), np.abs(ref_gR).max())
        assert np.abs(gL - exp_gL).max() < tol * scale
        assert np.abs(gR - exp_gR).max() < tol * scale


def couple_terms(model, name):
    return (model[name + "_left_ind"], model[name + "_right_ind"], model[name + "_m_sum_ind"], model[name + "_cg"])


@pytest.fixture(scope="module")
def model4():
    from grace_runtime_amd import workloads
    return workloads.model_config4()


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("name", ["A1_3", "A2_2"])
def test_blocked_couple_of_the_benchmark_model(tmp_path, model4, name, precision):
    d = model4
    run_case(tmp_path, "blocked", couple_terms(d, name), d[name + "_group_left"], d[name + "_group_right"], int(d[name + "_nfunc"][0]), precision)


def synthetic_blocks(seed):
    """3 left and 2 right groups of uneven sizes; a left function no term uses, a right function no term uses, outputs
    without terms; every output inside one block"""
    rng = np.random.default_rng(seed)
    group_l = [0, 0, 0, 1, 2, 2, 2, 2, 2, 1]          # function 9 (group 1) stays unused
    group_r = [0, 0, 1, 1, 1, 0]                      # function 5 (group 0) stays unused
    lf = {g: [f for f in range(9) if group_l[f] == g] for g in range(3)}
    rf = {g: [f for f in range(5) if group_r[f] == g] for g in range(2)}
    l, r, o, c = [], [], [], []
    nout = 0
    for a in (2, 0, 1):
        for b in (1, 0):
            if (a, b) == (1, 1):
                continue                               # a pair of groups that does not couple
            for _ in range(4):
                nout += 1 if rng.random() < 0.3 else 0  # an output without terms now and then
                for _ in range(int(rng.integers(1, 6))):
                    l.append(int(rng.choice(lf[a]))); r.append(int(rng.choice(rf[b]))); o.append(nout); c.append(float(rng.standard_normal()))
                nout += 1
    return (np.array(l), np.array(r), np.array(o), np.array(c)), group_l, group_r, nout + 1


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_blocked_generator_on_ragged_blocks(tmp_path, seed, precision):
    terms, gl, gr, nout = synthetic_blocks(seed)
    run_case(tmp_path, "blocked", terms, gl, gr, nout, precision, channels=3, natoms=2, seed=seed)


def test_blocked_generator_refuses_an_output_fed_by_two_blocks(tmp_path):
    terms = (np.array([0, 1]), np.array([0, 1]), np.array([0, 0]), np.array([1.0, 2.0]))
    assert host_library(tmp_path, "blocked", terms, [0, 1], [0, 1], 1, 4, 64) is None


@pytest.mark.parametrize("precision", [64, 32])
def test_register_generator_on_a_short_couple(tmp_path, model4, precision):
    """the generator of the products with few functions: operands of both sides in registers"""
    d = model4
    l, r, o, c = couple_terms(d, "A1_2")
    keep = (l < 16) & (r < 16)                         # the l <= 3 part: 16 functions a side
    sel = (l[keep], r[keep], o[keep], c[keep])
    run_case(tmp_path, "plain", sel, [0] * 16, [0] * 16, int(d["A1_2_nfunc"][0]), precision)
