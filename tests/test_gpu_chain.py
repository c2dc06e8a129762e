"""The fused dense chain of the GRACE-1L / 2L engines (grace_runtime_amd/csrc/jit_chain.hpp: A -> A1 -> AA -> AA1 / AA2 ->
AAA / AAAA as one generated kernel per direction; stage order of the reference, libgrace/src/fused_1l.cpp:260-349)
through the C ABI: against the CPU oracle, and against the same engine with the chain run stage by stage
(GRACE_HIP_CHAIN=0 at engine creation), for the model shapes the generator distinguishes: with and without the AAAA
stage, the legacy product AAA = AA1 x A, channel widths padded to 32, one and two elements, atom counts that do not fill
the last block of atoms, chunked passes, energy-only passes.  Needs an MI355X."""
import os

import numpy as np
import pytest

import cases
from grace_runtime_amd import kk
from oracle import grace_oracle as g1

pytestmark = pytest.mark.gpu

CASES = [("config1", "config1"), ("ch20", "alloy54"), ("ch3", "triclinic"), ("chleg", "alloy54"), ("ch20", "molecule")]


def _engine(path, species, precision, fused):
    old = os.environ.get("GRACE_HIP_CHAIN")
    os.environ["GRACE_HIP_CHAIN"] = "1" if fused else "0"
    try:
        return kk.Engine(kk.Model(path), species, precision)
    finally:
        if old is None:
            del os.environ["GRACE_HIP_CHAIN"]
        else:
            os.environ["GRACE_HIP_CHAIN"] = old


def _stages(eng):
    eng.set_profile(True)
    eng.run()
    names = set(eng.stage_times())
    eng.set_profile(False)
    return names


@pytest.mark.parametrize("precision", [64, 32])
@pytest.mark.parametrize("model,struct", CASES)
def test_fused_chain_equals_the_oracle_and_the_staged_chain(model_dir, model, struct, precision):
    path = cases.model_file(model_dir, model)
    om = g1.Model1L(path)
    species = [s.decode() for s in om.d["element_names"]]
    pos, cell, pbc, types = cases.STRUCTURES[struct]()
    types = np.minimum(types, om.n_elements).astype(np.int32)
    rc = float(np.max(om.cut))
    pcell, shift = kk._padded_cell_arrays(cell, pos, rc, pbc)
    perm, offset, j, image, shifts = kk.neighbor_search(pos + shift, pcell, pbc, rc)
    rij = cases.bond_vectors(pos, perm, offset, j, image, shifts)
    n = len(pos)
    ref = g1.compute_1l(om, types[perm] - 1, offset, j, rij)
    fused, staged = _engine(path, species, precision, True), _engine(path, species, precision, False)
    out = {}
    for tag, eng in (("fused", fused), ("staged", staged)):
        eng.upload(types[perm], offset, j, rij=rij)
        names = _stages(eng)
        assert ("chain_fwd" in names and "chain_bwd" in names and "fc_AA1" not in names) == (tag == "fused"), (tag, sorted(names))
        eng.run(energies=True)
        out[tag] = eng.fetch(energies=True)
    fs = max(1.0, np.abs(ref["forces"]).max())
    tol = (1e-10, 1e-9, 1e-9) if precision == 64 else (1e-6, 2e-5, 1e-5)
    for tag in ("fused", "staged"):
        o = out[tag]
        assert abs(o["energy"] - ref["energy"]) / n < tol[0] * fs, tag
        assert np.abs(o["forces"] - ref["forces"]).max() < tol[1] * fs, tag
        assert np.abs(o["energies"] - ref["energies"]).max() < tol[0] * fs, tag
        assert np.abs(o["virial"] - ref["virial"]).max() < tol[2] * max(1.0, np.abs(ref["virial"]).max()), tag
    # the two ways through the chain differ in summation order only
    same = 1e-11 if precision == 64 else 2e-5
    assert abs(out["fused"]["energy"] - out["staged"]["energy"]) / n < same * fs
    assert np.abs(out["fused"]["forces"] - out["staged"]["forces"]).max() < 10 * same * fs
    # energy-only pass and a pass in chunks that cut the blocks of atoms
    fused.run(energy_only=True)
    assert abs(fused.fetch()["energy"] - ref["energy"]) / n < tol[0] * fs
    fused.set_chunksize(13)
    fused.run(energies=True)
    o = fused.fetch(energies=True)
    assert fused.chunksize == 13
    assert abs(o["energy"] - ref["energy"]) / n < tol[0] * fs and np.abs(o["forces"] - ref["forces"]).max() < tol[1] * fs
    fused.close()
    staged.close()


def test_models_outside_the_generator_keep_the_staged_chain(model_dir):
    """channel widths other than 32 (the fixture models of the reference: 16; mix2: 32 and 64) run stage by stage"""
    for name, fixture, species in (("grace_1l_order3", True, ["Mo", "W"]), ("mix2", False, ["Mo", "W"])):
        path = os.path.join(cases.REF_FIXTURES, name + ".npz") if fixture else cases.model_file(model_dir, name)
        eng = kk.Engine(kk.Model(path), species, 64)
        pos, cell, pbc, types = cases.structure_alloy54()
        perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, 5.0)
        eng.upload(types[perm], offset, j, positions=pos[perm], image=image, shifts=shifts)
        names = _stages(eng)
        assert "chain_fwd" not in names and "fc_A1" in names
        eng.close()


def test_compiled_kernels_are_kept_on_disk_for_the_next_process(model_dir, tmp_path):
    """GRACE_HIP_CACHE: the first process compiles the generated kernels and leaves their code objects in the directory, the
    second one loads them (no compiler run: engine creation in a fraction of the time) and computes the same numbers"""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    path = cases.model_file(model_dir, "ch20")
    code = (
        "import sys, time, numpy as np\n"
        f"sys.path.insert(0, {root!r}); sys.path.insert(0, {os.path.join(root, 'tests')!r})\n"
        "import cases\n"
        "from grace_runtime_amd import kk\n"
        "t = time.perf_counter()\n"
        f"eng = kk.Engine(kk.Model({path!r}), ['Mo', 'W'], 64)\n"
        "dt = time.perf_counter() - t\n"
        "pos, cell, pbc, types = cases.structure_alloy54()\n"
        "perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, 5.0)\n"
        "out = eng.compute(types[perm], offset, j, positions=pos[perm], image=image, shifts=shifts)\n"
        "print(dt, repr(out['energy']), repr(float(np.abs(out['forces']).sum())))\n")
    env = dict(os.environ, GRACE_HIP_CACHE=str(tmp_path / "cache"))
    runs = []
    for _ in range(2):
        res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=300)
        assert res.returncode == 0, res.stderr
        runs.append(res.stdout.strip().split("\n")[-1].split())
    files = os.listdir(tmp_path / "cache")
    assert len(files) >= 3 and all(f.endswith(".co") for f in files)          # three products and the chain
    assert float(runs[1][0]) < 0.5 * float(runs[0][0])
    assert abs(float(runs[0][1]) - float(runs[1][1])) < 1e-9 * abs(float(runs[0][1]))
    assert abs(float(runs[0][2]) - float(runs[1][2])) < 1e-9 * abs(float(runs[0][2]))
    # a file that the driver does not load (cut short here) is dropped, its source compiled again and the file replaced
    sizes = {f: os.path.getsize(tmp_path / "cache" / f) for f in files}
    for f in files:
        with open(tmp_path / "cache" / f, "r+b") as fh:
            fh.truncate(200)
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=300)
    assert res.returncode == 0, res.stderr
    third = res.stdout.strip().split("\n")[-1].split()
    assert abs(float(third[1]) - float(runs[0][1])) < 1e-9 * abs(float(runs[0][1]))
    assert {f: os.path.getsize(tmp_path / "cache" / f) for f in os.listdir(tmp_path / "cache")} == sizes
    # switched off: nothing is written
    env0 = dict(os.environ, GRACE_HIP_CACHE="0", HOME=str(tmp_path / "home"))
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env0, timeout=300)
    assert res.returncode == 0, res.stderr
    assert not os.path.exists(tmp_path / "home" / ".cache" / "grace_hip")
