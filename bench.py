#!/usr/bin/env python3
"""Benchmark of the GRACE energy + forces + virial pass on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--precision 64|32] [--no-cpu] [--workload config2|config3|config4|config5]

Default workload (the second benchmark configuration, the one the metric is quoted on): GRACE-1L-shaped random-init model (lmax 4, 32 radial channels, 8 Chebyshev
functions, radial MLP 8-64-64-160, SiLU) on a bcc W 16x16x16 supercell (8192 atoms, a = 3.165 A, N(0, 0.05 A) jitter,
r_cut 6 A, 475 136 directed edges), fp64.  A step is one full pass (bond filter, radial MLP, A basis, dense chain,
readout, reverse pass, forces, virial) over the structure, which is uploaded to HBM before the timed region.

--workload config3 runs the third configuration instead: GRACE-2L-shaped model (two layers, lmax 4, 32 channels, two radial
MLPs 8-64-64-160, body order 3) on the 4-species fcc 20x20x20 alloy (32 000 atoms, ~2.5 M edges), fp64.
--workload config4 the fourth: GRACE-3L-shaped model (three layers, lmax 5, 64 channels, radial MLPs (8 + 2 x 32)-128-128-384,
89-species embedding table) on an amorphous cube of 10 000 atoms with 8 species (~0.72 M edges), fp64.
--workload config5 the fifth: the GRACE-2L-shaped model with 3 species over 512 independent periodic cells of 32 .. 128 atoms
(41 701 atoms, ~2.2 M edges) as ONE resident ragged batch; a step is one engine pass over all cells.

Timing: `value` / `ms_per_step` are the mean over the K timed passes (one synchronisation before and one after the K
passes); `median_ms_per_step` is the median of K passes timed one by one, the reference's protocol
(docs/benchmarks.md:13: median of the calls after the first).

Prints one JSON line: the metric (us/atom per call), the roofline of the dominant kernel (duration from HIP events
on the engine's stream, algorithmic flops/bytes of that stage) and the reference CPU path timed on this host.
"""
import argparse
import json
import os
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {64: 78.6, 32: 157.3}      # dense matrix TFLOP/s of MI355X (fp64, fp32)
HBM_PEAK = 8000.0                 # GB/s


# HBM bytes per launch of the dominant kernel measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs of this
# script, counters scaled by what they read for the 1 GiB copy kernel; summaries under profiles/): (workload, kernel)
MEASURED_TRAFFIC = {
    ("config2", "radial_mlp"): 14.3e6 + 1175.4e6,       # fetch + write of k_radial<double,4,0,0,true> (its launches on the full edge list)
    ("config3", "pair_bwd"): 10754.5e6 + 2764.4e6,      # fetch + write of k_pair_bwd_mfma<double,5,2>
    ("config4", "pair_bwd_L3"): 44870e6 + 31121e6,      # the layer-3 launches of k_pair_bwd_mfma<double,6,2> (layer 2: 24.5 + 15.6 GB)
    ("config5", "pair_bwd"): 8993.2e6 + 2467.7e6,       # fetch + write of k_pair_bwd_mfma<double,5,2> over the ragged batch
}
# the per-atom dense chain of configuration 2 (chain_fwd 0.72 GB, k_reduce_fwd 0.19, k_energy < 0.01, k_reduce_bwd 0.19, chain_bwd
# 0.79 GB: every launch between the A basis and the bond reverse), same counters
DENSE_TRAFFIC = {"config2": 1.90e9}
DENSE_PREFIXES = ("fc_", "prod_", "reduce_", "energy_mlp", "zero_grads", "chain_")


def stage_model(name, ms, E, N, C, nl, nlm, s, prec, dense_flops, nslot=5, nI=4, radial_flops=59392.0, slots=None, stream_bytes=None):
    """Roofline entry of one stage: algorithmic work / measured time."""
    base = name.rsplit("_L", 1)[0] if slots else name     # GRACE-3L stages carry their layer: pair_fwd_L2, radial_L1 ...
    if slots and base in ("pair_fwd", "pair_bwd"):
        nslot = nI = slots[name[-1]]
        name = base
    elif slots and base in ("scatter_A", "bond_bwd"):
        name = base
    elif slots and base == "radial":
        name = "radial_mlp"
    if name == "pair_fwd":
        # per edge: R1 row, Y, neighbour index, the neighbour's message rows; per atom: the pair tensor written once
        by = E * (s * C * nl + s * nlm + 4 + nslot * C * s) + N * nslot * nlm * C * s
        return {"bound": "hbm", "achieved": by / (ms * 1e-3) / 1e9, "peak": HBM_PEAK, "unit": "GB/s", "work": by}
    if name == "pair_bwd":
        # per edge: R1 and dR1 rows, Y and its two tangential gradients, neighbour rows, dE/dI rows read-modify-written,
        # geometry, forces
        by = E * (2 * s * C * nl + 3 * s * nlm + nslot * C * s + 2 * nI * C * s + 28 + 24) + N * (nslot * nlm * C * s + 24)
        return {"bound": "hbm", "achieved": by / (ms * 1e-3) / 1e9, "peak": HBM_PEAK, "unit": "GB/s", "work": by}
    if name in ("radial_mlp", "radial_R", "radial_R1") and radial_flops == 0.0:
        # radial tables: per edge x and the neighbour element read, one row of values and one of derivatives written
        by = E * (12 + 2 * s * C * nl)
        return {"bound": "hbm", "achieved": by / (ms * 1e-3) / 1e9, "peak": HBM_PEAK, "unit": "GB/s", "work": by}
    if name in ("radial_mlp", "radial_R", "radial_R1"):
        # value + tangent through the 3 layers: 2 * 2 * E * sum n_in n_out
        fl = radial_flops * E
        return {"bound": "mfma", "achieved": fl / (ms * 1e-3) / 1e12, "peak": PEAK[prec], "unit": "TFLOP/s", "work": fl}
    if name == "scatter_A":
        by = E * (s * C * nl + 4 + 24) + N * s * C * nlm
        return {"bound": "hbm", "achieved": by / (ms * 1e-3) / 1e9, "peak": HBM_PEAK, "unit": "GB/s", "work": by}
    if name == "bond_bwd":
        by = E * (2 * s * C * nl + 28 + 24) + N * (s * C * nlm + 24)
        return {"bound": "hbm", "achieved": by / (ms * 1e-3) / 1e9, "peak": HBM_PEAK, "unit": "GB/s", "work": by}
    if name in dense_flops:
        fl = dense_flops[name]
        return {"bound": "mfma", "achieved": fl / (ms * 1e-3) / 1e12, "peak": PEAK[prec], "unit": "TFLOP/s", "work": fl}
    if stream_bytes and name in stream_bytes:
        by = stream_bytes[name]
        return {"bound": "hbm", "achieved": by / (ms * 1e-3) / 1e9, "peak": HBM_PEAK, "unit": "GB/s", "work": by}
    return None


def couple_stream_bytes(md, N, s):
    """Algorithmic bytes of the cp_l couples and of the sparse Clebsch-Gordan map of a GRACE-3L model, per stage name:
    every operand row, output row and adjoint row once (forward: both projections in, the product out; reverse: the
    projections and the product's adjoint in, both projection adjoints out)."""
    out = {}
    for layer in (1, 2, 3):
        for q in ("2", "3", "4"):
            P = f"A{layer}_{q}"
            nfl, nfr, nout, rank = len(md[P + "_group_left"]), len(md[P + "_group_right"]), int(md[P + "_nfunc"][0]), int(md[P + "_rank"][0])
            out[f"couple_{q}_L{layer}"] = N * rank * s * (nfl + nfr + nout)
            out[f"couple_{q}_bwd_L{layer}"] = N * rank * s * (nfl + nfr + nout + nfl + nfr)
        if layer > 1:
            npair, nfa = md[f"A{layer}_cg_W"].shape
            width = int(md[f"A{layer}_n_rad_max"][0])
            out[f"couple_YI_L{layer}"] = out[f"couple_YI_bwd_L{layer}"] = N * width * s * (npair + nfa)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--precision", type=int, default=64, choices=[64, 32])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--workload", default="config2", choices=["config2", "config3", "config4", "config5", "sizes"])
    ap.add_argument("--reps", type=int, default=0, help="supercell repetitions (default: 16 bcc cells / 20 fcc cells per edge)")
    ap.add_argument("--atoms", type=int, default=10000, help="atoms of the amorphous cube of config4")
    ap.add_argument("--spline", type=int, default=0, help="intervals of the radial tables of the GRACE-1L / 2L engines (the reference's engines "
                                                            "use 1024); 0: the radial MLP is evaluated for every bond")
    ap.add_argument("--chunksize", type=int, default=-1, help="atoms per engine pass: -1 chosen from the free device memory (one pass when "
                                                              "the structure fits), 0 one pass, > 0 fixed")
    ap.add_argument("--no-others", action="store_true", help="default workload only: skip the short runs of configurations 3, 4 and 5 "
                                                             "that the default run reports under other_workloads")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (no collectives in the path); run with --gpus 1")
    if a.workload == "sizes":
        print(json.dumps(run_sizes(a)))
        return
    res = run_workload(a)
    if a.workload == "config2" and a.precision == 64 and not a.no_others and a.reps == 0 and a.spline == 0 and a.chunksize == -1:
        # the other benchmark configurations, a few steps each, in the same run (the same code path as --workload <name>)
        others = {}
        for w in ("config3", "config4", "config5"):
            for prec in (64, 32):
                b = argparse.Namespace(**vars(a))
                b.workload, b.precision, b.steps, b.warmup = w, prec, 5, 1
                b.no_cpu = a.no_cpu or prec == 32
                r = run_workload(b, light=True)
                key = w if prec == 64 else w + "_fp32"
                others[key] = {"value": r["value"], "unit": r["unit"], "ms_per_step": r["ms_per_step"], "dtype": r["dtype"], "steps": r["steps"],
                               "atoms": r["config"]["atoms"], "edges": r["config"]["edges"], "workload": r["config"]["workload"],
                               "ms_per_calculator_call": r["ms_per_calculator_call"],
                               "ms_per_step_radial_tables_1024": r["ms_per_step_radial_tables_1024"],
                               "roofline": {k: r["roofline"][k] for k in ("kernel", "bound", "achieved", "peak", "unit", "frac", "avg_ms", "traffic")},
                               "stages_ms": r["stages_ms"], "engine_create_s": r["engine_create_s"], "device_memory_GB": r["device_memory_GB"],
                               "cpu_baseline": r["cpu_baseline"]}
        res["other_workloads"] = others
        # us/atom of the calculator-level call from 128 to 65 536 atoms (GRACE-1L; --workload sizes goes on to millions)
        res["size_range"] = [{k: e[k] for k in ("structure", "atoms", "edges", "ms_per_call_list_kept", "us_per_atom", "device_memory_GB")}
                             for e in run_sizes(a, short=True)["entries"]]
    print(json.dumps(res))


def run_sizes(a, short=False):
    """The calculator-level call (kk.System.compute: positions in, device neighbour list kept between calls, results out; the
    reference's protocol, docs/benchmarks.md:9-20) over a range of structure sizes: the GRACE-1L model from 128 atoms to a
    bcc 128^3 supercell, and one structure per model kind well past the benchmark size, evaluated in the chunks the engine
    chooses from the free device memory (the reference's "largest system" column, docs/benchmarks.md:17, is the same
    mechanism pushed to the limit of a 64 GB device; here the sizes are fixed and chosen to fit).  Prints atoms, bonds per
    atom, ms per call, us/atom, atoms per engine pass and the device memory the library holds."""
    import torch

    from grace_runtime_amd import kk, synth, workloads
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    tmp = tempfile.mkdtemp()
    pbc = [True, True, True]
    out = []

    def measure(label, model, species, types, pos, cell, calls):
        t0 = time.perf_counter()
        sysm = kk.System(model, species, skin=0.5, precision=a.precision)
        create_s = time.perf_counter() - t0
        t0 = time.perf_counter()
        r = sysm.compute(types, pos, cell, pbc)
        first_s = time.perf_counter() - t0
        ts = []
        for _ in range(calls):
            t0 = time.perf_counter()
            r = sysm.compute(types, pos, cell, pbc)
            ts.append(time.perf_counter() - t0)
        n = len(pos)
        ms = float(np.median(ts)) * 1e3
        e = {"structure": label, "atoms": n, "edges": int(sysm.engine.edge_count()), "ms_per_call_list_kept": round(ms, 3),
             "us_per_atom": round(ms * 1e3 / n, 5), "first_call_s_with_list_build": round(first_s, 3), "atoms_per_engine_pass": sysm.chunksize or n,
             "device_memory_GB": round(kk.memory_in_use() / 1e9, 3), "engine_create_s": round(create_s, 2), "energy_per_atom": r["energy"] / n,
             "net_force": float(np.abs(r["forces"].sum(0)).max())}
        print(json.dumps(e), file=sys.stderr, flush=True)
        out.append(e)
        del sysm

    m1 = kk.Model(workloads.write_model("config1", tmp))
    for reps in ((4, 8, 10, 16, 32) if short else (4, 8, 10, 16, 32, 64, 128)):
        pos, cell = synth.bcc_supercell(3.165, reps)
        pos = synth.jitter(pos, 0.05, 2)
        measure(f"GRACE-1L, bcc W {reps}^3", m1, ["W"], np.ones(len(pos), np.int32), pos, cell, 5 if reps <= 32 else 3)
    if short:    # the default run: the GRACE-1L sizes from 128 to 65 536 atoms only
        return {"workload": "size range, calculator-level call with the neighbour list kept", "dtype": "f64" if a.precision == 64 else "f32", "entries": out}
    m2 = kk.Model(workloads.write_model("config3", tmp))
    pos, cell = synth.fcc_supercell(3.6, 63)
    pos = synth.jitter(pos, 0.08, 3)
    measure("GRACE-2L, 4-species fcc alloy 63^3", m2, ["Al", "Co", "Ni", "Ti"], np.random.default_rng(3).integers(1, 5, size=len(pos)).astype(np.int32),
            pos, cell, 3)
    mp = workloads.write_model("config4", tmp)
    with np.load(mp) as z:
        names = [x.decode() for x in z["element_names"]]
    p0, c0, _, t89 = workloads.structure_config4(natoms=10000)
    # the amorphous cube of configuration 4 repeated 3 x 3 x 3 (a periodic structure again) with its own jitter: 270 000 atoms
    shifts = np.array([[i, j, k] for i in range(3) for j in range(3) for k in range(3)], float) @ c0
    pos = (p0[None, :, :] + shifts[:, None, :]).reshape(-1, 3) + np.random.default_rng(9).normal(0.0, 0.02, (27 * len(p0), 3))
    measure("GRACE-3L, amorphous cube of configuration 4 repeated 3x3x3", kk.Model(mp), workloads.config4_species(names),
            np.tile(workloads.config4_types(t89), 27), pos, 3.0 * c0, 2)
    return {"workload": "size range, calculator-level call with the neighbour list kept", "dtype": "f64" if a.precision == 64 else "f32", "entries": out}


def run_workload(a, light=False):
    """One workload at one precision: the resident pass timed over a.steps steps, the calculator-level calls, the stage
    times and rooflines, and (unless a.no_cpu) the reference CPU path on the host.  light: the short form used for the
    other_workloads entries of the default run (no ordered-sums leg, no host-buffer leg)."""
    import torch

    from grace_runtime_amd import kk, synth, workloads
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    tmp = tempfile.mkdtemp()
    batch = a.workload == "config5"
    two = a.workload == "config3" or batch
    three = a.workload == "config4"
    reps = a.reps or (20 if two else 16)
    pbc = [True, True, True]
    structs = None
    if three:
        mpath = workloads.write_model("config4", tmp)
        with np.load(mpath) as z:
            names = [x.decode() for x in z["element_names"]]
        pos, cell, _, t89 = workloads.structure_config4(natoms=a.atoms)
        # the 8 species present become atom types 1..8 of the engine (as a LAMMPS pair_coeff line would map them)
        species = workloads.config4_species(names)
        types = workloads.config4_types(t89)
    elif batch:
        mpath = workloads.write_model("config5", tmp)
        species = ["Al", "Ni", "Ti"]
        structs = workloads.structures_config5()
        b_natoms, types, pos, b_cells, b_pbc = workloads.batch_arrays(structs)
    elif two:
        mpath = workloads.write_model("config3", tmp)
        species = ["Al", "Co", "Ni", "Ti"]
        pos, cell = synth.fcc_supercell(3.6, reps)
        pos = synth.jitter(pos, 0.08, 3)
        types = np.random.default_rng(3).integers(1, 5, size=len(pos)).astype(np.int32)
    else:
        mpath = workloads.write_model("config1", tmp)
        species = ["W"]
        pos, cell = synth.bcc_supercell(3.165, reps)
        pos = synth.jitter(pos, 0.05, 2)
        types = np.ones(len(pos), np.int32)
    N = len(pos)
    model = kk.Model(mpath)
    t1 = time.perf_counter()
    eng = kk.Engine(model, species, precision=a.precision)
    create_s = time.perf_counter() - t1        # includes the run-time compilation of the model-specialised product kernels
    eng.set_chunksize(a.chunksize)
    eng.set_spline(a.spline)
    if batch:
        def upload():
            eng.upload_batch(structs, 6.0)
    else:
        perm, offset, j, image, shifts = kk.neighbor_search(pos, cell, pbc, 6.0, num_threads=len(os.sched_getaffinity(0)))

        def upload():
            eng.upload(types[perm], offset, j, positions=pos[perm], image=image, shifts=shifts)
    upload()
    eng.debug_copy(1 << 30)     # k_copy_calibration over 1 GiB: scales the rocprof FETCH_SIZE / WRITE_SIZE counters
    copy_gbs, read_gbs = eng.stream_rates(1 << 30)      # what plain stream kernels reach on this GPU (HIP events)

    for _ in range(a.warmup):
        eng.run()
    eng.sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        eng.run()
    eng.sync()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / a.steps
    one = []
    for _ in range(a.steps):
        t1 = time.perf_counter()
        eng.run()
        eng.sync()
        one.append(time.perf_counter() - t1)
    median_ms = float(np.median(one)) * 1e3
    mem_gb = kk.memory_in_use() / 1e9          # device memory the library holds after the timed passes (weights + work buffers)
    out = eng.fetch_batch() if batch else eng.fetch()
    E = eng.edge_count()
    host_ms, list_ms, batch_ms = None, None, None
    if batch:
        # the calculator-level calls: Batch.compute (host arrays, host lists) and Batch.compute_device (device arrays,
        # device lists), whole batch per call
        bt = kk.Batch(model, species, precision=a.precision)
        bt.keep_buffers = True
        dev = torch.device("cuda", 0)
        d_t, d_x = torch.tensor(types, device=dev), torch.tensor(pos, device=dev)
        d_e = torch.zeros(len(structs), dtype=torch.float64, device=dev)
        d_f = torch.zeros((N, 3), dtype=torch.float64, device=dev)
        d_v = torch.zeros((len(structs), 6), dtype=torch.float64, device=dev)
        th, td = [], []
        for _ in range(3):
            t1 = time.perf_counter()
            bt.compute(b_natoms, types, pos, b_cells, b_pbc)
            th.append(time.perf_counter() - t1)
            t1 = time.perf_counter()
            bt.compute_device(b_natoms, d_t, d_x, b_cells, b_pbc, d_e, forces=d_f, virial=d_v)
            torch.cuda.synchronize()
            td.append(time.perf_counter() - t1)
        batch_ms = {"Batch.compute_host_arrays": round(float(np.median(th[1:])) * 1e3, 3),
                    "Batch.compute_device": round(float(np.median(td[1:])) * 1e3, 3)}
        del bt
    else:
        # the same pass through the one-call entry point: host buffers in (PCIe), pass, results out; reported beside, never as `value`
        th = []
        for _ in range(2 if light else 4):
            t1 = time.perf_counter()
            eng.compute(types[perm], offset, j, positions=pos[perm], image=image, shifts=shifts)
            th.append(time.perf_counter() - t1)
        host_ms = float(np.median(th[1:])) * 1e3
        # the calculator's call (kk.System.compute: positions, cell, types in; neighbour list, pass, results out), with
        # the list rebuilt on every call (skin 0) and with the list kept (skin 0.5 A, unmoved atoms)
        list_ms = {}
        for label, skin in (("rebuilt", 0.0), ("kept", 0.5)):
            sysm = kk.System(model, species, skin=skin, precision=a.precision)
            tl = []
            for k in range(3):
                t1 = time.perf_counter()
                sysm.compute(types, pos + (1e-9 * k if skin == 0.0 else 0.0), cell, pbc)     # any displacement rebuilds a skin-0 list
                tl.append(time.perf_counter() - t1)
            assert sysm.rebuilds == (3 if skin == 0.0 else 1)
            list_ms[label] = float(np.median(tl[1:])) * 1e3
            del sysm
    upload()

    # the same passes with ordered (atomic-free) sums of forces, virial, energy and message adjoints: reported beside
    ordered_ms = None
    if not light:
        eng.set_ordered_sums(True)
        eng.run()
        eng.sync()
        t1 = time.perf_counter()
        for _ in range(a.steps):
            eng.run()
        eng.sync()
        ordered_ms = (time.perf_counter() - t1) / a.steps * 1e3
        eng.set_ordered_sums(False)

    # the same passes with the radial functions from tables of 1024 intervals, as the reference's engines take them (1L / 2L)
    spline_ms = None
    if not three and a.spline == 0:
        eng.set_spline(1024)
        eng.run()
        eng.sync()
        t1 = time.perf_counter()
        for _ in range(a.steps):
            eng.run()
        eng.sync()
        spline_ms = (time.perf_counter() - t1) / a.steps * 1e3
        eng.set_spline(0)

    # per-stage durations: HIP events around every launch on the engine's stream, averaged over the same K steps
    eng.set_profile(True)
    acc = {}
    for _ in range(a.steps):
        eng.run()
        for k, (ms, cnt) in eng.stage_times().items():
            acc[k] = acc.get(k, 0.0) + ms
    gemm_flops = eng.stage_flops()       # tile-GEMM flops per stage (live functions only), counted by the engine
    eng.set_profile(False)
    stages = {k: v / a.steps for k, v in acc.items()}

    C, nl, nlm, s = (64, 6, 36, a.precision // 8) if three else (32, 5, 25, a.precision // 8)
    # GRACE-3L: message functions gathered by the pair kernels of layers 2 and 3; radial MLP 8-128-128-384, value + tangent
    extra = dict(radial_flops=4.0 * (8 * 128 + 128 * 128 + 128 * 384), slots={"2": 36, "3": 72},
                 stream_bytes=couple_stream_bytes(workloads.model_config4(), N, s)) if three else {}
    if a.spline > 0 and not three:
        extra = dict(radial_flops=0.0)    # the radial stages are table look-ups: a stream, not a GEMM
    # FC / reduce tile GEMMs: flops of the live functions as the engine counts them
    dense_flops = dict(gemm_flops)
    roof = {}
    for k, ms in stages.items():
        r = stage_model(k, ms, E, N, C, nl, nlm, s, a.precision, dense_flops, **extra)
        if r:
            r["ms"] = ms
            r["frac"] = r["achieved"] / r["peak"]
            roof[k] = r
    total_ms = sum(stages.values())
    # the per-atom dense chain as one entry: every FC, product, reduce and readout launch; flops = the tile GEMMs'
    dense_ms = sum(v for k, v in stages.items() if k.startswith(DENSE_PREFIXES))
    dense_fl = sum(v for k, v in gemm_flops.items() if k.startswith(DENSE_PREFIXES))
    dense = {"ms": round(dense_ms, 4), "share_of_pass": round(dense_ms / total_ms, 4), "gemm_flops": dense_fl,
             "bound": "mfma", "achieved": round(dense_fl / (dense_ms * 1e-3) / 1e12, 3) if dense_ms > 0 else 0.0, "peak": PEAK[a.precision],
             "unit": "TFLOP/s", "frac": round(dense_fl / (dense_ms * 1e-3) / 1e12 / PEAK[a.precision], 4) if dense_ms > 0 else 0.0,
             "traffic": DENSE_TRAFFIC.get(a.workload) if a.precision == 64 and reps == (20 if two else 16) else None,
             "minimal_bytes": N * (2 * nlm * C * s + 2 * 8 * 32) if not (two or three) else None}
    modelled = dict(roof)
    dom = max(modelled, key=lambda k: modelled[k]["ms"])
    d = modelled[dom]
    roofline = {"kernel": dom, "bound": d["bound"], "achieved": round(d["achieved"], 3), "peak": d["peak"],
                "unit": d["unit"], "frac": round(d["frac"], 4),
                "traffic": MEASURED_TRAFFIC.get((a.workload, dom)) if reps == (20 if two else 16) and a.atoms == 10000 and a.precision == 64 and a.spline == 0 else None,
                "avg_ms": round(d["ms"], 4), "algorithmic_work": d["work"]}

    cpu = None
    if not a.no_cpu:
        from oracle import ref_lib      # the compiled reference CPU path: the checker, timed here as the baseline
        if ref_lib.available() and batch:
            # the reference evaluates a batch one structure at a time (python/grace_runtime/batch.py); sample: the first cells
            nth = len(os.sched_getaffinity(0))
            ref = ref_lib.RefModel(mpath, [0, 1, 2])
            lists = [kk.neighbor_search(p, c, [True, True, True], 6.0) for p, c, _ in structs[:128]]
            t_end = time.perf_counter() + (8.0 if light else 20.0)
            done, secs, de, a0 = 0, 0.0, 0.0, 0
            for (p, c, t), (pm, of, jj, im, sh) in zip(structs[:128], lists):
                t1 = time.perf_counter()
                r = ref.compute(t[pm], of, jj, positions=p[pm], image=im, shifts=sh, nthreads=nth)
                secs += time.perf_counter() - t1
                de = max(de, abs(r["energy"] - out["energy"][done]) / len(p))
                done += 1
                a0 += len(p)
                if time.perf_counter() > t_end:
                    break
            cpu = {"value": round(secs / a0 * 1e6, 4), "unit": "us/atom", "cores": nth, "kind": "reference",
                   "sample": f"the first {done} cells ({a0} atoms) of the batch, one call of the compiled reference Grace2LFused (fp32 + spline "
                             f"tables) per cell, neighbour lists not timed",
                   "dE_per_atom_vs_gpu": de}
        elif ref_lib.available():
            nth = len(os.sched_getaffinity(0))
            ref = ref_lib.RefModel(mpath, [names.index(x) for x in species] if three else list(range(len(species))))
            args = dict(positions=pos[perm], image=image, shifts=shifts, nthreads=nth)
            ref.compute(types[perm], offset, j, **args)
            ts = []
            t_end = time.perf_counter() + (6.0 if light else 20.0)
            while len(ts) < 3 or (time.perf_counter() < t_end and len(ts) < 25):
                t1 = time.perf_counter()
                r = ref.compute(types[perm], offset, j, **args)
                ts.append(time.perf_counter() - t1)
            tm = float(np.median(ts))
            cpu = {"value": round(tm / N * 1e6, 4), "unit": "us/atom", "cores": nth, "kind": "reference",
                   "sample": f"{len(ts)} full calls of the compiled reference Grace{3 if three else 2 if two else 1}LFused (fp32 + spline tables) on the same "
                             f"{N}-atom structure, median",
                   "dE_per_atom_vs_gpu": abs(r["energy"] - out["energy"]) / N,
                   "max_dF_vs_gpu": float(np.abs(r["forces"] - out["forces"]).max())}

    res = {
        # value: the energy + forces + virial pass on the structure resident in HBM (inputs on the device when the timed
        # region starts); the reference's own protocol times the calculator call with a kept neighbour list
        # (docs/benchmarks.md:9-20): that figure is us_per_atom_calculator_call_kept_list beside it
        "metric": "us_per_atom_EFS_call_resident_pass", "value": round(dt / N * 1e6, 5), "unit": "us/atom", "n_gpus": 1,
        "us_per_atom_calculator_call_kept_list": round(list_ms["kept"] / N * 1e3, 5) if list_ms else None,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(dt * 1e3, 4), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "f64" if a.precision == 64 else "f32", "data": "synthetic",
        "config": {"workload": (f"GRACE-2L-shaped random-init model (2 layers, lmax 4, 32 ch, 3 species) over {len(structs)} independent periodic "
                                f"cells of 32-128 atoms as one ragged batch, {N} atoms, {E} edges, rc 6 A (benchmark configuration 5)") if batch else
                               (f"GRACE-3L-shaped random-init model (3 layers, lmax 5, 64 ch, radial MLPs (8 + 2 x 32)-128-128-384, 89-species "
                                f"embedding table, 8 species present) on an amorphous cube of {N} atoms at 0.08 / A^3, {E} edges, rc 6 A "
                                f"(benchmark configuration 4)") if three else
                               (f"GRACE-2L-shaped random-init model (2 layers, lmax 4, 32 ch, MLPs 8-64-64-160, body order 3) on the "
                                f"4-species fcc alloy {reps}x{reps}x{reps}, {N} atoms, {E} edges, rc 6 A (benchmark configuration 3)") if two else
                               (f"GRACE-1L-shaped random-init model (lmax 4, 32 ch, MLP 8-64-64-160) on bcc W "
                                f"{reps}x{reps}x{reps}, {N} atoms, {E} edges, rc 6 A (benchmark configuration 2)"),
                   "atoms": N, "edges": int(E)},
        "atoms_steps_per_s": round(N / dt, 1),
        "median_ms_per_step": round(median_ms, 4),
        "timing": "value, ms_per_step: mean of the K passes on the resident structure; median_ms_per_step: median of K passes timed one by one",
        "ms_per_call_host_buffers": round(host_ms, 3) if host_ms is not None else None,
        "ms_per_calculator_call": batch_ms if batch else {"neighbour_list_rebuilt": round(list_ms["rebuilt"], 3),
                                                          "neighbour_list_kept": round(list_ms["kept"], 3)},
        "ms_per_step_ordered_sums": round(ordered_ms, 4) if ordered_ms is not None else None,
        "ms_per_step_radial_tables_1024": round(spline_ms, 4) if spline_ms is not None else None,
        "spline": a.spline,
        "engine_create_s": round(create_s, 3),
        "chunksize": eng.chunksize,              # atoms per engine pass the timed steps ran with (0: the whole structure in one pass)
        "device_memory_GB": round(mem_gb, 3),
        "roofline": roofline,
        "hbm_calibration": {"copy_GBs": round(copy_gbs, 1), "read_only_GBs": round(read_gbs, 1), "bytes": 1 << 30,
                            "note": "plain stream kernels over 1 GiB, best of 5: copy counts bytes read + written; roofline.frac "
                                    "divides by the published 8000 GB/s, not by these"},
        "dense_chain": dense,
        "stages_ms": {k: round(v, 4) for k, v in stages.items()},
        "stages_roofline": {k: {"bound": v["bound"], "achieved": round(v["achieved"], 2), "unit": v["unit"],
                                "frac": round(v["frac"], 4)} for k, v in roof.items()},
        "sum_stage_ms": round(total_ms, 4),
        "cpu_baseline": cpu,
        "energy": float(np.sum(out["energy"])),
    }
    eng.close()
    return res


if __name__ == "__main__":
    main()
