"""The radial entry point that allocates no device memory (gr_engine_radial_noalloc) against the existing entry point
gr_engine_debug_radial, through the C ABI: bit-identical values in fp64 and fp32 (both run the same kernel; the fixed
device array only replaces the allocated staging rows), on calls in a row that share the fixed array, the second with
a smaller input; the size limit and the argument errors."""
import os

import numpy as np
import pytest

import cases
from grace_runtime_amd import _lib, kk

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def model_path(tmp_path_factory):
    return cases.write_model("mix2", str(tmp_path_factory.mktemp("noalloc")))


def _args(m, nel, seed):
    rng = np.random.default_rng(seed)
    return rng.uniform(0.02, 0.9995, m), rng.integers(0, nel, m).astype(np.int32)


@pytest.mark.parametrize("precision", [64, 32])
def test_no_alloc_radial_equals_debug_radial_on_consecutive_calls(model_path, precision):
    import torch
    model = kk.Model(model_path)
    eng = kk.Engine(model, ["Mo", "W"], precision)
    nl, Cn, nel = model.lmax + 1, model.n_radial, len(model.element_names)
    dev = torch.device("cuda", 0)
    used = _lib.lib().gr_memory_in_use()
    # the second call is smaller than the first: rows of the first stay in the fixed array behind those of the second
    for m, seed in ((3000, 11), (777, 12), (1, 13), (3000, 14)):
        x, mu = _args(m, nel, seed)
        R_ref, dR_ref = eng.debug_radial(x, mu)
        xd, mud = torch.tensor(x, device=dev), torch.tensor(mu, device=dev)
        R = torch.full((m, nl, Cn), float("nan"), dtype=torch.float64, device=dev)
        dR = torch.full((m, nl, Cn), float("nan"), dtype=torch.float64, device=dev)
        # no synchronisation here: the fills above are still queued on torch's stream when the call starts
        eng.radial_noalloc(xd, mud, R, dR)
        assert np.array_equal(R.cpu().numpy(), R_ref), (precision, m)
        assert np.array_equal(dR.cpu().numpy(), dR_ref), (precision, m)
    assert _lib.lib().gr_memory_in_use() == used    # the library's own allocations did not change
    eng.close()


def test_no_alloc_radial_waits_for_arguments_written_on_another_stream(model_path):
    """x is produced on torch's stream right before the call, behind a long queue of work, with no synchronisation by
    the caller: the entry point itself waits for the device before its kernels read x."""
    import torch
    model = kk.Model(model_path)
    eng = kk.Engine(model, ["Mo", "W"], 64)
    nl, Cn, nel = model.lmax + 1, model.n_radial, len(model.element_names)
    dev = torch.device("cuda", 0)
    m = 2048
    x, mu = _args(m, nel, 21)
    R_ref, dR_ref = eng.debug_radial(x, mu)
    mud = torch.tensor(mu, device=dev)
    R = torch.empty((m, nl, Cn), dtype=torch.float64, device=dev)
    dR = torch.empty_like(R)
    xh = torch.tensor(x).pin_memory()
    big = torch.ones((4096, 4096), dtype=torch.float64, device=dev)
    torch.cuda.synchronize()
    for _ in range(4):
        big = big @ big * 1e-4                   # a few hundred milliseconds of queued work in front of x
    xd = torch.full((m,), 0.5, dtype=torch.float64, device=dev)
    xd.copy_(xh, non_blocking=True)              # x arrives last on torch's stream
    eng.radial_noalloc(xd, mud, R, dR)
    assert np.array_equal(R.cpu().numpy(), R_ref) and np.array_equal(dR.cpu().numpy(), dR_ref)
    eng.close()


def test_no_alloc_radial_calls_of_two_threads_and_two_engines_do_not_mix(model_path):
    """Two engines called from two threads share the one fixed array of the GPU: the library serialises the calls, so
    each gets its own values."""
    import threading

    import torch
    model = kk.Model(model_path)
    nl, Cn, nel = model.lmax + 1, model.n_radial, len(model.element_names)
    dev = torch.device("cuda", 0)
    engines = [kk.Engine(model, ["Mo", "W"], 64), kk.Engine(model, ["Mo", "W"], 64)]
    jobs = []
    for t in range(2):
        m = 1500 + 700 * t
        x, mu = _args(m, nel, 31 + t)
        jobs.append((m, x, mu, engines[t].debug_radial(x, mu)))
    bad = []

    def work(t):
        m, x, mu, (R_ref, dR_ref) = jobs[t]
        xd, mud = torch.tensor(x, device=dev), torch.tensor(mu, device=dev)
        R = torch.empty((m, nl, Cn), dtype=torch.float64, device=dev)
        dR = torch.empty_like(R)
        for _ in range(20):
            engines[t].radial_noalloc(xd, mud, R, dR)
            if not (np.array_equal(R.cpu().numpy(), R_ref) and np.array_equal(dR.cpu().numpy(), dR_ref)):
                bad.append(t)
                return

    th = [threading.Thread(target=work, args=(t,)) for t in range(2)]
    for t in th:
        t.start()
    for t in th:
        t.join()
    assert not bad
    for e in engines:
        e.close()


def test_no_alloc_radial_limits_and_errors(model_path):
    import torch
    model = kk.Model(model_path)
    eng = kk.Engine(model, ["Mo", "W"], 64)
    nl, Cn = model.lmax + 1, model.n_radial
    dev = torch.device("cuda", 0)
    m = 2_000_000                              # far beyond the fixed 32 MiB array
    xd = torch.zeros(m, dtype=torch.float64, device=dev)
    mud = torch.zeros(m, dtype=torch.int32, device=dev)
    R = torch.zeros((m, nl, Cn), dtype=torch.float64, device=dev)
    dR = torch.zeros_like(R)
    with pytest.raises(ValueError, match="fixed"):
        eng.radial_noalloc(xd, mud, R, dR)
    # an element outside the model is reported, and the call does not leave the tables
    m = 100
    x, mu = _args(m, 2, 5)
    mu[17] = 9
    R = torch.zeros((m, nl, Cn), dtype=torch.float64, device=dev)
    dR = torch.zeros_like(R)
    with pytest.raises(ValueError, match="element"):
        eng.radial_noalloc(torch.tensor(x, device=dev), torch.tensor(mu, device=dev), R, dR)
    # host memory is refused
    with pytest.raises(ValueError):
        eng.radial_noalloc(torch.tensor(x), torch.tensor(mu), torch.zeros((m, nl, Cn), dtype=torch.float64),
                           torch.zeros((m, nl, Cn), dtype=torch.float64))
    # the engine still works afterwards
    mu[17] = 1
    R_ref, dR_ref = eng.debug_radial(x, mu)
    eng.radial_noalloc(torch.tensor(x, device=dev), torch.tensor(mu, device=dev), R, dR)
    assert np.array_equal(R.cpu().numpy(), R_ref) and np.array_equal(dR.cpu().numpy(), dR_ref)
    eng.close()


def test_no_alloc_radial_is_for_one_layer_engines(tmp_path):
    import torch
    path = cases.write_model("l2mix", str(tmp_path))
    eng = kk.Engine(kk.Model(path), ["Mo", "W"], 64)
    dev = torch.device("cuda", 0)
    model = eng.model
    R = torch.zeros((4, model.lmax + 1, model.n_radial), dtype=torch.float64, device=dev)
    with pytest.raises(RuntimeError, match="GRACE-1L"):
        eng.radial_noalloc(torch.zeros(4, dtype=torch.float64, device=dev), torch.zeros(4, dtype=torch.int32, device=dev), R, R.clone())
    eng.close()
