"""ctypes access to oracle/_ref/libgrace_ref_<isa>.so: the reference's own CPU drivers, compiled by oracle/Makefile
from the reference checkout (TEST INFRASTRUCTURE; see oracle/ref_shim.cpp).  Used to validate the numpy restatement
and as the CPU baseline of the benchmark.  `available()` is False when the library was not built."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


def _has_avx512():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    fl = line.split()
                    return all(k in fl for k in ("avx512f", "avx512bw", "avx512dq", "avx512vl", "avx512cd"))
    except OSError:
        pass
    return False


def lib_path():
    tags = ["v4", "v3"] if _has_avx512() else ["v3"]
    for t in tags:
        p = os.path.join(_HERE, "_ref", f"libgrace_ref_{t}.so")
        if os.path.exists(p):
            return p
    return None


def available():
    return lib_path() is not None


def _load():
    global _lib
    if _lib is not None:
        return _lib
    p = lib_path()
    if p is None:
        raise RuntimeError("oracle/_ref is not built (make -C oracle both REF=/path/to/reference)")
    L = C.CDLL(p)
    L.ref_last_error.restype = C.c_char_p
    L.ref_open.restype = C.c_void_p
    L.ref_open.argtypes = [C.c_char_p, C.c_int]
    L.ref_layers.argtypes = [C.c_void_p]
    L.ref_n_elements.argtypes = [C.c_void_p]
    L.ref_setup_types.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
    L.ref_cutoff.restype = C.c_double
    L.ref_cutoff.argtypes = [C.c_void_p, C.c_int, C.c_int]
    L.ref_compute.argtypes = [C.c_void_p, C.c_int] + [C.c_void_p] * 7 + [C.c_int, C.c_int] + [C.c_void_p] * 4
    L.ref_compute_uq.argtypes = [C.c_void_p, C.c_int] + [C.c_void_p] * 7 + [C.c_int] + [C.c_void_p] * 4
    if hasattr(L, "ref_compute_vatom"):
        L.ref_compute_vatom.argtypes = [C.c_void_p, C.c_int] + [C.c_void_p] * 4 + [C.c_int] + [C.c_void_p] * 4
    L.ref_close.argtypes = [C.c_void_p]
    L.ref_nl_build.restype = C.c_void_p
    L.ref_nl_build.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_double, C.c_int]
    L.ref_nl_nbonds.restype = C.c_int64
    L.ref_nl_nbonds.argtypes = [C.c_void_p]
    L.ref_nl_nimages.restype = C.c_int64
    L.ref_nl_nimages.argtypes = [C.c_void_p]
    L.ref_nl_get.argtypes = [C.c_void_p] * 6
    L.ref_nl_free.argtypes = [C.c_void_p]
    _lib = L
    return L


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


class RefModel:
    """The reference Grace{1,2,3}LFused driver on a kokkos.npz file."""

    def __init__(self, path, type2mu, spline_n=1024):
        L = _load()
        self._L = L
        self._h = L.ref_open(os.fsencode(path), int(spline_n))
        if not self._h:
            raise RuntimeError(L.ref_last_error().decode())
        self.layers = L.ref_layers(self._h)
        t = np.ascontiguousarray(np.concatenate([[-1], np.asarray(type2mu)]), dtype=np.int32)
        self.ntypes = t.size - 1
        if L.ref_setup_types(self._h, self.ntypes, _p(t)):
            raise RuntimeError(L.ref_last_error().decode())

    def cutoff(self, t1, t2):
        return self._L.ref_cutoff(self._h, t1, t2)

    def compute(self, types, offset, j, rij=None, positions=None, image=None, shifts=None, nthreads=1,
                energy_only=False):
        """types are 1-based (index into type2mu + 1), as the reference's Model.compute."""
        types = np.ascontiguousarray(types, dtype=np.int32)
        offset = np.ascontiguousarray(offset, dtype=np.int64)
        j = np.ascontiguousarray(j, dtype=np.int32)
        n = types.size
        cv = lambda a: None if a is None else np.ascontiguousarray(a, dtype=np.float64)
        rij, positions, shifts = cv(rij), cv(positions), cv(shifts)
        image = None if image is None else np.ascontiguousarray(image, dtype=np.int32)
        e = C.c_double(0.0)
        eat = np.zeros(n)
        f = np.zeros((n, 3))
        v = np.zeros(6)
        rc = self._L.ref_compute(self._h, n, _p(types), _p(offset), _p(j), _p(rij), _p(positions), _p(image),
                                 _p(shifts), int(nthreads), int(energy_only), C.addressof(e), _p(eat), _p(f), _p(v))
        if rc:
            raise RuntimeError(self._L.ref_last_error().decode())
        return {"energy": e.value, "energies": eat, "forces": f, "virial": v}

    def compute_vatom(self, types, offset, j, rij, nthreads=1):
        """the call with ComputeFlags::vflag_atom: also virials [n, 6], the reference's Outputs::vatom"""
        types = np.ascontiguousarray(types, dtype=np.int32)
        offset = np.ascontiguousarray(offset, dtype=np.int64)
        j = np.ascontiguousarray(j, dtype=np.int32)
        rij = np.ascontiguousarray(rij, dtype=np.float64)
        n = types.size
        e = C.c_double(0.0)
        f, v, va = np.zeros((n, 3)), np.zeros(6), np.zeros((n, 6))
        rc = self._L.ref_compute_vatom(self._h, n, _p(types), _p(offset), _p(j), _p(rij), int(nthreads), C.addressof(e), _p(f), _p(v), _p(va))
        if rc:
            raise RuntimeError(self._L.ref_last_error().decode())
        return {"energy": e.value, "forces": f, "virial": v, "virials": va}

    def compute_uq(self, types, offset, j, rij, nthreads=1):
        """GRACE-1L UQ head of the reference (forward only): energy, gamma, atomic_sigma, gmm_cluster per atom."""
        types = np.ascontiguousarray(types, dtype=np.int32)
        offset = np.ascontiguousarray(offset, dtype=np.int64)
        j = np.ascontiguousarray(j, dtype=np.int32)
        rij = np.ascontiguousarray(rij, dtype=np.float64)
        n = types.size
        e = C.c_double(0.0)
        g, sg, cl = np.zeros(n), np.zeros(n), np.zeros(n)
        rc = self._L.ref_compute_uq(self._h, n, _p(types), _p(offset), _p(j), _p(rij), None, None, None, int(nthreads),
                                    C.addressof(e), _p(g), _p(sg), _p(cl))
        if rc:
            raise RuntimeError(self._L.ref_last_error().decode())
        return {"energy": e.value, "gamma": g, "atomic_sigma": sg, "gmm_cluster": cl}

    def close(self):
        if self._h:
            self._L.ref_close(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def neighbor_search(positions, cell, pbc, cutoff, nthreads=1):
    """The reference's neighbor_search (python/src/neighbors.cpp:15-95): dict(perm, offset, j, image, shifts)."""
    L = _load()
    pos = np.ascontiguousarray(positions, dtype=np.float64)
    cell = np.ascontiguousarray(cell, dtype=np.float64)
    pb = np.ascontiguousarray(pbc, dtype=np.uint8)
    n = pos.shape[0]
    h = L.ref_nl_build(_p(pos), n, _p(cell), _p(pb), float(cutoff), int(nthreads))
    if not h:
        raise ValueError(L.ref_last_error().decode())
    try:
        nb, ni = L.ref_nl_nbonds(h), L.ref_nl_nimages(h)
        out = {"perm": np.zeros(n, np.int64), "offset": np.zeros(n + 1, np.int64), "j": np.zeros(nb, np.int32),
               "image": np.zeros(nb, np.int32), "shifts": np.zeros((ni, 3))}
        L.ref_nl_get(h, _p(out["perm"]), _p(out["offset"]), _p(out["j"]), _p(out["image"]), _p(out["shifts"]))
    finally:
        L.ref_nl_free(h)
    return out
