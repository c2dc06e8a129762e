"""MI355X plug-in module with the interface of the reference's GPU module `_kk_<arch>` (python/kk/kk_api.h:16-156,
bindings python/kk/kk_module.cpp:200-275): module functions `initialize / finalize / initialized / device / arch /
platform / blas / cublas / memory_info`, classes `Model`, `System`, `Batch`, and the plug-in attributes `ABI`,
`PLATFORM` (python-rocm6/grace_runtime_rocm6/__init__.py:8-22).  `Engine` is the CSR-level entry
(`_core.Model.compute`, python/src/core.cpp:292-396) and `neighbor_search` the list of `_core.neighbor_search`.

All arithmetic runs in libgrace_hip.so on the GPU; there is no CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from . import _lib
from ._lib import FLAG_EATOM, FLAG_ENERGY_ONLY, FLAG_UQ, as_array, check, ptr

ABI = 7
PLATFORM = "rocm"
ROCM_MAJOR = 7

_state = {"device": None}


def archs():
    return ["gfx950"]


def initialize(device: int = 0):
    """One GPU per process (python/kk/kk_core.cpp:86-98): a second call with another device is an error."""
    L = _lib.lib()
    if _state["device"] is not None:
        if _state["device"] != int(device):
            raise RuntimeError(f"already initialised on device {_state['device']}")
        return
    n = L.gr_device_count()
    if n <= 0:
        raise RuntimeError("no HIP device found")
    if not 0 <= int(device) < n:
        raise ValueError(f"device {device} out of range (0 .. {n - 1})")
    _state["device"] = int(device)


def finalize():
    _state["device"] = None


def initialized() -> bool:
    return _state["device"] is not None


def device() -> int:
    if _state["device"] is None:
        raise RuntimeError("not initialised")
    return _state["device"]


def arch() -> str:
    return "gfx950"


def platform() -> str:
    return PLATFORM


def blas() -> str:
    return ""    # hand-written MFMA kernels, no BLAS library


def cublas() -> bool:
    return False


def memory_info():
    import torch
    free, total = torch.cuda.mem_get_info(device())
    return int(free), int(total)


def memory_in_use() -> int:
    """bytes of device memory held by the library's buffers (all engines of the process)"""
    return int(_lib.lib().gr_memory_in_use())


def set_memory_limit(nbytes: int):
    """cap on memory_in_use(): an allocation beyond it fails like one the device refuses (MemoryError, or the smaller
    passes of Batch); 0 removes the cap"""
    _lib.lib().gr_set_memory_limit(int(nbytes))


def _dev():
    if _state["device"] is None:
        initialize(0)
    return _state["device"]


_LOG_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_int, C.c_char_p)
_log_keepalive = None


def set_logger(fn):
    """fn(level, message) receives the library's messages (level 0 information, 1 warning); None switches them off"""
    global _log_keepalive
    if fn is None:
        _lib.lib().gr_set_logger(None, None)
        _log_keepalive = None
        return
    cb = _LOG_FN(lambda user, level, msg: fn(int(level), msg.decode(errors="replace")))
    _lib.lib().gr_set_logger(C.cast(cb, C.c_void_p), None)
    _log_keepalive = cb


def neighbor_search(positions, cell, pbc, cutoff, num_threads: int = 0):
    """(perm, offset, j, image, shifts) of the Verlet list at `cutoff`; identical to the reference list
    (python/src/neighbors.cpp:15-95)."""
    L = _lib.lib()
    pos = as_array(positions, np.float64, 3) if len(positions) else np.zeros((0, 3))
    cell = np.ascontiguousarray(cell, dtype=np.float64).reshape(3, 3)
    pb = np.ascontiguousarray([bool(p) for p in pbc], dtype=np.uint8)
    h = C.c_void_p()
    check(L.gr_neighbor_build(pos.shape[0], ptr(pos), ptr(cell), ptr(pb), float(cutoff), max(int(num_threads), 1) if
                              num_threads else 8, C.byref(h)))
    try:
        n, nb, ni = pos.shape[0], L.gr_nlist_nbonds(h), L.gr_nlist_nimages(h)
        perm, offset = np.zeros(n, np.int64), np.zeros(n + 1, np.int64)
        j, image, shifts = np.zeros(nb, np.int32), np.zeros(nb, np.int32), np.zeros((ni, 3))
        check(L.gr_nlist_get(h, ptr(perm), ptr(offset), ptr(j), ptr(image), ptr(shifts)))
    finally:
        L.gr_nlist_free(h)
    return perm, offset, j, image, shifts


class Model:
    """A loaded kokkos.npz (host side).  `Model(path, spline=1024, asi="")`: python/kk/kk_api.h:51-64; `spline` is kept as
    the attribute of that name, which the reference's calculator hands to System / Batch (python/grace_runtime/
    calculator.py:358)."""

    def __init__(self, path, spline: int = 1024, asi: str = ""):
        L = _lib.lib()
        if asi:
            raise ValueError("PACE active-set files are not supported by this engine")
        self._h = C.c_void_p()
        check(L.gr_model_load(str(path).encode(), C.byref(self._h)))
        info = _lib.ModelInfo()
        check(L.gr_model_get_info(self._h, C.byref(info)))
        self.path = str(path)
        self.spline = int(spline)
        self.layers = info.layers
        self.lmax, self.n_radial, self.rcut, self.max_order = info.lmax, info.n_radial, info.rcut, info.max_order
        self.n_elements = info.n_elements
        self.element_names = [L.gr_model_element_name(self._h, k).decode() for k in range(info.n_elements)]
        self.has_uq = bool(L.gr_model_has_uq(self._h))
        self.slow_notice = ""
        self.needs_generic = False
        self.engine_setups = 0

    def validate_uq(self):
        """ValueError when the model's UQ head cannot be evaluated (none, another schema, sizes that do not fit):
        python/kk/kk_api.h:51-64, libgrace/src/model_1l.cpp:275-285.  The UQ head is evaluated for GRACE-1L models."""
        check(_lib.lib().gr_model_validate_uq(self._h))

    def type2mu(self, species):
        """[-1, mu(species[0]), ...]; unknown element -> ValueError (python/kk/kk_core.cpp: std::invalid_argument);
        None leaves the atom type unmapped (-1), the NULL of a LAMMPS pair_coeff line"""
        out = [-1]
        for s in species:
            if s is None:
                out.append(-1)
                continue
            if s not in self.element_names:
                raise ValueError(f"element {s} is not in the model (elements: {' '.join(self.element_names)})")
            out.append(self.element_names.index(s))
        return np.asarray(out, dtype=np.int32)

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                _lib.lib().gr_model_free(self._h)
                self._h = None
        except Exception:
            pass


class Engine:
    """One model + species set on the GPU.  `compute` is `_core.Model.compute` on CSR bonds
    (python/src/core.cpp:292-396); `upload / run / fetch` split it for callers that keep the structure resident."""

    def __init__(self, model: Model, species, precision: int = 64):
        L = _lib.lib()
        self.model, self.species, self.precision = model, list(species), int(precision)
        t2m = model.type2mu(self.species)
        self._h = C.c_void_p()
        check(L.gr_engine_create(model._h, len(self.species), ptr(t2m), self.precision, _dev(), C.byref(self._h)))
        model.engine_setups += 1
        self._n = 0

    def cutoff(self, t1: int, t2: int) -> float:
        return _lib.lib().gr_engine_cutoff(self._h, int(t1), int(t2))

    # ---- message exchange with ghost atoms (gr_engine_set_exchange and the row movers) ----
    class _Exchange(C.Structure):
        _fields_ = [("forward", C.c_void_p), ("reverse", C.c_void_p), ("user", C.c_void_p)]

    def set_exchange(self, forward=None, reverse=None):
        """forward(layer) / reverse(layer) are called inside compute_lammps when the message rows / adjoint rows of a layer
        are complete (the Exchange of the reference's drivers); both None removes the exchange."""
        cbt = C.CFUNCTYPE(None, C.c_void_p, C.c_int)
        if forward is None and reverse is None:
            check(_lib.lib().gr_engine_set_exchange(self._h, None))
            self._exchange_keepalive = None
            return
        f = cbt(lambda user, layer: forward(int(layer))) if forward else None
        r = cbt(lambda user, layer: reverse(int(layer))) if reverse else None
        x = Engine._Exchange(C.cast(f, C.c_void_p) if f else None, C.cast(r, C.c_void_p) if r else None, None)
        check(_lib.lib().gr_engine_set_exchange(self._h, C.byref(x)))
        self._exchange_keepalive = (f, r)

    @property
    def comm_layers(self) -> int:
        return int(_lib.lib().gr_engine_comm_layers(self._h))

    def comm_width(self, layer: int) -> int:
        return int(_lib.lib().gr_engine_comm_width(self._h, int(layer)))

    def pack_forward_host(self, layer, sendlist):
        sl = as_array(sendlist, np.int32)
        buf = np.zeros((sl.shape[0], self.comm_width(layer)))
        check(_lib.lib().gr_engine_pack_forward_host(self._h, int(layer), sl.shape[0], ptr(sl), ptr(buf)))
        return buf

    def unpack_forward_host(self, layer, first, buf):
        buf = np.ascontiguousarray(buf, dtype=np.float64)
        check(_lib.lib().gr_engine_unpack_forward_host(self._h, int(layer), buf.shape[0], int(first), ptr(buf)))

    def pack_reverse_host(self, layer, first, n):
        buf = np.zeros((int(n), self.comm_width(layer)))
        check(_lib.lib().gr_engine_pack_reverse_host(self._h, int(layer), int(n), int(first), ptr(buf)))
        return buf

    def unpack_reverse_host(self, layer, sendlist, buf):
        sl = as_array(sendlist, np.int32)
        buf = np.ascontiguousarray(buf, dtype=np.float64)
        check(_lib.lib().gr_engine_unpack_reverse_host(self._h, int(layer), sl.shape[0], ptr(sl), ptr(buf)))

    def pack_forward(self, layer, sendlist, buf):
        """device form: sendlist int32 [n] and buf float64 [n, comm_width] are arrays of the module's GPU"""
        n = int(sendlist.shape[0])
        check(_lib.lib().gr_engine_pack_forward(self._h, int(layer), n, _device_pointer(sendlist, "sendlist", (n,), "int32"),
                                                _device_pointer(buf, "buf", (n, self.comm_width(layer)), "float64")))

    def unpack_forward(self, layer, first, buf):
        n = int(buf.shape[0])
        check(_lib.lib().gr_engine_unpack_forward(self._h, int(layer), n, int(first), _device_pointer(buf, "buf", (n, self.comm_width(layer)), "float64")))

    def pack_reverse(self, layer, first, buf):
        n = int(buf.shape[0])
        check(_lib.lib().gr_engine_pack_reverse(self._h, int(layer), n, int(first), _device_pointer(buf, "buf", (n, self.comm_width(layer)), "float64")))

    def unpack_reverse(self, layer, sendlist, buf):
        n = int(sendlist.shape[0])
        check(_lib.lib().gr_engine_unpack_reverse(self._h, int(layer), n, _device_pointer(sendlist, "sendlist", (n,), "int32"),
                                                  _device_pointer(buf, "buf", (n, self.comm_width(layer)), "float64")))

    def set_chunksize(self, atoms: int):
        """atoms per engine pass: 0 one pass, < 0 automatic, > 0 as given"""
        check(_lib.lib().gr_engine_set_chunksize(self._h, int(atoms)))

    @property
    def chunksize(self) -> int:
        return int(_lib.lib().gr_engine_chunksize(self._h))

    def set_spline(self, intervals: int):
        """radial tables of `intervals` cubic pieces for GRACE-1L / 2L engines, as the reference's engines use (0: the radial
        MLP is evaluated for every bond; GRACE-3L engines keep their MLPs)"""
        check(_lib.lib().gr_engine_set_spline(self._h, int(intervals)))

    @property
    def spline(self) -> int:
        return int(_lib.lib().gr_engine_spline(self._h))

    def set_ordered_sums(self, on: bool = True):
        """forces, virial, energy and message adjoints added in a fixed order instead of with floating-point atomics: the
        same bits on every call with the same input; no per-atom virials in this mode."""
        check(_lib.lib().gr_engine_set_ordered_sums(self._h, 1 if on else 0))

    @property
    def ordered_sums(self) -> bool:
        return bool(_lib.lib().gr_engine_ordered_sums(self._h))

    def release_buffers(self):
        """frees the work buffers and the uploaded structure; weights, tables and compiled kernels stay"""
        check(_lib.lib().gr_engine_release_buffers(self._h))
        self._n = 0

    def reset(self):
        """a fresh engine in place of this one, every device buffer dropped (after an allocation failure)"""
        check(_lib.lib().gr_engine_reset(self._h))
        self._n = 0

    def cutoff_matrix(self):
        k = len(self.species)
        return np.array([[self.cutoff(a + 1, b + 1) for b in range(k)] for a in range(k)])

    def _csr_args(self, types, offset, j, rij, positions, image, shifts):
        types = as_array(types, np.int32)
        offset = as_array(offset, np.int64)
        j = as_array(j, np.int32)
        n = types.shape[0]
        if offset.shape[0] != n + 1:
            raise ValueError("offset must have len(types) + 1 entries")
        table = positions is not None and image is not None and shifts is not None
        if (rij is not None) == (positions is not None or image is not None or shifts is not None) or \
                (rij is None and not table):
            raise ValueError("give rij or positions, image and shifts")
        rij = None if rij is None else np.ascontiguousarray(rij, dtype=np.float64).reshape(-1, 3)
        positions = None if positions is None else np.ascontiguousarray(positions, dtype=np.float64).reshape(-1, 3)
        image = as_array(image, np.int32)
        shifts = None if shifts is None else np.ascontiguousarray(shifts, dtype=np.float64).reshape(-1, 3)
        if n and offset[-1] != j.shape[0]:
            raise ValueError("offset[0] must be 0 and offset[-1] == len(j)")
        if rij is not None and rij.shape[0] != j.shape[0]:
            raise ValueError("j and rij differ in length")
        if image is not None and image.shape[0] != j.shape[0]:
            raise ValueError("j and image differ in length")
        if positions is not None and positions.shape[0] != n:
            raise ValueError("positions must have len(types) rows")
        if shifts is not None and shifts.shape[0] == 0:
            shifts = np.zeros((1, 3))
            nimg = 0
        else:
            nimg = 0 if shifts is None else shifts.shape[0]
        return n, (types, offset, j, rij, positions, image, shifts), nimg

    def compute_lammps(self, nlocal, types, x, ilist, numneigh, firstneigh, owner=None, neighmask=0x1FFFFFFF, energies=False,
                       energy_only=False, forces=None, eatom=None, vatom=None, cvatom=None):
        """The call of a LAMMPS pair style (gr_compute_lammps): owned + ghost atoms `x[nall, 3]`, `types[nall]`, the full
        neighbour list as `numneigh[nlocal]` and a list of index arrays `firstneigh[i]`, `owner[nall]` the owned atom of every
        ghost.  Forces are ADDED to `forces[nall, 3]` (zeros when not given), per-atom energies to `eatom[nall]`, per-atom
        virials to `vatom[nall, 6]` and, in the centroid form xx yy zz xy xz yz yx zx zy, to `cvatom[nall, 9]` when given."""
        types = as_array(types, np.int32)
        x = as_array(x, np.float64, 3)
        nall = types.shape[0]
        ilist = as_array(ilist, np.int32)
        numneigh = as_array(numneigh, np.int32)
        rows = [np.ascontiguousarray(r, dtype=np.int32) for r in firstneigh]
        fn = (C.c_void_p * max(len(rows), 1))(*[r.ctypes.data if r.size else None for r in rows])
        own = as_array(owner, np.int32) if owner is not None else None
        f = np.zeros((nall, 3)) if forces is None else forces
        ea = (np.zeros(nall) if eatom is None else eatom) if energies else None
        e, v = C.c_double(), np.zeros(6)
        want_v = vatom is not None or cvatom is not None
        flags = (FLAG_ENERGY_ONLY if energy_only else 0) | (FLAG_EATOM if energies else 0) | (_lib.FLAG_VATOM if want_v else 0)
        check(_lib.lib().gr_compute_lammps(self._h, int(nlocal), nall, ptr(types), ptr(x), ilist.shape[0], ptr(ilist), ptr(numneigh), fn,
                                           int(neighmask), ptr(own) if own is not None else None, flags, C.byref(e),
                                           None if energy_only else ptr(f), ptr(v), ptr(ea) if ea is not None else None))
        out = {"energy": e.value}
        if vatom is not None:
            check(_lib.lib().gr_lammps_add_vatom(self._h, nall, ptr(vatom)))
            out["vatom"] = vatom
        if cvatom is not None:
            check(_lib.lib().gr_lammps_add_cvatom(self._h, nall, ptr(cvatom)))
            out["cvatom"] = cvatom
        if not energy_only:
            out["forces"], out["virial"] = f, v
        if energies:
            out["energies"] = ea
        return out

    def compute_lammps_device(self, nlocal, types, x, ilist, numneigh, neighbors, owner=None, neighmask=0x1FFFFFFF, energy_only=False,
                              forces=None, eatom=None, same_list=False, vatom=None, cvatom=None):
        """The call of a KOKKOS pair style (gr_compute_lammps_device): every array is a device array of the module's GPU
        (torch tensors): `types[nall]` int32, `x[nall, 3]`, `ilist[inum]`, `numneigh[nlocal]`, the 2-d neighbour view
        `neighbors[nlocal, maxneigh]` in either layout, `owner[nall]`.  Forces are ADDED to `forces[nall, 3]` and per-atom
        energies to `eatom[nall]` in place; energy and virial come back on the host.  `same_list`: the arrays are those
        of the previous call and only the contents of `x` changed (the steps between two reneighbourings): the converted
        list is kept and only its bond vectors are renewed."""
        nall, inum = int(types.shape[0]), int(ilist.shape[0])
        p_t = _device_pointer(types, "types", (nall,), "int32")
        p_x = _device_pointer(x, "x", (nall, 3), "float64")
        p_il = _device_pointer(ilist, "ilist", (inum,), "int32")
        p_nn = _device_pointer(numneigh, "numneigh", (int(numneigh.shape[0]),), "int32")
        if numneigh.shape[0] < nlocal or neighbors.dim() != 2 or neighbors.shape[0] < nlocal or str(neighbors.dtype) != "torch.int32" or \
                neighbors.device != types.device:
            raise ValueError("neighbors: expected an int32 device array [nlocal, maxneigh]")
        p_own = _device_pointer(owner, "owner", (nall,), "int32") if owner is not None else None
        p_f = _device_pointer(forces, "forces", (nall, 3), "float64") if forces is not None else None
        p_ea = _device_pointer(eatom, "eatom", (nall,), "float64") if eatom is not None else None
        e, v = C.c_double(), np.zeros(6)
        flags = (FLAG_ENERGY_ONLY if energy_only else 0) | (FLAG_EATOM if eatom is not None else 0) | (_lib.FLAG_SAME_LIST if same_list else 0) | \
            (_lib.FLAG_VATOM if vatom is not None or cvatom is not None else 0)
        p_va = _device_pointer(vatom, "vatom", (nall, 6), "float64") if vatom is not None else None
        p_cva = _device_pointer(cvatom, "cvatom", (nall, 9), "float64") if cvatom is not None else None
        check(_lib.lib().gr_compute_lammps_device(self._h, int(nlocal), nall, len(self.species), p_t, p_x, inum, p_il, p_nn,
                                                  C.c_void_p(neighbors.data_ptr()), int(neighbors.stride(0)), int(neighbors.stride(1)),
                                                  int(neighmask), p_own, flags, C.byref(e), None if energy_only else p_f, ptr(v), p_ea))
        if vatom is not None:
            check(_lib.lib().gr_lammps_add_vatom_device(self._h, nall, p_va))
        if cvatom is not None:
            check(_lib.lib().gr_lammps_add_cvatom_device(self._h, nall, p_cva))
        out = {"energy": e.value}
        if not energy_only:
            out["virial"] = v
        return out

    def compute(self, types, offset, j, rij=None, energies=False, energy_only=False, positions=None, image=None,
                shifts=None, add_to=None):
        """add_to: a result of an earlier call (energy, forces, virial, energies) that this call's outputs are ADDED to,
        as the reference's Outputs accumulate"""
        n, arrs, nimg = self._csr_args(types, offset, j, rij, positions, image, shifts)
        flags = (FLAG_ENERGY_ONLY if energy_only else 0) | (FLAG_EATOM if energies else 0)
        e = C.c_double(0.0)
        f, v, ea = np.zeros((n, 3)), np.zeros(6), np.zeros(n)
        if add_to is not None:
            flags |= _lib.FLAG_ACCUMULATE
            e = C.c_double(float(add_to["energy"]))
            f, v = np.array(add_to.get("forces", f), dtype=np.float64), np.array(add_to.get("virial", v), dtype=np.float64)
            ea = np.array(add_to.get("energies", ea), dtype=np.float64)
        check(_lib.lib().gr_compute_csr(self._h, n, *[ptr(a) for a in arrs], nimg, flags, C.addressof(e), ptr(f), ptr(v),
                                        ptr(ea) if energies else None))
        out = {"energy": e.value}
        if not energy_only:
            out["forces"], out["virial"] = f, v
        if energies:
            out["energies"] = ea
        return out

    def upload(self, types, offset, j, rij=None, positions=None, image=None, shifts=None):
        n, arrs, nimg = self._csr_args(types, offset, j, rij, positions, image, shifts)
        check(_lib.lib().gr_engine_upload(self._h, n, *[ptr(a) for a in arrs], nimg))
        self._n = n

    def run(self, energies=False, energy_only=False, uq=False, virials=False):
        flags = (FLAG_ENERGY_ONLY if energy_only else 0) | (FLAG_EATOM if energies else 0) | (FLAG_UQ if uq else 0) | \
            (_lib.FLAG_VATOM if virials else 0)
        check(_lib.lib().gr_engine_run(self._h, flags))

    def fetch_vatom(self, rows=None):
        """per-atom virials [rows, 6] = xx yy zz xy xz yz of the last run(virials=True), in the order of the uploaded list
        (Outputs::vatom, libgrace/include/grace/system.h:71): half of every bond's virial to each of its two atoms"""
        v = np.zeros((self._n if rows is None else int(rows), 6))
        check(_lib.lib().gr_engine_fetch_vatom(self._h, ptr(v)))
        return v

    def fetch_cvatom(self, rows=None):
        """the same rows in the centroid form [rows, 9] = xx yy zz xy xz yz yx zx zy (cvatom of the reference's GPU engines,
        libgrace/include/grace/kk/grace_1l_kk.h:94)"""
        v = np.zeros((self._n if rows is None else int(rows), 9))
        check(_lib.lib().gr_engine_fetch_cvatom(self._h, ptr(v)))
        return v

    def fetch_uq(self):
        """gamma, atomic_sigma, gmm_cluster [n] of the last run(uq=True), in the order of the uploaded list"""
        n = self._n
        g, sg, cl = np.empty(n), np.empty(n), np.empty(n)
        check(_lib.lib().gr_engine_fetch_uq(self._h, ptr(g), ptr(sg), ptr(cl)))
        return {"gamma": g, "atomic_sigma": sg, "gmm_cluster": cl}

    def sync(self):
        check(_lib.lib().gr_engine_sync(self._h))

    def fetch(self, energies=False):
        n = self._n
        e = C.c_double(0.0)
        f, v, ea = np.zeros((n, 3)), np.zeros(6), np.zeros(n)
        check(_lib.lib().gr_engine_fetch(self._h, C.addressof(e), ptr(f), ptr(v), ptr(ea) if energies else None))
        out = {"energy": e.value, "forces": f, "virial": v}
        if energies:
            out["energies"] = ea
        return out

    def edge_count(self) -> int:
        return int(_lib.lib().gr_engine_edge_count(self._h))

    def set_profile(self, on=True):
        check(_lib.lib().gr_engine_set_profile(self._h, int(bool(on))))

    def stage_times(self):
        """{stage: (milliseconds, launches)} of the last run (HIP events on the engine's stream)"""
        L = _lib.lib()
        n = L.gr_engine_stage_count(self._h)
        if n < 0:
            check(_lib.GR_ERROR)
        out = {}
        buf = C.create_string_buffer(64)
        for k in range(n):
            ms, cnt = C.c_double(0.0), C.c_int(0)
            check(L.gr_engine_stage_get(self._h, k, buf, 64, C.byref(ms), C.byref(cnt)))
            out[buf.value.decode()] = (ms.value, cnt.value)
        return out

    def stage_flops(self):
        """{stage: flops of its tile GEMMs in the last run} (stages without tile GEMMs are left out)"""
        L = _lib.lib()
        out = {}
        buf = C.create_string_buffer(64)
        for k in range(max(L.gr_engine_stage_count(self._h), 0)):
            ms, cnt, fl = C.c_double(0.0), C.c_int(0), C.c_double(0.0)
            check(L.gr_engine_stage_get(self._h, k, buf, 64, C.byref(ms), C.byref(cnt)))
            check(L.gr_engine_stage_flops(self._h, k, C.byref(fl)))
            if fl.value > 0:
                out[buf.value.decode()] = fl.value
        return out

    def upload_batch(self, structures, cutoff=None):
        """Several independent periodic structures [(positions, cell, types), ...] as ONE resident list (host neighbour
        lists, gr_engine_upload_batch): run() then evaluates all of them in one pass, fetch_batch() returns energy [S],
        virial [S, 6], forces [N, 3] in the order of the uploaded lists (perm of every structure is returned)."""
        rc = float(self.cutoff_matrix().max()) if cutoff is None else float(cutoff)
        tt, off, jj, xx, im, sh, sid, perms = [], [np.zeros(1, np.int64)], [], [], [], [], [], []
        a0 = b0 = s0 = 0
        for k, (pos, cell, types) in enumerate(structures):
            perm, offset, j, image, shifts = neighbor_search(pos, cell, [True, True, True], rc)
            tt.append(np.asarray(types, np.int32)[perm]); xx.append(np.asarray(pos)[perm]); perms.append(perm)
            off.append(offset[1:] + b0); jj.append(j + a0); im.append(image + s0); sh.append(shifts.reshape(-1, 3))
            sid.append(np.full(len(perm), k, np.int32))
            a0 += len(perm); b0 += len(j); s0 += len(shifts)
        types, offset, j = np.concatenate(tt), np.concatenate(off), np.concatenate(jj).astype(np.int32)
        n, arrs, nimg = self._csr_args(types, offset, j, None, np.concatenate(xx), np.concatenate(im).astype(np.int32), np.concatenate(sh))
        sid = np.concatenate(sid)
        check(_lib.lib().gr_engine_upload_batch(self._h, n, *[ptr(a) for a in arrs], nimg, len(structures), ptr(sid)))
        self._n, self._nstruct = n, len(structures)
        return perms

    def fetch_batch(self):
        n, S = self._n, self._nstruct
        e, f, v = np.zeros(S), np.zeros((n, 3)), np.zeros((S, 6))
        check(_lib.lib().gr_engine_fetch_batch(self._h, S, ptr(e), ptr(f), ptr(v), None))
        return {"energy": e, "forces": f, "virial": v}

    def debug_radial(self, x, mu_j):
        x = as_array(x, np.float64)
        mu_j = as_array(mu_j, np.int32)
        nl, Cn = self.model.lmax + 1, self.model.n_radial
        R, dR = np.zeros((x.shape[0], nl, Cn)), np.zeros((x.shape[0], nl, Cn))
        check(_lib.lib().gr_engine_debug_radial(self._h, x.shape[0], ptr(x), ptr(mu_j), ptr(R), ptr(dR)))
        return R, dR

    def radial_noalloc(self, x, mu_j, R, dR):
        """debug_radial on device arrays of the module's GPU (x [m] float64, mu_j [m] int32, R and dR [m, lmax + 1,
        n_radial] float64, written in place) through the entry point that allocates no device memory."""
        m = int(x.shape[0])
        nl, Cn = self.model.lmax + 1, self.model.n_radial
        check(_lib.lib().gr_engine_radial_noalloc(self._h, m, _device_pointer(x, "x", (m,), "float64"),
                                                  _device_pointer(mu_j, "mu_j", (m,), "int32"),
                                                  _device_pointer(R, "R", (m, nl, Cn), "float64"),
                                                  _device_pointer(dR, "dR", (m, nl, Cn), "float64")))

    def debug_copy(self, nbytes):
        check(_lib.lib().gr_engine_debug_copy(self._h, int(nbytes)))

    def stream_rates(self, nbytes=1 << 30):
        """(copy GB/s counting bytes read + written, read-only GB/s) of two plain stream kernels over nbytes: the HBM
        rates this GPU shows to a kernel that moves memory and does nothing else"""
        c, r = C.c_double(), C.c_double()
        check(_lib.lib().gr_engine_stream_rates(self._h, int(nbytes), C.byref(c), C.byref(r)))
        return c.value, r.value

    def close(self):
        if getattr(self, "_h", None):
            _lib.lib().gr_engine_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _padded_cell_arrays(cell, pos, reach, pbc=None):
    """A full-rank box for a structure with open directions (what the reference does before its search,
    python/grace_runtime/neighbors.py:27-47): every cell vector that is zero or whose direction is not periodic is replaced
    by a unit normal to the remaining vectors, scaled to the extent of the atoms along it plus 2 * reach + 1, so that no
    image lies within reach.  Returns the box and the translation that moves the atoms inside it.  The same construction as
    the library uses for gr_compute / gr_system_compute."""
    box = np.array(cell, dtype=np.float64).reshape(3, 3)
    pos = np.asarray(pos, dtype=np.float64).reshape(-1, 3)
    is_open = [not box[k].any() or (pbc is not None and not pbc[k]) for k in range(3)]
    kept = [box[k] for k in range(3) if not is_open[k]]
    if len(kept) == 3:
        return box, np.zeros(3)

    def unit(v):
        length = np.sqrt(v @ v)
        if not length > 0.0:
            raise ValueError("the periodic cell vectors are linearly dependent")
        return v / length

    if not kept:
        normals = list(np.eye(3))
    elif len(kept) == 2:
        normals = [unit(np.cross(kept[0], kept[1]))]
    else:
        a = unit(kept[0])
        e = np.zeros(3)
        e[int(np.argmin(np.abs(a)))] = 1.0        # the axis least aligned with the one periodic vector
        b = unit(np.cross(a, e))
        normals = [b, unit(np.cross(a, b))]
    move = np.zeros(3)
    for k, d in zip([k for k in range(3) if is_open[k]], normals):
        along = pos @ d if len(pos) else np.zeros(1)
        box[k] = d * ((along.max() - along.min()) + 2.0 * reach + 1.0)
        if len(pos):
            move += d * (reach + 0.5 - along.min())
    return box, move


class System:
    """One structure on the device with a Verlet list at cutoff + skin, rebuilt when an atom moved more than
    skin / 2 or the atoms / cell / pbc change (python/kk/kk_api.h:66-93, list policy python/grace_runtime/
    neighbors.py:68-89).  The list lives on the device (gr_system_*): its pair search runs there, and calls between
    rebuilds send positions only."""

    def __init__(self, model: Model, species, skin: float = 0.5, spline: int = 0, chunksize: int = -1,
                 precision: int = 64):
        """spline: intervals of the radial tables of GRACE-1L / 2L engines (the reference's engines always use tables,
        1024 intervals unless told otherwise: docs/advanced.md:34); 0, the default HERE: the radial MLP is evaluated for
        every bond, without interpolation error.  The reference's calculator passes its model's spline (1024)."""
        skin = float(skin)
        if not (np.isfinite(skin) and skin >= 0.0):
            raise ValueError(f"skin must be a finite number >= 0, got {skin!r}")
        self.engine = Engine(model, species, precision)
        self.engine.set_spline(int(spline))
        self.skin = skin
        self.cutoff = float(self.engine.cutoff_matrix().max()) if len(species) else 0.0
        self._h = C.c_void_p()
        check(_lib.lib().gr_system_create(self.engine._h, skin, C.byref(self._h)))
        # atoms per engine pass: 0 one pass, < 0 from the free device memory, > 0 as given (ValueError for a model kind
        # that is evaluated in one pass only)
        check(_lib.lib().gr_system_set_chunksize(self._h, int(chunksize)))

    def __del__(self):
        if getattr(self, "_h", None) is not None and self._h.value:
            _lib.lib().gr_system_free(self._h)
            self._h = C.c_void_p()

    @property
    def rebuilds(self) -> int:
        return int(_lib.lib().gr_system_rebuilds(self._h))

    @property
    def chunksize(self) -> int:
        """atoms per engine pass in the last compute (0: one pass), python/kk/kk_api.h:86"""
        return int(_lib.lib().gr_system_chunksize(self._h))

    @property
    def list_on_device(self) -> bool:
        """True when the list of the last rebuild was searched on the device."""
        return bool(_lib.lib().gr_system_list_on_device(self._h))

    def release_buffers(self):
        """frees the engine's work buffers (python/kk/kk_api.h:66-93); the next compute builds its list again"""
        self.engine.release_buffers()

    def set_dispersion(self, *a, **k):
        raise ValueError("dispersion corrections are not part of this engine")

    def neighbor_list(self):
        """(perm, offset, j, image, shifts) of the last rebuild, as neighbor_search returns them."""
        nb, nimg = C.c_int64(), C.c_int64()
        check(_lib.lib().gr_system_list_sizes(self._h, C.byref(nb), C.byref(nimg)))
        n = self._n
        perm, offset = np.empty(n, np.int64), np.empty(n + 1, np.int64)
        j, image = np.empty(nb.value, np.int32), np.empty(nb.value, np.int32)
        shifts = np.empty((nimg.value, 3))
        check(_lib.lib().gr_system_list_get(self._h, ptr(perm), ptr(offset), ptr(j), ptr(image), ptr(shifts)))
        return perm, offset, j, image, shifts

    def compute(self, types, positions, cell, pbc, energies=False, uq=False, energy_only=False, virials=False):
        """energy, forces [n, 3], virial [6], energies [n]; with `uq` also gamma, atomic_sigma, gmm_cluster [n] of the
        model's UQ head (ValueError when the model has none that can be evaluated); with `virials` the per-atom virials
        [n, 6] (the reference's vatom) and `centroid_virials` [n, 9] = xx yy zz xy xz yz yx zx zy (its cvatom)."""
        types = as_array(types, np.int32)
        pos = np.ascontiguousarray(positions, dtype=np.float64).reshape(-1, 3)
        cell = np.ascontiguousarray(cell, dtype=np.float64).reshape(3, 3)
        pb = np.ascontiguousarray([1 if p else 0 for p in pbc], dtype=np.uint8)
        n = types.shape[0]
        if pos.shape[0] != n:
            raise ValueError("positions must have len(types) rows")
        if n and (types.min() < 1 or types.max() > len(self.engine.species)):
            raise ValueError("types must be 1 .. len(species)")
        self._n = n
        e = C.c_double()
        forces = None if energy_only else np.empty((n, 3))
        virial = None if energy_only else np.empty(6)
        eat = np.empty(n) if energies else None
        flags = (FLAG_ENERGY_ONLY if energy_only else 0) | (FLAG_EATOM if energies else 0) | (FLAG_UQ if uq else 0) | \
            (_lib.FLAG_VATOM if virials and not energy_only else 0)
        check(_lib.lib().gr_system_compute(self._h, n, ptr(types), ptr(pos), ptr(cell), ptr(pb), flags, C.byref(e),
                                      ptr(forces) if forces is not None else None, ptr(virial) if virial is not None else None,
                                      ptr(eat) if eat is not None else None))
        res = {"energy": e.value}
        if not energy_only:
            res["forces"], res["virial"] = forces, virial
        if energies:
            res["energies"] = eat
        if uq:
            g, sg, cl = np.empty(n), np.empty(n), np.empty(n)
            check(_lib.lib().gr_system_fetch_uq(self._h, ptr(g), ptr(sg), ptr(cl)))
            res["gamma"], res["atomic_sigma"], res["gmm_cluster"] = g, sg, cl
        if virials and not energy_only:
            va = np.zeros((n, 6))
            check(_lib.lib().gr_system_fetch_vatom(self._h, ptr(va)))
            res["virials"] = va
            cva = np.zeros((n, 9))
            check(_lib.lib().gr_system_fetch_cvatom(self._h, ptr(cva)))
            res["centroid_virials"] = cva
        return res


class Batch:
    """Many structures per call (python/kk/kk_api.h:116-156): energy [S], virial [S, 6], forces [N, 3] in input
    order.  All structures are packed into one atom list and evaluated in one engine pass."""

    def __init__(self, model: Model, species, spline: int = 0, chunksize: int = -1, precision: int = 64):
        """spline: as for System (0: the radial MLP itself; n: radial tables of n intervals, the reference's default is 1024)"""
        self.engine = Engine(model, species, precision)
        self.engine.set_spline(int(spline))
        self.cutoff = float(self.engine.cutoff_matrix().max()) if len(species) else 0.0
        self.passes = 0
        self.keep_buffers = False
        self.engine.set_chunksize(int(chunksize))    # atoms per engine pass within a batch pass (0 one pass, < 0 automatic)
        self._nall_cap = 1 << 62    # atoms per pass after an allocation failure (python/kk/kk_core.cpp:1461: nall_cap)

    @property
    def chunksize(self) -> int:
        """atoms per engine pass in the last compute (0: one pass)"""
        return self.engine.chunksize

    def release_buffers(self):
        """frees the engine's work buffers (python/kk/kk_api.h:116-156)"""
        self.engine.release_buffers()

    def _done(self):
        # a batch is a job: its device memory goes back after the call unless keep_buffers is set (an MD loop over the
        # same batch), python/kk/kk_core.cpp:1466-1469
        if not self.keep_buffers:
            self.release_buffers()

    def compute(self, natoms, types, positions, cells, pbc, energies=False, uq=False, energy_only=False,
                max_nall=1 << 21, dispersion_parts=False):
        if uq and not self.engine.model.has_uq:
            raise ValueError("uq=True: the model has no UQ head")
        natoms = np.asarray(natoms, dtype=np.int32)
        types = as_array(types, np.int32)
        pos = np.ascontiguousarray(positions, dtype=np.float64).reshape(-1, 3)
        cells = np.ascontiguousarray(cells, dtype=np.float64).reshape(-1, 3, 3)
        pbc = np.ascontiguousarray(pbc, dtype=bool).reshape(-1, 3)
        S = natoms.shape[0]
        if cells.shape[0] != S or pbc.shape[0] != S or natoms.sum() != types.shape[0] or pos.shape[0] != types.shape[0]:
            raise ValueError("natoms, types, positions, cells and pbc do not describe the same structures")
        if types.size and (types.min() < 1 or types.max() > len(self.engine.species)):
            raise ValueError("types must be 1 .. len(species)")
        if int(max_nall) < 1:
            raise ValueError("max_nall must be >= 1")
        N = types.shape[0]
        out = {"energy": np.zeros(S)}
        f, v = np.zeros((N, 3)), np.zeros((S, 6))
        ea = np.zeros(N) if energies else None
        ug, us, uc = (np.zeros(N), np.zeros(N), np.zeros(N)) if uq else (None, None, None)
        pb = np.ascontiguousarray(pbc, dtype=np.uint8)
        flags = (FLAG_ENERGY_ONLY if energy_only else 0) | (FLAG_EATOM if energies else 0)
        nth = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else 1
        # every structure's list is built on the host (in parallel); the structures go through the GPU in passes of whole
        # structures with at most max_nall atoms (python/kk/kk_core.cpp:1311-1347: ONE pass unless the batch is larger)
        start = np.concatenate([[0], np.cumsum(natoms, dtype=np.int64)])
        # after an allocation failure: a fresh engine and passes of half as many atoms, down to 16384, from the first
        # structure again (every pass overwrites its outputs); python/kk/kk_core.cpp:1452-1484 compute_with_retry
        limit = min(int(max_nall), self._nall_cap)
        while True:
            try:
                self.passes, g0 = 0, 0
                while g0 < S:
                    g1 = g0 + 1
                    # what the device memory holds, once a pass has shown the engine's bytes per atom
                    fit = min(limit, int(_lib.lib().gr_engine_atoms_that_fit(self.engine._h)))
                    while g1 < S and start[g1 + 1] - start[g0] <= fit:
                        g1 += 1
                    a0, a1 = int(start[g0]), int(start[g1])
                    check(_lib.lib().gr_compute_batch_uq(self.engine._h, g1 - g0, ptr(natoms[g0:g1]), ptr(types[a0:a1]), ptr(pos[a0:a1]),
                                                         ptr(cells[g0:g1]), ptr(pb[g0:g1]), flags, min(nth, 16), ptr(out["energy"][g0:g1]),
                                                         ptr(f[a0:a1]), ptr(v[g0:g1]), ptr(ea[a0:a1]) if energies else None,
                                                         ptr(ug[a0:a1]) if uq else None, ptr(us[a0:a1]) if uq else None,
                                                         ptr(uc[a0:a1]) if uq else None))
                    self.passes += 1 if a1 > a0 else 0
                    g0 = g1
                break
            except MemoryError:
                tried = min(limit, N)
                self.engine.reset()
                if tried <= 16384:
                    raise RuntimeError(f"the batch ({N} atoms) does not fit the GPU memory even in passes of {tried} atoms; "
                                       "use a GPU with more memory") from None
                limit = self._nall_cap = max(16384, tried // 2)
        self._done()
        if not energy_only:
            out["forces"], out["virial"] = f, v
        if energies:
            out["energies"] = ea
        if uq:
            out["gamma"], out["atomic_sigma"], out["gmm_cluster"] = ug, us, uc
        return out

    def compute_device(self, natoms, types, positions, cells, pbc, energy, forces=None, virial=None, energies=None,
                       gamma=None, atomic_sigma=None, gmm_cluster=None, energy_only=False, max_nall=1 << 21):
        """`Batch.compute_device` of the reference module (python/kk/kk_module.cpp:142-193): `types` int32 [N],
        `positions` float64 [N, 3] and the outputs `energy` [S], `forces` [N, 3], `virial` [S, 6], `energies` [N] are
        arrays ON the module's GPU (torch tensors, or anything with `__cuda_array_interface__` such as CuPy arrays),
        read and written in place; `natoms`, `cells`, `pbc` are host arrays.  `gamma`, `atomic_sigma`, `gmm_cluster`
        (float64 [N] on the GPU, each optional) receive the UQ head's outputs.  The neighbour lists are built on the
        device; positions, forces and energies never visit the host.  `max_nall`: atoms per engine pass (whole
        structures, at least one per pass); `passes` holds the number of passes made."""
        if (gamma is not None or atomic_sigma is not None or gmm_cluster is not None) and not self.engine.model.has_uq:
            raise ValueError("gamma / atomic_sigma / gmm_cluster: the model has no UQ head")
        natoms = np.ascontiguousarray(natoms, dtype=np.int32)
        cells = np.ascontiguousarray(cells, dtype=np.float64).reshape(-1, 3, 3)
        pb = np.ascontiguousarray(np.asarray(pbc, dtype=bool).reshape(-1, 3), dtype=np.uint8)
        S, N = natoms.shape[0], int(natoms.sum())
        if cells.shape[0] != S or pb.shape[0] != S:
            raise ValueError("natoms, cells and pbc differ in length")
        p_types = _device_pointer(types, "types", (N,), "int32")
        p_pos = _device_pointer(positions, "positions", (N, 3), "float64")
        p_e = _device_pointer(energy, "energy", (S,), "float64")
        p_f = _device_pointer(forces, "forces", (N, 3), "float64") if forces is not None else None
        p_v = _device_pointer(virial, "virial", (S, 6), "float64") if virial is not None else None
        p_ea = _device_pointer(energies, "energies", (N,), "float64") if energies is not None else None
        p_uq = [_device_pointer(a, nm, (N,), "float64") if a is not None else None
                for a, nm in ((gamma, "gamma"), (atomic_sigma, "atomic_sigma"), (gmm_cluster, "gmm_cluster"))]
        flags = (FLAG_ENERGY_ONLY if energy_only else 0) | (FLAG_EATOM if energies is not None else 0)
        if int(max_nall) < 1:
            raise ValueError("max_nall must be >= 1")
        passes = C.c_int(0)
        check(_lib.lib().gr_compute_batch_device_uq(self.engine._h, S, ptr(natoms), p_types, p_pos, ptr(cells), ptr(pb), flags, int(max_nall),
                                                    p_e, p_f, p_v, p_ea, p_uq[0], p_uq[1], p_uq[2], C.byref(passes)))
        self.passes = passes.value if N else 0
        self._done()


_CAI_TYPES = {"int32": "<i4", "float64": "<f8"}


def _device_pointer(a, name, shape, dtype):
    """Address of a C-contiguous device array of the given shape and dtype on the module's GPU (torch tensor or
    `__cuda_array_interface__`); ValueError otherwise, with the reference's messages (python/kk/kk_module.cpp:129-134)."""
    where = f"{name} must be on the module's GPU ({PLATFORM}:{_dev()})"
    if hasattr(a, "data_ptr") and hasattr(a, "is_contiguous"):    # torch
        if a.device.type != "cuda" or (a.device.index or 0) != _dev():
            raise ValueError(where)
        if str(a.dtype).split(".")[-1] != dtype or tuple(a.shape) != tuple(shape) or not a.is_contiguous():
            raise ValueError(f"{name}: expected a contiguous {dtype} array of shape {tuple(shape)}")
        return C.c_void_p(a.data_ptr() if a.numel() else 0)
    cai = getattr(a, "__cuda_array_interface__", None)
    if cai is None and hasattr(a, "__dlpack__"):    # any other DLPack exporter: through torch, without a copy
        try:
            import torch
            return _device_pointer(torch.from_dlpack(a), name, shape, dtype)
        except ImportError:
            pass
    if cai is None:
        raise ValueError(where)
    if cai["typestr"] != _CAI_TYPES[dtype] or tuple(cai["shape"]) != tuple(shape) or cai.get("strides") is not None:
        raise ValueError(f"{name}: expected a contiguous {dtype} array of shape {tuple(shape)}")
    return C.c_void_p(cai["data"][0])

