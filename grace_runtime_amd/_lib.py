"""ctypes binding of libgrace_hip.so (the C ABI declared in include/grace_hip.h).

The library is loaded from this package directory (built in-tree by grace_runtime_amd/csrc/Makefile).  There is no
fallback: without the library, or without a GPU, every compute entry point raises."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgrace_hip.so")

GR_OK, GR_INVALID, GR_ERROR, GR_NOMEM = 0, 1, 2, 3
FLAG_ENERGY_ONLY, FLAG_EATOM, FLAG_UQ, FLAG_ACCUMULATE, FLAG_SAME_LIST, FLAG_VATOM = 1, 2, 4, 8, 16, 32

# every symbol include/grace_hip.h declares (checked by the CPU test-suite against the header and the library)
SYMBOLS = [
    "gr_last_error", "gr_set_logger", "gr_abi_version", "gr_device_count", "gr_device_arch", "gr_model_load", "gr_model_get_info",
    "gr_model_element_name", "gr_model_free", "gr_engine_create", "gr_engine_free", "gr_engine_cutoff",
    "gr_compute_csr", "gr_engine_upload", "gr_engine_run", "gr_engine_sync", "gr_engine_fetch",
    "gr_engine_edge_count", "gr_engine_set_profile", "gr_engine_stage_count", "gr_engine_stage_get", "gr_engine_stage_flops",
    "gr_engine_debug_radial", "gr_engine_radial_noalloc", "gr_engine_debug_copy", "gr_engine_stream_rates", "gr_engine_fetch_vatom", "gr_system_fetch_vatom", "gr_lammps_add_vatom",
    "gr_lammps_add_vatom_device", "gr_neighbor_build", "gr_nlist_nbonds", "gr_nlist_nimages", "gr_nlist_get",
    "gr_nlist_free", "gr_compute", "gr_compute_batch", "gr_engine_upload_batch", "gr_engine_fetch_batch",
    "gr_system_create", "gr_system_free", "gr_system_compute", "gr_system_rebuilds", "gr_system_list_on_device",
    "gr_system_list_sizes", "gr_system_list_get", "gr_compute_lammps", "gr_compute_batch_device", "gr_compute_batch_uq", "gr_compute_batch_device_uq", "gr_engine_reset", "gr_engine_release_buffers", "gr_set_memory_limit", "gr_memory_in_use", "gr_compute_lammps_device", "gr_model_has_uq", "gr_model_validate_uq", "gr_engine_fetch_uq",
    "gr_system_fetch_uq", "gr_engine_atoms_that_fit", "gr_engine_set_exchange", "gr_engine_comm_layers", "gr_engine_comm_width", "gr_engine_pack_forward", "gr_engine_unpack_forward", "gr_engine_pack_reverse", "gr_engine_unpack_reverse", "gr_engine_pack_forward_host", "gr_engine_unpack_forward_host", "gr_engine_pack_reverse_host", "gr_engine_unpack_reverse_host", "gr_engine_set_chunksize", "gr_engine_chunksize", "gr_system_set_chunksize", "gr_system_chunksize",
    "gr_engine_set_ordered_sums", "gr_engine_ordered_sums", "gr_engine_fetch_cvatom", "gr_system_fetch_cvatom", "gr_lammps_add_cvatom",
    "gr_lammps_add_cvatom_device", "gr_engine_set_spline", "gr_engine_spline",
]


class ModelInfo(C.Structure):
    _fields_ = [("layers", C.c_int), ("n_elements", C.c_int), ("lmax", C.c_int), ("n_radial", C.c_int),
                ("n_radbase", C.c_int), ("max_order", C.c_int), ("rcut", C.c_double)]


_lib = None


def lib():
    """The loaded library; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `make -C grace_runtime_amd/csrc` "
                           "(there is no CPU fallback in this package)")
    # One HIP runtime per process.  PyTorch ships a copy of its own: when PyTorch is installed it is imported BEFORE
    # the library is opened, so that the library binds to the runtime PyTorch uses and device arrays can be shared
    # (Batch.compute_device).  With the library opened first, PyTorch would bring up a second runtime and find no GPU.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(LIB_PATH)
    vp, i32, i64, dbl, u32 = C.c_void_p, C.c_int, C.c_int64, C.c_double, C.c_uint
    L.gr_last_error.restype = C.c_char_p
    L.gr_set_logger.restype = None
    L.gr_set_logger.argtypes = [vp, vp]
    L.gr_abi_version.restype = i32
    L.gr_device_count.restype = i32
    L.gr_device_arch.argtypes = [i32, C.c_char_p, i32]
    L.gr_model_load.argtypes = [C.c_char_p, C.POINTER(vp)]
    L.gr_model_get_info.argtypes = [vp, C.POINTER(ModelInfo)]
    L.gr_model_element_name.restype = C.c_char_p
    L.gr_model_element_name.argtypes = [vp, i32]
    L.gr_model_free.argtypes = [vp]
    L.gr_engine_create.argtypes = [vp, i32, vp, i32, i32, C.POINTER(vp)]
    L.gr_engine_free.argtypes = [vp]
    L.gr_engine_reset.argtypes = [vp]
    L.gr_engine_release_buffers.argtypes = [vp]
    L.gr_set_memory_limit.restype = None
    L.gr_set_memory_limit.argtypes = [i64]
    L.gr_memory_in_use.restype = i64
    L.gr_memory_in_use.argtypes = []
    L.gr_engine_cutoff.restype = dbl
    L.gr_engine_cutoff.argtypes = [vp, i32, i32]
    L.gr_compute_csr.argtypes = [vp, i32, vp, vp, vp, vp, vp, vp, vp, i64, u32, vp, vp, vp, vp]
    L.gr_engine_upload.argtypes = [vp, i32, vp, vp, vp, vp, vp, vp, vp, i64]
    L.gr_engine_run.argtypes = [vp, u32]
    L.gr_engine_sync.argtypes = [vp]
    L.gr_engine_fetch.argtypes = [vp, vp, vp, vp, vp]
    L.gr_engine_edge_count.restype = i64
    L.gr_engine_edge_count.argtypes = [vp]
    L.gr_engine_set_profile.argtypes = [vp, i32]
    L.gr_engine_stage_count.argtypes = [vp]
    L.gr_engine_stage_get.argtypes = [vp, i32, C.c_char_p, i32, C.POINTER(dbl), C.POINTER(i32)]
    L.gr_engine_debug_radial.argtypes = [vp, i32, vp, vp, vp, vp]
    L.gr_engine_stage_flops.argtypes = [vp, i32, vp]
    L.gr_engine_set_chunksize.argtypes = [vp, i32]
    L.gr_engine_set_exchange.argtypes = [vp, vp]
    L.gr_engine_comm_layers.argtypes = [vp]
    L.gr_engine_comm_width.argtypes = [vp, i32]
    for name in ("gr_engine_pack_forward", "gr_engine_unpack_reverse", "gr_engine_pack_forward_host", "gr_engine_unpack_reverse_host"):
        getattr(L, name).argtypes = [vp, i32, i32, vp, vp]          # engine, layer, n, sendlist, buf
    for name in ("gr_engine_unpack_forward", "gr_engine_pack_reverse", "gr_engine_unpack_forward_host", "gr_engine_pack_reverse_host"):
        getattr(L, name).argtypes = [vp, i32, i32, i32, vp]         # engine, layer, n, first, buf
    L.gr_engine_atoms_that_fit.argtypes = [vp]
    L.gr_engine_atoms_that_fit.restype = i64
    L.gr_engine_chunksize.argtypes = [vp]
    L.gr_engine_set_ordered_sums.argtypes = [vp, i32]
    L.gr_engine_ordered_sums.argtypes = [vp]
    L.gr_engine_set_spline.argtypes = [vp, i32]
    L.gr_engine_spline.argtypes = [vp]
    L.gr_system_set_chunksize.argtypes = [vp, i32]
    L.gr_system_chunksize.argtypes = [vp]
    L.gr_engine_radial_noalloc.argtypes = [vp, i32, vp, vp, vp, vp]
    L.gr_engine_debug_copy.argtypes = [vp, i64]
    L.gr_engine_stream_rates.argtypes = [vp, i64, vp, vp]
    L.gr_engine_fetch_vatom.argtypes = [vp, vp]
    L.gr_system_fetch_vatom.argtypes = [vp, vp]
    L.gr_lammps_add_vatom.argtypes = [vp, i32, vp]
    L.gr_lammps_add_vatom_device.argtypes = [vp, i32, vp]
    L.gr_engine_fetch_cvatom.argtypes = [vp, vp]
    L.gr_system_fetch_cvatom.argtypes = [vp, vp]
    L.gr_lammps_add_cvatom.argtypes = [vp, i32, vp]
    L.gr_lammps_add_cvatom_device.argtypes = [vp, i32, vp]
    L.gr_neighbor_build.argtypes = [i64, vp, vp, vp, dbl, i32, C.POINTER(vp)]
    L.gr_nlist_nbonds.restype = i64
    L.gr_nlist_nbonds.argtypes = [vp]
    L.gr_nlist_nimages.restype = i64
    L.gr_nlist_nimages.argtypes = [vp]
    L.gr_nlist_get.argtypes = [vp, vp, vp, vp, vp, vp]
    L.gr_nlist_free.argtypes = [vp]
    L.gr_compute.argtypes = [vp, i32, vp, vp, vp, vp, u32, vp, vp, vp, vp]
    L.gr_compute_batch.argtypes = [vp, i32, vp, vp, vp, vp, vp, u32, i32, vp, vp, vp, vp]
    L.gr_engine_upload_batch.argtypes = [vp, i32, vp, vp, vp, vp, vp, vp, vp, i64, i32, vp]
    L.gr_engine_fetch_batch.argtypes = [vp, i32, vp, vp, vp, vp]
    L.gr_compute_batch_device.argtypes = [vp, i32, vp, vp, vp, vp, vp, u32, i64, vp, vp, vp, vp, vp]
    L.gr_compute_batch_uq.argtypes = [vp, i32, vp, vp, vp, vp, vp, u32, i32, vp, vp, vp, vp, vp, vp, vp]
    L.gr_compute_batch_device_uq.argtypes = [vp, i32, vp, vp, vp, vp, vp, u32, i64, vp, vp, vp, vp, vp, vp, vp, vp]
    L.gr_compute_lammps_device.argtypes = [vp, i32, i32, i32, vp, vp, i32, vp, vp, vp, i64, i64, i32, vp, u32, vp, vp, vp, vp]
    L.gr_model_has_uq.argtypes = [vp]
    L.gr_model_validate_uq.argtypes = [vp]
    L.gr_engine_fetch_uq.argtypes = [vp, vp, vp, vp]
    L.gr_system_fetch_uq.argtypes = [vp, vp, vp, vp]
    L.gr_compute_lammps.argtypes = [vp, i32, i32, vp, vp, i32, vp, vp, vp, i32, vp, u32, vp, vp, vp, vp]
    L.gr_system_create.argtypes = [vp, dbl, C.POINTER(vp)]
    L.gr_system_free.argtypes = [vp]
    L.gr_system_compute.argtypes = [vp, i32, vp, vp, vp, vp, u32, vp, vp, vp, vp]
    L.gr_system_rebuilds.argtypes = [vp]
    L.gr_system_list_on_device.argtypes = [vp]
    L.gr_system_list_sizes.argtypes = [vp, C.POINTER(i64), C.POINTER(i64)]
    L.gr_system_list_get.argtypes = [vp, vp, vp, vp, vp, vp]
    _lib = L
    return L


def check(status):
    """Status code -> exception, as the reference binding maps them (python/kk/kk_module.cpp: invalid_argument ->
    ValueError, everything else RuntimeError; allocation failure -> MemoryError)."""
    if status == GR_OK:
        return
    msg = lib().gr_last_error().decode(errors="replace")
    if status == GR_INVALID:
        raise ValueError(msg)
    if status == GR_NOMEM:
        raise MemoryError(msg)
    raise RuntimeError(msg)


def ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def as_array(a, dtype, shape_last=None):
    if a is None:
        return None
    a = np.ascontiguousarray(a, dtype=dtype)
    if shape_last is not None and (a.ndim != 2 or a.shape[1] != shape_last):
        raise ValueError(f"expected an array of shape (n, {shape_last})")
    return a
