"""ctypes bindings of the C ABI declared in include/shmt.h.

Thin and explicit: pointers are passed as integers (tensor.data_ptr()), the
stream as the raw hipStream_t of torch's current stream. The library must
have been built (python -m shmtensor_amd.build); there is no fallback path.
"""
import ctypes
import os

from .build import LIB_PATH

_c = ctypes
_vp, _i64, _int, _dbl = _c.c_void_p, _c.c_int64, _c.c_int, _c.c_double

SIGNATURES = {
    "shmt_abi_version": (_int, []),
    "shmt_last_error": (_c.c_char_p, []),
    "shmt_host_register": (_int, [_vp, _i64]),
    "shmt_host_unregister": (_int, [_vp]),
    "shmt_host_devptr": (_int, [_vp, _c.POINTER(_vp)]),
    "shmt_hashmap_capacity": (_i64, [_i64, _dbl]),
    "shmt_hashmap_table_bytes": (_i64, [_i64, _dbl, _int, _int]),
    "shmt_hashmap_create": (_int, [_c.POINTER(_vp), _vp, _vp, _i64, _int, _int, _dbl, _vp, _i64, _vp]),
    "shmt_hashmap_plan_scratch_bytes": (_i64, [_i64]),
    "shmt_hashmap_plan": (_int, [_vp, _vp, _i64, _int, _int, _dbl, _vp, _i64, _vp, _vp]),
    "shmt_hashmap_create_planned": (_int, [_c.POINTER(_vp), _vp, _vp, _vp, _i64, _int, _int, _dbl, _vp, _i64, _vp]),
    "shmt_hashmap_kind": (_int, [_vp]),
    "shmt_hashmap_used_bytes": (_i64, [_vp]),
    "shmt_hashmap_query": (_int, [_vp, _vp, _int, _i64, _vp, _vp]),
    "shmt_hashmap_key_bytes": (_int, [_vp]),
    "shmt_hashmap_val_bytes": (_int, [_vp]),
    "shmt_hashmap_size": (_i64, [_vp]),
    "shmt_hashmap_destroy": (None, [_vp]),
    "shmt_fetch": (_int, [_vp, _vp, _vp, _int, _vp, _vp, _int, _vp, _i64, _i64, _vp]),
    "shmt_fetch_counted": (_int, [_vp, _vp, _vp, _int, _vp, _vp, _int, _vp, _i64, _vp, _vp, _i64, _vp]),
    "shmt_fetch_cached_part": (_int, [_vp, _vp, _vp, _int, _vp, _vp, _int, _vp, _i64, _vp, _i64, _vp, _vp]),
    "shmt_fetch_missed_part": (_int, [_vp, _vp, _int, _vp, _vp, _i64, _vp, _i64, _int, _vp]),
    "shmt_set": (_int, [_vp, _vp, _vp, _int, _vp, _vp, _int, _vp, _i64, _i64, _vp]),
    "shmt_set_through": (_int, [_vp, _vp, _vp, _int, _vp, _vp, _int, _vp, _i64, _i64, _vp]),
    "shmt_scan_tmp_bytes": (_i64, [_i64]),
    "shmt_exclusive_scan": (_int, [_vp, _i64, _int, _vp, _i64, _vp]),
    "shmt_inclusive_scan_i32": (_int, [_vp, _i64, _vp, _i64, _vp]),
    "shmt_exclusive_scan_noalloc": (_int, [_vp, _i64, _int, _vp]),
    "shmt_scan_workspace_clear": (_int, [_vp, _i64, _vp]),
    "shmt_exclusive_scan_kept": (_int, [_vp, _i64, _int, _vp, _i64, _vp]),
    "shmt_inclusive_scan_i32_kept": (_int, [_vp, _i64, _vp, _i64, _vp]),
    "shmt_async_error": (_int, [_c.POINTER(_int)]),
    "shmt_async_error_inject": (_int, [_int]),
    "shmt_async_error_mirror": (_int, [_vp, _vp]),
    "shmt_relabel_scratch_bytes": (_i64, [_i64]),
    "shmt_relabel": (_int, [_vp, _i64, _int, _vp, _i64, _vp, _vp, _vp, _vp]),
    "shmt_relabel_wide_scratch_bytes": (_i64, [_i64]),
    "shmt_relabel_wide": (_int, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp]),
    "shmt_relabel_tuning": (_int, [_i64, _int, _int]),
    "shmt_relabel_segments": (_int, [_c.POINTER(_vp), _c.POINTER(_i64), _c.POINTER(_int), _int, _vp, _int, _int,
                                     _vp, _vp, _i64, _vp, _vp, _vp, _vp]),
    "shmt_sample_plan_bytes": (_i64, [_i64]),
    "shmt_sample_plan": (_int, [_vp, _int, _vp, _vp, _vp, _int, _i64, _i64, _int, _vp, _vp, _i64, _vp, _vp]),
    "shmt_sample_pick": (_int, [_vp, _vp, _int, _vp, _int, _i64, _i64, _int, _vp, _int, _vp, _vp,
                                _c.c_uint64, _c.c_uint32, _vp]),
    "shmt_sample": (_int, [_vp, _int, _vp, _int, _vp, _vp, _vp, _vp, _int, _i64, _i64, _int, _c.c_uint64,
                           _c.c_uint32, _vp, _vp, _vp, _i64, _vp, _vp]),
    "shmt_sample_hop": (_int, [_vp, _int, _vp, _int, _vp, _vp, _vp, _vp, _int, _i64, _i64, _int, _c.c_uint64,
                               _c.c_uint32, _vp, _vp, _vp, _i64, _int, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "shmt_sample_hop_chained": (_int, [_vp, _int, _vp, _int, _vp, _vp, _vp, _vp, _int, _i64, _vp, _i64, _int,
                                       _c.c_uint64, _vp, _c.c_uint32, _vp, _vp, _vp, _i64, _int, _vp, _vp, _i64,
                                       _vp, _vp, _vp, _vp, _vp, _vp]),
    "shmt_sample_hops_chained": (_int, [_vp, _int, _vp]),
    "shmt_busy_wait": (_int, [_vp, _int]),
    "shmt_capture_begin": (_int, [_vp]),
    "shmt_capture_end": (_int, [_vp, _c.POINTER(_vp)]),
    "shmt_graph_launch": (_int, [_vp, _vp]),
    "shmt_graph_destroy": (None, [_vp]),
    "shmt_stage_seeds": (_int, [_vp, _int, _i64, _vp, _int, _vp, _c.c_uint64, _vp, _vp]),
    "shmt_csr_rows": (_int, [_vp, _int, _i64, _i64, _vp, _int, _vp]),
    "shmt_subcsr_plan": (_int, [_vp, _int, _vp, _int, _i64, _vp, _vp, _i64, _vp, _vp]),
    "shmt_subcsr_copy": (_int, [_vp, _vp, _int, _int, _vp, _int, _i64, _vp, _i64, _vp, _vp]),
}

class HashmapLayout(_c.Structure):
    """shmt_hashmap_layout of include/shmt.h."""
    _fields_ = [("kind", _int), ("slot_bytes", _int), ("lo", _i64), ("span", _i64), ("delta", _i64),
                ("table_bytes", _i64)]


class HopJob(_c.Structure):
    """shmt_hop_job of include/shmt.h: the parameters of one shmt_sample_hop_chained call."""
    _fields_ = [("indptr", _vp), ("ptr_bytes", _int), ("indices", _vp), ("idx_bytes", _int),
                ("cache_indptr", _vp), ("cache_indices", _vp), ("map", _vp), ("seeds", _vp),
                ("seed_bytes", _int), ("max_seeds", _i64), ("seeds_len", _vp), ("k", _i64), ("replace", _int),
                ("rng_seed", _c.c_uint64), ("rng_seed_dev", _vp), ("rng_stream", _c.c_uint32),
                ("sub_indptr", _vp), ("sub_indices", _vp), ("plan", _vp), ("plan_bytes", _i64),
                ("elem_bytes", _int), ("total_out", _vp), ("scratch", _vp), ("scratch_bytes", _i64),
                ("unique_out", _vp), ("labels_out", _vp), ("nnz_out", _vp), ("count_out", _vp),
                ("count_dev_out", _vp), ("coo_dst", _vp), ("coo_bytes", _int)]


_lib = None


class ShmtError(RuntimeError):
    pass


def load():
    """Load libshmt.so (after torch, so that both share one HIP runtime)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ShmtError("libshmt.so is not built: run `python -m shmtensor_amd.build`")
    import torch  # noqa: F401  (loads the HIP runtime this library must share)
    lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.shmt_abi_version() != 2:
        raise ShmtError("libshmt.so ABI version mismatch")
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        raise ShmtError(load().shmt_last_error().decode() or "shmt error %d" % rc)


def current_stream():
    import torch
    return torch.cuda.current_stream().cuda_stream
