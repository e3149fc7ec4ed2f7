"""numpy front end of the CPU oracle (oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py. The product never imports this module.

Each function takes and returns numpy arrays and restates the reference
operator named in its docstring (file:line relative to the ShmTensor tree).
"""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_DIR, "liboracle.so")
_lib = None

_vp, _i64, _int = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int


def build():
    subprocess.check_call(["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-fopenmp", "-Wall",
                           os.path.join(_DIR, "oracle.c"), "-o", _LIB_PATH, "-lm"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.orc_num_threads.restype = _int
        L.orc_set_num_threads.argtypes = [_int]
        L.orc_map_capacity.restype = _i64
        L.orc_map_capacity.argtypes = [_i64, ctypes.c_double]
        L.orc_map_build.restype = _vp
        L.orc_map_build.argtypes = [_vp, _vp, _i64, _int, _int, ctypes.c_double]
        L.orc_map_query.argtypes = [_vp, _vp, _int, _i64, _vp]
        L.orc_map_reported_capacity.restype = _i64
        L.orc_map_reported_capacity.argtypes = [_vp]
        L.orc_map_free.argtypes = [_vp]
        L.orc_fetch.argtypes = [_vp, _vp, _vp, _int, _int, _vp, _vp, _int, _vp, _i64, _i64]
        L.orc_set.argtypes = [_vp, _vp, _vp, _int, _int, _vp, _vp, _int, _vp, _i64, _i64]
        L.orc_exclusive_scan.argtypes = [_vp, _i64, _int]
        L.orc_inclusive_scan_i32.argtypes = [_vp, _i64]
        L.orc_relabel.restype = _i64
        L.orc_relabel.argtypes = [_vp, _i64, _vp, _vp]
        L.orc_relabel_sweep.restype = _i64
        L.orc_relabel_sweep.argtypes = [_vp, _i64, _vp, _vp]
        L.orc_relabel_parallel.restype = _i64
        L.orc_relabel_parallel.argtypes = [_vp, _i64, _vp, _vp]
        L.orc_philox4x32_10.argtypes = [_vp, _vp, _vp]
        L.orc_sample_counts.restype = _i64
        L.orc_sample_counts.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _vp]
        L.orc_sample_fill.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _vp, _vp,
                                      ctypes.c_uint64, ctypes.c_uint32, _int]
        L.orc_subcsr_counts.restype = _i64
        L.orc_subcsr_counts.argtypes = [_vp, _vp, _i64, _vp]
        L.orc_subcsr_copy.argtypes = [_vp, _vp, _vp, _i64, _vp, _vp]
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def _ids(a):
    a = np.ascontiguousarray(a)
    assert a.dtype in (np.int32, np.int64), a.dtype
    return a


def _i64a(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def num_threads():
    return lib().orc_num_threads()


def set_num_threads(n):
    lib().orc_set_num_threads(int(n))


class Hashmap:
    """CUCOStaticHashmap: src/cuco_hashmap.cu:10-41, include/cuco_hashmap.cuh:57-87."""

    def __init__(self, keys, values, load_factor):
        keys, values = _ids(keys), _ids(values)
        assert keys.shape == values.shape
        self.key_dtype, self.value_dtype = keys.dtype, values.dtype
        self._h = lib().orc_map_build(_p(keys), _p(values), keys.size, keys.itemsize,
                                      values.itemsize, float(load_factor))

    def query(self, requests):
        req = np.ascontiguousarray(requests)
        if req.dtype not in (np.int32, np.int64):
            req = req.astype(self.key_dtype)
        out = np.empty(req.shape, dtype=self.value_dtype)
        lib().orc_map_query(self._h, _p(req), req.itemsize, req.size, _p(out))
        return out

    def capacity(self):
        return lib().orc_map_reported_capacity(self._h)

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.orc_map_free(self._h)
            self._h = None


def _rows(data):
    data = np.ascontiguousarray(data)
    row_bytes = data.itemsize * int(np.prod(data.shape[1:], dtype=np.int64))
    return data, row_bytes


def fetch(host, gpu, indices, hashmap=None, mask=None):
    """uva_fetch / cache_fetch / cache_fetch_with_mask:
    src/cache_feature_fetch.cu:47-87, :131-185, :226-272."""
    host, row_bytes = _rows(host)
    idx = _ids(indices)
    out = np.empty((idx.size,) + host.shape[1:], dtype=host.dtype)
    mode, m, mk, mkb = 0, None, None, 0
    if hashmap is not None:
        mode, m = 1, hashmap._h
    elif mask is not None:
        mk = _ids(mask)
        mode, mkb = 2, mk.itemsize
    g = None if gpu is None else np.ascontiguousarray(gpu)
    lib().orc_fetch(_p(host), _p(g), _p(idx), idx.itemsize, mode, m, _p(mk), mkb, _p(out), idx.size,
                    row_bytes)
    return out


def set_rows(host, gpu, indices, update, hashmap=None, mask=None):
    """uva_set / cache_set / cache_set_with_mask (in place on host and gpu):
    src/cache_feature_set.cu:39-75, :118-165, :209-248."""
    assert host.flags.c_contiguous and (gpu is None or gpu.flags.c_contiguous)
    _, row_bytes = _rows(host)
    idx = _ids(indices)
    upd = np.ascontiguousarray(update)
    assert upd.dtype == host.dtype and upd.nbytes == idx.size * row_bytes
    mode, m, mk, mkb = 0, None, None, 0
    if hashmap is not None:
        mode, m = 1, hashmap._h
    elif mask is not None:
        mk = _ids(mask)
        mode, mkb = 2, mk.itemsize
    lib().orc_set(_p(host), _p(gpu), _p(idx), idx.itemsize, mode, m, _p(mk), mkb, _p(upd), idx.size,
                  row_bytes)


def exclusive_scan(a):
    """cub_exclusiveSum: src/tensor_relabel.cu:11-26 (returns a scanned copy)."""
    a = _ids(a).copy()
    lib().orc_exclusive_scan(_p(a), a.size, a.itemsize)
    return a


def inclusive_scan_i32(a):
    """thrust_scan in program order: src/thrust_scan.cu:9-18."""
    a = np.ascontiguousarray(a, dtype=np.int32).copy()
    lib().orc_inclusive_scan_i32(_p(a), a.size)
    return a


def relabel(tensors, algo="passes"):
    """tensor_relabel: src/tensor_relabel.cu:125-209. Returns (unique, [labels...])
    with the dtype torch.cat would give (int64 if any input is int64). algo: "passes"
    (the reference's four parallel passes over its low-bit hash table, OpenMP) or
    "sweep" (one sequential sweep with a mixed hash: the plain CPU way, same results) or
    "parallel" (the tuned multi-core form: ids dealt to one partition per thread by their hash, every
    thread sweeping its own; tables kept between calls)."""
    tensors = [_ids(t) for t in tensors]
    dt = np.result_type(*[t.dtype for t in tensors]) if tensors else np.int64
    total = _i64a(np.concatenate(tensors)) if tensors else np.zeros(0, np.int64)
    unique = np.empty(total.size, np.int64)
    labels = np.empty(total.size, np.int64)
    fn = {"passes": lib().orc_relabel, "sweep": lib().orc_relabel_sweep, "parallel": lib().orc_relabel_parallel}[algo]
    u = fn(_p(total), total.size, _p(unique), _p(labels))
    out, off = [], 0
    for t in tensors:
        out.append(labels[off:off + t.size].astype(dt, copy=False))
        off += t.size
    return unique[:u].astype(dt, copy=False), out


def philox4x32_10(ctr, key):
    ctr = np.ascontiguousarray(ctr, dtype=np.uint32)
    key = np.ascontiguousarray(key, dtype=np.uint32)
    out = np.empty(4, np.uint32)
    lib().orc_philox4x32_10(_p(ctr), _p(key), _p(out))
    return out


def sample(indptr, indices, seeds, num_picks, replace, cache=None, seed=7777, stream=0,
           algo="reservoir"):
    """csr_sampling / csr_cache_sampling: src/cache_graph_sampling.cu:179-220, :382-426.
    cache = (gpu_indptr, gpu_indices, Hashmap) or None. Returns (sub_indptr, sub_indices)
    with the dtypes of indptr / indices. algo: "reservoir" (Algorithm R, the reference's
    selection) or "floyd" (the device kernel's selection rule)."""
    ip, ix, sd = _i64a(indptr), _i64a(indices), _i64a(seeds)
    gp = gi = m = None
    if cache is not None:
        gp, gi, m = _i64a(cache[0]), _i64a(cache[1]), cache[2]._h
    sub_indptr = np.empty(sd.size + 1, np.int64)
    nnz = lib().orc_sample_counts(_p(ip), _p(ix), _p(gp), _p(gi), m, _p(sd), sd.size, int(num_picks),
                                  int(bool(replace)), _p(sub_indptr))
    out = np.empty(nnz, np.int64)
    lib().orc_sample_fill(_p(ip), _p(ix), _p(gp), _p(gi), m, _p(sd), sd.size, int(num_picks),
                          int(bool(replace)), _p(sub_indptr), _p(out), int(seed), int(stream),
                          {"reservoir": 0, "floyd": 1}[algo])
    return sub_indptr.astype(np.asarray(indptr).dtype), out.astype(np.asarray(indices).dtype)


def create_subcsr(indptr, indices, seeds):
    """create_subcsr: src/cache_graph_sampling.cu:455-492."""
    ip, ix, sd = _i64a(indptr), _i64a(indices), _i64a(seeds)
    gp = np.empty(sd.size + 1, np.int64)
    nnz = lib().orc_subcsr_counts(_p(ip), _p(sd), sd.size, _p(gp))
    gi = np.empty(nnz, np.int64)
    lib().orc_subcsr_copy(_p(ip), _p(ix), _p(sd), sd.size, _p(gp), _p(gi))
    return gp.astype(np.asarray(indptr).dtype), gi.astype(np.asarray(indices).dtype)
