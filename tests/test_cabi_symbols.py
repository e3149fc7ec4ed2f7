"""The C-ABI library loads and exports every symbol include/shmt.h declares;
argument validation that needs no GPU returns the documented codes."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "shmt.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(shmt_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(cabi):
    lib = cabi.load()
    names = declared_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(cabi.SIGNATURES) == names      # the ctypes table covers the whole header


def test_size_queries_and_validation(cabi):
    lib = cabi.load()
    assert lib.shmt_abi_version() == 2
    assert lib.shmt_hashmap_capacity(50000, 0.8) == 62500
    assert lib.shmt_hashmap_capacity(3, 0.8) == 4
    # 8 wide slots or 16 narrow slots per 128-byte bucket
    assert lib.shmt_hashmap_table_bytes(4194304, 0.5, 8, 8) == 8388608 * 16
    assert lib.shmt_hashmap_table_bytes(1000, 0.5, 4, 4) == 2000 * 8
    assert lib.shmt_hashmap_table_bytes(8, 1.0, 8, 8) == 2 * 128      # never denser than 50 %: 16 slots
    assert lib.shmt_hashmap_table_bytes(0, 0.5, 8, 8) == 128          # an empty map keeps one empty bucket
    assert lib.shmt_hashmap_table_bytes(10, 0.5, 3, 8) == -1
    assert b"bad arguments" in lib.shmt_last_error()
    assert lib.shmt_scan_tmp_bytes(1000) == 0 and lib.shmt_scan_tmp_bytes(1 << 20) == 64 + (64 + 1 + 1) * 16
    assert lib.shmt_relabel_scratch_bytes(1000) >= 2000 * 16 + 4000
    assert lib.shmt_sample_plan_bytes(1024) >= 1024 * 16
    # relabel with 64-bit positions: 16-byte slots at load <= 0.5, 8-byte ranks; shmt_relabel uses it from 2^31 ids
    assert lib.shmt_relabel_wide_scratch_bytes(1000) >= 2000 * 16 + 1000 * 8
    big = 1 << 31
    assert lib.shmt_relabel_scratch_bytes(big) == lib.shmt_relabel_wide_scratch_bytes(big) >= big * (32 + 8)
    assert lib.shmt_relabel_scratch_bytes(big - 1) < big * 40
    assert lib.shmt_relabel(None, big, 4, None, 0, None, None, None, None) == -1
    assert b"8 bytes wide" in lib.shmt_last_error()
    # empty inputs are no-ops that need no device
    assert lib.shmt_fetch(None, None, None, 8, None, None, 0, None, 0, 512, None) == 0
    assert lib.shmt_set(None, None, None, 8, None, None, 0, None, 0, 512, None) == 0
    assert lib.shmt_exclusive_scan(None, 0, 8, None, 0, None) == 0
    assert lib.shmt_hashmap_query(None, None, 8, 0, None, None) == -1      # null map
    assert lib.shmt_fetch(None, None, None, 3, None, None, 0, None, 0, 512, None) == -1
    assert b"int32 or int64" in lib.shmt_last_error()


def test_operator_surface_matches_reference(capi):
    """Names and keyword names of src/pybind.cc:31-64 (hot-path part)."""
    expected = {
        "thrust_scan": ["tensor"],
        "pin_memory": ["data"], "unpin_memory": ["data"],
        "uva_fetch": ["data", "indices"],
        "cache_fetch": ["uva_data", "gpu_data", "indices", "hashmap"],
        "cache_fetch_with_mask": ["uva_data", "gpu_data", "indices", "mask"],
        "uva_set": ["data", "indices", "update"],
        "cache_set": ["uva_data", "gpu_data", "indices", "update", "hashmap"],
        "cache_set_with_mask": ["uva_data", "gpu_data", "indices", "update", "mask"],
        "csr_sampling": ["indptr", "indices", "seeds", "num_picks", "replace"],
        "csr_cache_sampling": ["uva_indptr", "uva_indices", "gpu_indptr", "gpu_indices", "hashmap",
                               "seeds", "num_picks", "replace"],
        "create_subcsr": ["uva_indptr", "uva_indices", "seeds"],
        "tensor_relabel": ["tensors"],
    }
    for name, args in expected.items():
        doc = getattr(capi, name).__doc__
        sig = doc.split("\n")[0]
        got = re.findall(r"(\w+): ", sig)
        assert got[: len(args)] == args, (name, sig)
    for meth in ("query", "capacity", "memory_usage"):
        assert hasattr(capi.CUCOStaticHashmap, meth)
    import sys
    assert sys.modules["ShmTensorLib"] is capi
