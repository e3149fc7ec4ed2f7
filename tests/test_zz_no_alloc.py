"""The entry point that allocates nothing: shmt_exclusive_scan_noalloc keeps its
tile counter and tile words in an array inside the library's code object. Called through the
C ABI and checked bit for bit against shmt_exclusive_scan (caller-provided
workspace) and the CPU oracle, on two calls in a row, the second on a smaller
input."""
import numpy as np
import pytest
import torch


def test_rejects_lengths_beyond_the_static_workspace(cabi):
    # argument checks come before any device call, so this needs no GPU
    lib = cabi.load()
    assert lib.shmt_exclusive_scan_noalloc(None, (1 << 28) + 1, 8, None) == -1
    assert b"exceeds the static workspace" in lib.shmt_last_error()
    assert lib.shmt_exclusive_scan_noalloc(None, -1, 8, None) == -1
    assert lib.shmt_exclusive_scan_noalloc(None, 10, 3, None) == -1
    assert lib.shmt_exclusive_scan_noalloc(None, 10, 8, None) == -1      # null data
    assert b"data is null" in lib.shmt_last_error()


def _both(cabi, a, bytes_):
    lib = cabi.load()
    n = a.size
    with_ws = torch.from_numpy(a.copy()).cuda()
    tmp_bytes = lib.shmt_scan_tmp_bytes(n)
    tmp = torch.empty(max(tmp_bytes, 1), dtype=torch.uint8, device="cuda")
    cabi.check(lib.shmt_exclusive_scan(with_ws.data_ptr(), n, bytes_, tmp.data_ptr(), tmp_bytes,
                                       cabi.current_stream()))
    no_alloc = torch.from_numpy(a.copy()).cuda()
    torch.cuda.synchronize()
    # nothing allocated: neither through torch's caching allocator nor behind its back (the driver's own
    # count of free device memory, which a hipMalloc inside the library would lower)
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info()[0]
    cabi.check(lib.shmt_exclusive_scan_noalloc(no_alloc.data_ptr(), n, bytes_, cabi.current_stream()))
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    assert torch.cuda.mem_get_info()[0] == free_before
    return with_ws.cpu().numpy(), no_alloc.cpu().numpy()


@pytest.mark.gpu
def test_no_alloc_scan_equals_workspace_scan_twice_in_a_row(cabi, oracle):
    lib = cabi.load()
    # set-up call: looks up the workspace's device address, moves nothing
    cabi.check(lib.shmt_exclusive_scan_noalloc(None, 0, 8, cabi.current_stream()))
    rng = np.random.default_rng(11)
    # first call: 5,000,001 int64 (306 tiles of 16,384 elements); second, smaller: 300,001 int32 (10 tiles of
    # 32,768), on the workspace the first call used and left clean; third: one workgroup, no workspace use
    for n, dt in ((5_000_001, np.int64), (300_001, np.int32), (4_097, np.int64)):
        hi = 2**61 if dt is np.int64 else 2**30                  # sums wrap around
        a = rng.integers(0, hi, size=n).astype(dt)
        print("no-alloc scan n=%d dtype=%s" % (n, dt.__name__), flush=True)
        ws, na = _both(cabi, a, a.itemsize)
        assert np.array_equal(na, ws)
        assert np.array_equal(na, oracle.exclusive_scan(a))
