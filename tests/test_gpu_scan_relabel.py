"""Scan and relabel on the GPU: reference KAT (example/test_cache_sampling.py:129-140),
the CPU oracle, closed forms and the edge cases of the capacity rule."""
import numpy as np
import pytest
import torch

from conftest import load_golden

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 1023, 1024, 1025, 8192, 65536, 65537, 1_000_003, 5_000_000])
def test_thrust_scan_inclusive_int32(capi, oracle, n):
    rng = np.random.default_rng(n)
    a = rng.integers(-1000, 1000, size=n).astype(np.int32)
    t = torch.from_numpy(a.copy()).cuda()
    capi.thrust_scan(t)
    assert np.array_equal(t.cpu().numpy(), oracle.inclusive_scan_i32(a))
    assert np.array_equal(t.cpu().numpy(), np.cumsum(a, dtype=np.int32))


def test_thrust_scan_wraps_and_pinned_host(capi):
    a = torch.full((3_000_000,), 2**30, dtype=torch.int32).cuda()
    capi.thrust_scan(a)
    assert np.array_equal(a.cpu().numpy(), np.cumsum(np.full(3_000_000, 2**30, np.int32), dtype=np.int32))
    h = torch.arange(100, dtype=torch.int32).pin_memory()      # device-addressable host memory
    capi.thrust_scan(h)
    torch.cuda.synchronize()
    assert torch.equal(h, torch.cumsum(torch.arange(100), 0).int())


@pytest.mark.parametrize("bytes_", [4, 8])
@pytest.mark.parametrize("n", [1, 100, 4096, 65536, 65537, 2_000_000])
def test_exclusive_scan_c_abi(cabi, oracle, bytes_, n):
    lib = cabi.load()
    dt = np.int32 if bytes_ == 4 else np.int64
    rng = np.random.default_rng(n + bytes_)
    a = rng.integers(0, 2**30 if bytes_ == 4 else 2**61, size=n + 1).astype(dt)     # wraps
    t = torch.from_numpy(a.copy()).cuda()
    tmp_bytes = lib.shmt_scan_tmp_bytes(n + 1)
    tmp = torch.empty(max(tmp_bytes, 1), dtype=torch.uint8).cuda()
    cabi.check(lib.shmt_exclusive_scan(t.data_ptr(), n + 1, bytes_, tmp.data_ptr(), tmp_bytes, cabi.current_stream()))
    assert np.array_equal(t.cpu().numpy(), oracle.exclusive_scan(a))


@pytest.mark.parametrize("bytes_", [4, 8])
def test_single_pass_scan_tile_edges_and_unaligned_data(cabi, oracle, bytes_):
    """Inputs beyond one workgroup are scanned in one pass over 128 KiB tiles (16,384 int64 / 32,768 int32
    elements) that look back at each other: lengths on and around tile boundaries, several hundred tiles,
    and a data pointer that is not 16-byte aligned (element-wise loads instead of vector loads)."""
    lib = cabi.load()
    dt = np.int32 if bytes_ == 4 else np.int64
    tile = 131072 // bytes_
    rng = np.random.default_rng(bytes_)
    for n in (65_537, tile * 3 - 1, tile * 3, tile * 3 + 1, tile * 64, tile * 65 + 5, tile * 700 + 12345):
        for shift in (0, 1):                                        # shift 1: data starts bytes_ past a 16-byte boundary
            a = rng.integers(0, 2**29 if bytes_ == 4 else 2**60, size=n).astype(dt)      # sums wrap around
            buf = torch.zeros(n + 4, dtype=torch.int32 if bytes_ == 4 else torch.int64).cuda()
            t = buf[shift:shift + n]
            t.copy_(torch.from_numpy(a))
            tmp_bytes = lib.shmt_scan_tmp_bytes(n)
            tmp = torch.empty(tmp_bytes, dtype=torch.uint8).cuda()
            cabi.check(lib.shmt_exclusive_scan(t.data_ptr(), n, bytes_, tmp.data_ptr(), tmp_bytes,
                                               cabi.current_stream()))
            assert np.array_equal(t.cpu().numpy(), oracle.exclusive_scan(a)), (n, shift)
            assert int(buf[shift + n]) == 0 and (shift == 0 or int(buf[0]) == 0)        # nothing written outside
    small = torch.empty(8, dtype=torch.uint8).cuda()
    big = torch.zeros(100_000, dtype=torch.int64).cuda()
    assert lib.shmt_exclusive_scan(big.data_ptr(), 100_000, 8, small.data_ptr(), 8, cabi.current_stream()) == -4


def test_single_pass_scan_all_three_levels_of_published_sums(cabi):
    """A tile adds up the tiles before it in its group of 64, the groups before its group in its run of 64
    groups, and the runs before its run. 3 x 2^26 int64 (12,289 tiles, 4 runs) against torch.cumsum; then
    ones over 268,145 int32 tiles (35 GB, more than 64 runs: the runs are read in several steps), where the
    exclusive scan is the position itself modulo 2^32."""
    lib = cabi.load()
    g = torch.Generator(device="cuda").manual_seed(9)
    n = 3 * (1 << 26) + 5
    a = torch.randint(0, 2**40, (n,), device="cuda", generator=g)
    ref = torch.cumsum(a, 0) - a
    tmp_bytes = lib.shmt_scan_tmp_bytes(n)
    tmp = torch.empty(tmp_bytes, dtype=torch.uint8, device="cuda")
    cabi.check(lib.shmt_exclusive_scan(a.data_ptr(), n, 8, tmp.data_ptr(), tmp_bytes, cabi.current_stream()))
    assert torch.equal(a, ref)
    del a, ref
    n = (262_144 + 6_000) * 32_768 + 17
    ones = torch.ones(n, dtype=torch.int32, device="cuda")
    tmp_bytes = lib.shmt_scan_tmp_bytes(n)
    tmp = torch.empty(tmp_bytes, dtype=torch.uint8, device="cuda")
    cabi.check(lib.shmt_exclusive_scan(ones.data_ptr(), n, 4, tmp.data_ptr(), tmp_bytes, cabi.current_stream()))
    probe = torch.cat([torch.randint(0, n, (1_000_000,), device="cuda", generator=g),
                       torch.tensor([0, n - 1, 262_144 * 32_768 - 1, 262_144 * 32_768], device="cuda")])
    assert torch.equal(ones[probe].long() & 0xFFFFFFFF, probe & 0xFFFFFFFF)


def test_scans_on_several_streams_at_once(cabi):
    """Scans queued on four streams without waiting in between share the GPU: every tile number is taken by
    a running workgroup, so kernels that hold compute units at the same time cannot wait for each other's
    unstarted workgroups. Each result against torch.cumsum."""
    lib = cabi.load()
    g = torch.Generator(device="cuda").manual_seed(4)
    n = (1 << 24) + 3
    streams = [torch.cuda.Stream() for _ in range(4)]
    data, refs, tmps = [], [], []
    for _ in range(8):
        a = torch.randint(0, 2**40, (n,), device="cuda", generator=g)
        refs.append(torch.cumsum(a, 0) - a)
        data.append(a)
        tmps.append(torch.empty(lib.shmt_scan_tmp_bytes(n), dtype=torch.uint8, device="cuda"))
    torch.cuda.synchronize()
    for i, a in enumerate(data):
        s = streams[i % 4]
        cabi.check(lib.shmt_exclusive_scan(a.data_ptr(), n, 8, tmps[i].data_ptr(), tmps[i].numel(), s.cuda_stream))
    torch.cuda.synchronize()
    for a, ref in zip(data, refs):
        assert torch.equal(a, ref)


def test_relabel_reference_kat(capi):
    g = load_golden("relabel_kat.json")
    u, labels = capi.tensor_relabel([torch.tensor(x).cuda() for x in g["inputs"]])
    assert u.tolist() == g["unique"]
    assert [l.tolist() for l in labels] == g["labels"]
    assert isinstance(labels, list) and u.dtype == torch.int64


# 5,460 / 5,461 / 5,462: 8,191 / 8,192 / 8,194 ids in all, either side of the largest input that one
# workgroup relabels in LDS
@pytest.mark.parametrize("n", [1, 2, 7, 8, 9, 255, 256, 257, 2047, 2048, 2049, 5460, 5461, 5462, 100_000,
                               3_000_000])
@pytest.mark.parametrize("dt", [np.int32, np.int64])
def test_relabel_matches_oracle(capi, oracle, n, dt):
    rng = np.random.default_rng(n)
    hi = 2**31 if dt == np.int64 else 0
    a = (rng.integers(0, max(2, n // 3), size=n) + hi).astype(dt)
    b = rng.integers(0, max(2, n // 3), size=n // 2 + 1).astype(dt)
    u, (la, lb) = capi.tensor_relabel([torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()])
    eu, (ea, eb) = oracle.relabel([a, b])
    assert u.dtype == la.dtype == torch.from_numpy(a).dtype
    assert np.array_equal(u.cpu().numpy(), eu)
    assert np.array_equal(la.cpu().numpy(), ea) and np.array_equal(lb.cpu().numpy(), eb)


@pytest.mark.parametrize("n", [9, 300, 2049, 5461, 5462, 100_000, 1_500_000])
@pytest.mark.parametrize("odd", ["one_wide_id_at_the_end", "many_wide", "negative", "uint32_max", "mixed_widths"])
def test_relabel_id_ranges_select_the_table_format(capi, oracle, n, odd):
    """8-byte ids that all fit 32 bits go through the packed table, anything else through
    16-byte slots; dense ranges and heavy repetition stress slot take-overs. Same labels either way."""
    rng = np.random.default_rng(n)
    a = rng.integers(0, max(2, n // 4), size=n).astype(np.int64)
    a[::5] = rng.integers(0, 2**32, size=a[::5].size)                  # spread over the full 32-bit range
    b = rng.integers(0, max(2, n // 4), size=n // 2 + 1)
    b = b.astype(np.int32 if odd == "mixed_widths" else np.int64)
    if odd == "one_wide_id_at_the_end":
        b[-1] = 2**32
    elif odd == "many_wide":
        a[1::3] += 2**40
    elif odd == "negative":
        b[::7] = -b[::7] - 1
    elif odd == "uint32_max":
        a[::9] = 2**32 - 1
    u, (la, lb) = capi.tensor_relabel([torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()])
    eu, (ea, eb) = oracle.relabel([a, b])
    assert np.array_equal(u.cpu().numpy(), eu)
    assert np.array_equal(la.cpu().numpy(), ea) and np.array_equal(lb.cpu().numpy(), eb)


def test_relabel_is_shift_invariant_across_table_formats(capi):
    """relabel(x + 2^40) must give the labels of relabel(x) and the shifted unique list: the first call
    runs on 16-byte slots, the second on packed slots, over many sizes and repetition patterns."""
    g = torch.Generator(device="cuda").manual_seed(21)
    shift = 1 << 40
    for case in range(40):
        n = int(torch.randint(1, 2_000_000 if case % 4 == 0 else 60_000, (1,), generator=g, device="cuda"))
        span = [3, 50, n // 8 + 1, n, 4 * n, 2**32][case % 6]
        x = torch.randint(0, span, (n,), generator=g, device="cuda")
        if case % 5 == 0:                      # hub-like skew: a few ids take most positions
            hubs = torch.randint(0, 7, (n,), generator=g, device="cuda")
            x = torch.where(torch.rand(n, generator=g, device="cuda") < 0.7, hubs, x)
        split = int(torch.randint(0, n + 1, (1,), generator=g, device="cuda"))
        u0, (a0, b0) = capi.tensor_relabel([x[:split], x[split:]])
        u1, (a1, b1) = capi.tensor_relabel([x[:split] + shift, x[split:] + shift])
        assert torch.equal(u0 + shift, u1), case
        assert torch.equal(a0, a1) and torch.equal(b0, b1), case
        assert torch.equal(u0[torch.cat([a0, b0])], x), case


def test_relabel_mixed_dtypes_prefix_property(capi, oracle):
    # the dataloader's call: [int64 seeds, int32 sub_indices] (python/shmtensor/sampling.py:137-138)
    rng = np.random.default_rng(5)
    seeds = rng.choice(100_000, size=1024, replace=False).astype(np.int64)
    nbrs = rng.integers(0, 100_000, size=15_000).astype(np.int32)
    u, (ls, ln) = capi.tensor_relabel([torch.from_numpy(seeds).cuda(), torch.from_numpy(nbrs).cuda()])
    assert u.dtype == torch.int64 and ln.dtype == torch.int64
    assert torch.equal(u[:1024].cpu(), torch.from_numpy(seeds))
    assert torch.equal(ls.cpu(), torch.arange(1024))
    assert torch.equal(u[ln].cpu(), torch.from_numpy(nbrs).long())
    eu, (es, en) = oracle.relabel([seeds, nbrs])
    assert np.array_equal(u.cpu().numpy(), eu) and np.array_equal(ln.cpu().numpy(), en)


def test_relabel_degenerate_inputs(capi):
    u, (l,) = capi.tensor_relabel([torch.full((1000,), 7).cuda()])
    assert u.tolist() == [7] and l.tolist() == [0] * 1000
    x = torch.randperm(5000).cuda()
    u, (l,) = capi.tensor_relabel([x])
    assert torch.equal(u, x) and torch.equal(l, torch.arange(5000).cuda())
    u, (l1, l2) = capi.tensor_relabel([torch.zeros(0, dtype=torch.int64).cuda(), torch.tensor([3, 3, 1]).cuda()])
    assert u.tolist() == [3, 1] and l1.numel() == 0 and l2.tolist() == [0, 0, 1]
    u, (l,) = capi.tensor_relabel([torch.zeros(0, dtype=torch.int64).cuda()])
    assert u.numel() == 0 and l.numel() == 0


def test_relabel_full_size_properties(capi):
    """N = 16M (config 5 scale): labels invert unique, unique is duplicate free
    and ordered by first occurrence (checked through the monotone first-index property)."""
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randint(0, 4_000_000, (16_000_000,), device="cuda", generator=g)
    u, (l,) = capi.tensor_relabel([x])
    assert torch.equal(u[l], x)
    assert u.numel() == torch.unique(x).numel()
    first = torch.full((u.numel(),), x.numel(), device="cuda", dtype=torch.int64)
    first.scatter_reduce_(0, l, torch.arange(x.numel(), device="cuda"), reduce="amin")
    assert bool((first[1:] > first[:-1]).all())


@pytest.mark.parametrize("n", [1, 100, 8191, 8192, 8193, 50_000])
@pytest.mark.parametrize("bytes_", [4, 8])
def test_c_abi_relabel_of_one_array(cabi, oracle, n, bytes_):
    """shmt_relabel (one id array, no concatenation) through raw pointers, on both sides of the
    size up to which one workgroup does all passes."""
    lib = cabi.load()
    rng = np.random.default_rng(n + bytes_)
    ids = rng.integers(0, max(2, n // 2), size=n).astype(np.int32 if bytes_ == 4 else np.int64)
    if bytes_ == 8:
        ids[::3] += 2**33                                  # ids beyond 32 bits
        ids[1::11] = -ids[1::11] - 2                       # and negative ones (-1 is the reserved value)
    total = torch.from_numpy(ids).cuda()
    unique, labels = torch.empty_like(total), torch.empty_like(total)
    sbytes = lib.shmt_relabel_scratch_bytes(n)
    scratch = torch.empty(sbytes, dtype=torch.uint8).cuda()
    count = torch.full((1,), -1, dtype=torch.int64).cuda()
    cabi.check(lib.shmt_relabel(total.data_ptr(), n, bytes_, scratch.data_ptr(), sbytes, unique.data_ptr(),
                                labels.data_ptr(), count.data_ptr(), cabi.current_stream()))
    torch.cuda.synchronize()
    eu, (el,) = oracle.relabel([ids])
    assert int(count.item()) == eu.size
    assert np.array_equal(unique[:eu.size].cpu().numpy(), eu) and np.array_equal(labels.cpu().numpy(), el)


def test_relabel_ids_at_the_top_of_32_bits(capi, oracle):
    """int64 ids that all fit 32 bits take the packed table and a 32-bit staging table per workgroup; the id
    2^32 - 1 looks like an empty staging slot and must still be relabelled (it bypasses the staging)."""
    rng = np.random.default_rng(9)
    top = 2**32 - 1
    a = rng.integers(top - 50, top + 1, size=60_000).astype(np.int64)          # includes 2^32 - 1 many times
    b = rng.integers(0, 1000, size=40_000).astype(np.int64)
    u, (la, lb) = capi.tensor_relabel([torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()])
    eu, (ea, eb_) = oracle.relabel([a, b])
    assert top in eu
    assert np.array_equal(u.cpu().numpy(), eu)
    assert np.array_equal(la.cpu().numpy(), ea) and np.array_equal(lb.cpu().numpy(), eb_)


# ---- 2^31 ids and more: 64-bit positions -------------------------------------------------------------

@pytest.mark.parametrize("n", [1, 2, 511, 512, 513, 70_000, 3_000_000])
def test_relabel_wide_matches_oracle(cabi, oracle, n):
    """shmt_relabel_wide (the form shmt_relabel switches to at 2^31 ids) at sizes the oracle handles: ids
    beyond 32 bits, negative ids, heavy repetition."""
    lib = cabi.load()
    rng = np.random.default_rng(n)
    pool = np.concatenate([rng.integers(-2**40, 2**40, size=max(1, n // 3)), [2**31, 2**32 + 5, -2, 0]])
    pool = pool[pool != -1]
    a = pool[rng.integers(0, pool.size, size=n)].astype(np.int64)
    total = torch.from_numpy(a).cuda()
    unique = torch.empty(n, dtype=torch.int64, device="cuda")
    labels = torch.empty(n, dtype=torch.int64, device="cuda")
    sb = lib.shmt_relabel_wide_scratch_bytes(n)
    scratch = torch.empty(sb, dtype=torch.uint8, device="cuda")
    count = torch.zeros(1, dtype=torch.int64).pin_memory()
    cabi.check(lib.shmt_relabel_wide(total.data_ptr(), n, scratch.data_ptr(), sb, unique.data_ptr(), labels.data_ptr(),
                                     count.data_ptr(), cabi.current_stream()))
    torch.cuda.synchronize()
    eu, (el,) = oracle.relabel([a])
    assert int(count[0]) == eu.size
    assert np.array_equal(unique[: eu.size].cpu().numpy(), eu) and np.array_equal(labels.cpu().numpy(), el)


def test_relabel_beyond_2_31_ids(capi):
    """tensor_relabel of 2^31 + 12,345 ids (the reference stops at 2^31: int numel, src/tensor_relabel.cu:136).
    ids[i] = (7919 i) mod 2^22: the first 2^22 elements are all different, everything after repeats them with
    period 2^22, so unique = ids[:2^22] and labels[i] = i mod 2^22. About 160 GB of HBM; skipped if the box
    cannot provide it."""
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    n, m, chunk = (1 << 31) + 12_345, 1 << 22, 1 << 27
    try:
        total = torch.empty(n, dtype=torch.int64, device="cuda")
        for lo in range(0, n, chunk):
            hi = min(n, lo + chunk)
            total[lo:hi] = (torch.arange(lo, hi, device="cuda") * 7919) % m
        unique, (labels,) = capi.tensor_relabel([total])
    except torch.OutOfMemoryError as exc:        # not the kernels' failure: the test needs ~160 GB
        pytest.skip("not enough HBM for a 2^31-id relabel: %s" % str(exc)[:80])
    assert unique.dtype == torch.int64 and unique.numel() == m and labels.numel() == n
    assert torch.equal(unique, total[:m])
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        assert torch.equal(labels[lo:hi], torch.arange(lo, hi, device="cuda") % m), lo
    del total, unique, labels
    torch.cuda.empty_cache()


def test_kept_workspace_scans_need_no_clearing_and_stay_clean(cabi, oracle):
    """A workspace that is all zero once stays all zero from scan to scan (the last workgroup clears what the
    scan used), so shmt_*_scan_kept runs without the clearing launch: several scans of different lengths and
    widths on one workspace, each against the oracle, and the workspace read back as zeros in between."""
    lib = cabi.load()
    sizes = [3_000_017, 70_001, 1 << 24, 200_000]
    tmp_bytes = max(lib.shmt_scan_tmp_bytes(n) for n in sizes)
    tmp = torch.full((tmp_bytes,), 0x5A, dtype=torch.uint8).cuda()          # dirty on purpose ...
    cabi.check(lib.shmt_scan_workspace_clear(tmp.data_ptr(), tmp_bytes, cabi.current_stream()))   # ... cleared once
    rng = np.random.default_rng(5)
    for n in sizes:
        a64 = rng.integers(-2**40, 2**40, size=n)
        d = torch.from_numpy(a64).cuda()
        cabi.check(lib.shmt_exclusive_scan_kept(d.data_ptr(), n, 8, tmp.data_ptr(), tmp_bytes, cabi.current_stream()))
        assert np.array_equal(d.cpu().numpy(), oracle.exclusive_scan(a64))
        assert int(tmp.count_nonzero()) == 0
        a32 = rng.integers(-1000, 1000, size=n).astype(np.int32)
        d = torch.from_numpy(a32).cuda()
        cabi.check(lib.shmt_inclusive_scan_i32_kept(d.data_ptr(), n, tmp.data_ptr(), tmp_bytes, cabi.current_stream()))
        assert np.array_equal(d.cpu().numpy(), np.cumsum(a32, dtype=np.int32))
        assert int(tmp.count_nonzero()) == 0
    # too small a workspace is an argument error
    assert lib.shmt_exclusive_scan_kept(d.data_ptr(), 1 << 24, 8, tmp.data_ptr(), 64, cabi.current_stream()) != 0


def test_a_wait_that_gave_up_is_reported(capi, cabi):
    """A scan tile whose look-back gives up sets a bit in the GPU's error word instead of finishing with a wrong
    result in silence. The word is set from the host here (no kernel has to starve): shmt_async_error returns
    and clears it, the shim turns it into a RuntimeError that names the scan."""
    import ctypes
    lib = cabi.load()
    code = ctypes.c_int(-1)
    cabi.check(lib.shmt_async_error(ctypes.byref(code)))
    assert code.value == 0
    capi.raise_async_error()                                    # nothing to report
    cabi.check(lib.shmt_async_error_inject(1))
    with pytest.raises(RuntimeError, match="look-back of a device-wide scan"):
        capi.raise_async_error()
    capi.raise_async_error()                                    # reading it cleared it
    cabi.check(lib.shmt_async_error_inject(1))
    cabi.check(lib.shmt_async_error(ctypes.byref(code)))
    assert code.value == 1 and b"gave up a bounded wait" in lib.shmt_last_error()
    cabi.check(lib.shmt_async_error(ctypes.byref(code)))
    assert code.value == 0
    # the shim also watches a pinned mirror of the word: the next operator that reads a size back raises, the
    # one after it works again
    a = torch.arange(100_000, device="cuda") % 977
    capi.tensor_relabel([a])                                    # first read-back registers the mirror word
    cabi.check(lib.shmt_async_error_inject(1))
    with pytest.raises(RuntimeError, match="look-back of a device-wide scan"):
        capi.tensor_relabel([a])
    uniq, _ = capi.tensor_relabel([a])
    assert uniq.numel() == 977
    capi.raise_async_error()
