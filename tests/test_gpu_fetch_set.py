"""Feature fetch / set through the HBM cache: the assertions of
example/test_cache_fetch.py:24-105 and example/test_cache_set.py:24-147, the CPU
oracle on the same inputs, and a routing check in which cache rows differ from
host rows so that hit/miss selection itself is observable."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _cache(capi, data, ids, lf=0.8, val_dtype=torch.int64):
    gpu_data = data[ids.cpu()].cuda()
    h = capi.CUCOStaticHashmap(ids, torch.arange(ids.numel(), device="cuda", dtype=val_dtype), lf)
    return gpu_data, h


@pytest.mark.parametrize("shape", [(100,), (100, 100, 100)])
def test_reference_unit_cases(capi, shape):
    # example/test_cache_fetch.py:24-105
    torch.manual_seed(0)
    data = (torch.arange(100).float() if len(shape) == 1 else torch.randn(shape)).pin_memory()
    indices = torch.randint(0, 100, (10,)).long().cuda()
    assert torch.equal(capi.uva_fetch(data, indices), data.cuda()[indices])
    ids = torch.randint(0, 100, (50,)).long().unique().cuda()
    gpu_data, h = _cache(capi, data, ids)
    query = torch.randint(0, 100, (20,)).long().cuda()
    expect = data[query.cpu()].cuda()
    assert torch.equal(capi.cache_fetch(data, gpu_data, query, h), expect)
    assert torch.equal(capi.cache_fetch_with_mask(data, gpu_data, query, h.query(query)), expect)


@pytest.mark.parametrize("D,dtype", [(1, torch.float32), (3, torch.float32), (7, torch.int8),
                                      (100, torch.float32), (128, torch.float32), (129, torch.float32),
                                      (128, torch.float16), (128, torch.bfloat16), (256, torch.float32),
                                      (10000, torch.float32), (33, torch.int16), (5, torch.float64)])
@pytest.mark.parametrize("idx_dtype", [torch.int32, torch.int64])
def test_fetch_matches_oracle_with_distinct_cache_rows(capi, oracle, D, dtype, idx_dtype):
    rng = np.random.default_rng(D * 7 + idx_dtype.itemsize)
    n = 3000 if D <= 256 else 300
    raw = torch.from_numpy(rng.integers(-120, 120, size=(n, D)).astype(np.int8 if dtype == torch.int8 else np.float32))
    data = raw.to(dtype).pin_memory()
    ids = torch.from_numpy(rng.choice(n, size=n // 4, replace=False)).cuda()
    gpu_data = (data[ids.cpu()].float() + 1).to(dtype).cuda()       # differs from the host rows
    h = capi.CUCOStaticHashmap(ids, torch.arange(ids.numel(), device="cuda"), 0.8)
    q = torch.from_numpy(rng.integers(0, n, size=1501)).to(idx_dtype).cuda()
    view = torch.int16 if dtype in (torch.float16, torch.bfloat16) else dtype    # compare raw bit patterns
    ref_h = oracle.Hashmap(ids.cpu().numpy(), np.arange(ids.numel()), 0.8)
    expect = oracle.fetch(data.view(view).numpy(), gpu_data.cpu().view(view).numpy(), q.cpu().numpy(), hashmap=ref_h)
    got = capi.cache_fetch(data, gpu_data, q, h)
    assert got.dtype == dtype and got.shape == (q.numel(), D)
    assert np.array_equal(got.cpu().view(view).numpy(), expect)
    for mask_dtype in (torch.int32, torch.int64):
        got_m = capi.cache_fetch_with_mask(data, gpu_data, q, h.query(q).to(mask_dtype))
        assert np.array_equal(got_m.cpu().view(view).numpy(), expect)
    assert torch.equal(capi.uva_fetch(data, q).cpu().view(view), data.view(view)[q.cpu().long()])


@pytest.mark.parametrize("hit", [0.0, 1.0])
def test_all_miss_and_all_hit(capi, hit):
    torch.manual_seed(3)
    data = torch.randn(5000, 128).pin_memory()
    ids = torch.randperm(5000)[:2000].cuda()
    gpu_data, h = _cache(capi, data, ids)
    cached = torch.zeros(5000, dtype=torch.bool)
    cached[ids.cpu()] = True
    pool = torch.nonzero(cached if hit else ~cached).flatten()
    q = pool[torch.randint(0, pool.numel(), (4096,))].cuda()
    assert ((h.query(q) >= 0).float().mean().item()) == hit
    assert torch.equal(capi.cache_fetch(data, gpu_data, q, h), data[q.cpu()].cuda())


def test_device_resident_table_and_empty_query(capi):
    data = torch.randn(1000, 16).cuda()      # the "uva" table may live on the device too
    q = torch.randint(0, 1000, (100,)).cuda()
    assert torch.equal(capi.uva_fetch(data, q), data[q])
    out = capi.uva_fetch(data, torch.zeros(0, dtype=torch.int64).cuda())
    assert out.shape == (0, 16)


def test_unpinned_host_tensor_is_an_error(capi):
    data = torch.randn(100, 8)
    with pytest.raises(RuntimeError, match="pin_memory"):
        capi.uva_fetch(data, torch.tensor([1]).cuda())


@pytest.mark.parametrize("shape", [(100_000,), (100_000, 128)])
def test_set_then_fetch_reference_case(capi, shape):
    # example/test_cache_set.py:24-147, sizes scaled down 10x
    torch.manual_seed(1)
    n = shape[0]
    data = torch.randn(shape).pin_memory()
    for size in [10, 1000, 100_000]:
        idx = torch.randint(0, n, (size,)).long().cuda().unique()
        upd = torch.randn((idx.numel(),) + shape[1:]).cuda()
        capi.uva_set(data, idx, upd)
        assert torch.equal(capi.uva_fetch(data, idx), upd)
    ids = torch.randperm(n).long().cuda()[: int(n * 0.7)]
    gpu_data, h = _cache(capi, data, ids)
    for size in [10, 1000, 100_000]:
        idx = torch.randint(0, n, (size,)).long().cuda().unique()
        upd = torch.randn((idx.numel(),) + shape[1:]).cuda()
        capi.cache_set(data, gpu_data, idx, upd, h)
        assert torch.equal(capi.cache_fetch(data, gpu_data, idx, h), upd)
        upd2 = torch.randn_like(upd)
        capi.cache_set_with_mask(data, gpu_data, idx, upd2, h.query(idx))
        assert torch.equal(capi.cache_fetch_with_mask(data, gpu_data, idx, h.query(idx)), upd2)


def test_set_final_state_matches_oracle(capi, oracle):
    rng = np.random.default_rng(11)
    host = rng.standard_normal((4000, 24)).astype(np.float32)
    ids = rng.choice(4000, size=1500, replace=False)
    gpu = host[ids] + 1
    q = np.unique(rng.integers(0, 4000, size=3000))
    upd = rng.standard_normal((q.size, 24)).astype(np.float32)
    data_t = torch.from_numpy(host.copy()).pin_memory()
    gpu_t = torch.from_numpy(gpu.copy()).cuda()
    h = capi.CUCOStaticHashmap(torch.from_numpy(ids).cuda(), torch.arange(ids.size).cuda(), 0.8)
    capi.cache_set(data_t, gpu_t, torch.from_numpy(q).cuda(), torch.from_numpy(upd).cuda(), h)
    torch.cuda.synchronize()
    ref_h = oracle.Hashmap(ids, np.arange(ids.size), 0.8)
    oracle.set_rows(host, gpu, q, upd, hashmap=ref_h)
    assert np.array_equal(data_t.numpy(), host)        # hits leave the host row stale, misses write it
    assert np.array_equal(gpu_t.cpu().numpy(), gpu)


@pytest.mark.parametrize("D,dtype", [(24, np.float32), (64, np.float16), (5, np.int8), (300, np.float32), (3, np.int16)])
@pytest.mark.parametrize("route", ["map64", "map32", "mask"])
def test_write_through_set_keeps_the_host_table_current(capi, D, dtype, route):
    """write_through=True (no counterpart in the reference): hits update the cache row and
    the host row, misses the host row; closed form on both tables."""
    rng = np.random.default_rng(D)
    n, c = 5000, 1800
    host = (rng.standard_normal((n, D)) * 50).astype(dtype)
    ids = rng.choice(n, size=c, replace=False)
    gpu = (host[ids] + 1).astype(dtype)                      # stale-looking cache rows: routing is observable
    q = np.unique(rng.integers(0, n, size=3000))
    upd = (rng.standard_normal((q.size, D)) * 50).astype(dtype)
    data_t = torch.from_numpy(host.copy()).pin_memory()
    gpu_t = torch.from_numpy(gpu.copy()).cuda()
    it = torch.int32 if route == "map32" else torch.int64
    h = capi.CUCOStaticHashmap(torch.from_numpy(ids).to(it).cuda(), torch.arange(c, dtype=it).cuda(), 0.8)
    q_t, upd_t = torch.from_numpy(q).cuda(), torch.from_numpy(upd).cuda()
    if route == "mask":
        capi.cache_set_with_mask(data_t, gpu_t, q_t, upd_t, h.query(q_t), write_through=True)
    else:
        capi.cache_set(data_t, gpu_t, q_t, upd_t, h, write_through=True)
    torch.cuda.synchronize()
    exp_host, exp_gpu = host.copy(), gpu.copy()
    exp_host[q] = upd                                        # every updated id, hit or miss
    slot_of = {int(k): s for s, k in enumerate(ids)}
    for j, k in enumerate(q):
        if int(k) in slot_of:
            exp_gpu[slot_of[int(k)]] = upd[j]
    assert np.array_equal(data_t.numpy().view(np.uint8), exp_host.view(np.uint8))
    assert np.array_equal(gpu_t.cpu().numpy().view(np.uint8), exp_gpu.view(np.uint8))
    # and the reference's own post-condition: a following fetch returns the update
    assert torch.equal(capi.cache_fetch(data_t, gpu_t, q_t, h), upd_t)
    assert torch.equal(capi.uva_fetch(data_t, q_t), upd_t)   # also straight from the host table


def test_config1_small_fetch(capi, oracle):
    """Small fetch configuration: 200,000 x 128 f32 table, 50,000 cached ids, 65,536 uniform queries."""
    torch.manual_seed(0)
    table = torch.randn(200_000, 128).pin_memory()
    ids = torch.randperm(200_000)[:50_000]
    gpu_data = table[ids].cuda()
    h = capi.CUCOStaticHashmap(ids.cuda(), torch.arange(50_000).cuda(), 0.8)
    q = torch.randint(0, 200_000, (65_536,))
    out = capi.cache_fetch(table, gpu_data, q.cuda(), h)
    hit = (h.query(q.cuda()) >= 0).float().mean().item()
    assert 0.23 < hit < 0.27
    ref_h = oracle.Hashmap(ids.numpy(), np.arange(50_000), 0.8)
    expect = oracle.fetch(table.numpy(), gpu_data.cpu().numpy(), q.numpy(), hashmap=ref_h)
    assert np.array_equal(out.cpu().numpy(), expect)
    assert torch.equal(out.cpu(), torch.index_select(table, 0, q))


def test_direct_c_abi_fetch(cabi):
    """Same operator called straight through the C ABI (raw pointers, sizes, stream)."""
    import ctypes
    lib = cabi.load()
    data = torch.randn(1000, 64).cuda()
    idx = torch.randint(0, 1000, (333,), dtype=torch.int32).cuda()
    out = torch.empty(333, 64).cuda()
    cabi.check(lib.shmt_fetch(data.data_ptr(), None, idx.data_ptr(), 4, None, None, 0, out.data_ptr(),
                              333, 256, cabi.current_stream()))
    assert torch.equal(out, data[idx.long()])
    keys = torch.arange(0, 2000, 2).cuda()
    vals = torch.arange(1000).cuda()
    nbytes = lib.shmt_hashmap_table_bytes(1000, 0.8, 8, 8)
    table = torch.empty(nbytes, dtype=torch.uint8).cuda()
    hnd = ctypes.c_void_p()
    cabi.check(lib.shmt_hashmap_create(ctypes.byref(hnd), keys.data_ptr(), vals.data_ptr(), 1000, 8, 8, 0.8,
                                       table.data_ptr(), nbytes, cabi.current_stream()))
    req = torch.arange(2000).cuda()
    res = torch.empty(2000, dtype=torch.int64).cuda()
    cabi.check(lib.shmt_hashmap_query(hnd, req.data_ptr(), 8, 2000, res.data_ptr(), cabi.current_stream()))
    expect = torch.where(req % 2 == 0, req // 2, torch.full_like(req, -1))
    assert torch.equal(res, expect)
    assert lib.shmt_hashmap_create(ctypes.byref(ctypes.c_void_p()), keys.data_ptr(), vals.data_ptr(), 1000, 8, 8,
                                   0.8, table.data_ptr(), 128, None) == -4          # table too small
    lib.shmt_hashmap_destroy(hnd)


def test_sliced_tables_and_grid_stride(capi):
    """Tables whose base pointers are only element-aligned (views into larger
    tensors) and a query count large enough that every wave loops over tiles."""
    torch.manual_seed(5)
    big = torch.randn(4001, 3).pin_memory()
    data = big[1:]                                  # 12-byte rows starting 12 bytes into the allocation
    gpu_big = torch.randn(1001, 3).cuda()
    ids = torch.randperm(4000)[:1000].cuda()
    gpu_data = gpu_big[1:]
    gpu_data.copy_(data[ids.cpu()])
    h = capi.CUCOStaticHashmap(ids, torch.arange(1000).cuda(), 0.5)
    q = torch.randint(0, 4000, (3_000_001,)).cuda()
    out = capi.cache_fetch(data, gpu_data, q, h)
    assert torch.equal(out.cpu(), data[q.cpu()])
    upd = torch.randn(1000, 3).cuda()
    capi.cache_set(data, gpu_data, ids, upd, h)     # all hits: only the cache changes
    assert torch.equal(gpu_big[1:], upd) and torch.equal(capi.uva_fetch(data, ids).cpu(), data[ids.cpu()])


def test_large_skewed_fetch_full_size(capi):
    """The large fetch configuration at its full size: 100,000,000 x 128 fp16 rows (25.6 GB) pinned, the
    40,000,000 lowest ids cached in HBM, 1,048,576 Zipf(1.1) queries. Cached rows are made to differ from
    their host copies (sign bit flipped), so the result shows which table every row came from; then the set
    pass over 262,144 cached rows. Skipped when the machine cannot pin the table."""
    from shmtensor_amd.synthetic import zipf_ranks
    n, c, d = 100_000_000, 40_000_000, 128
    try:
        table = torch.empty((n, d), dtype=torch.float16, pin_memory=True)
    except RuntimeError as exc:
        pytest.skip("cannot pin 25.6 GB here: %s" % str(exc)[:80])
    g = torch.Generator(device="cuda").manual_seed(2)
    cache = torch.empty((c, d), dtype=torch.float16, device="cuda")
    chunk = 4_000_000
    for lo in range(0, n, chunk):
        part = torch.randn((chunk, d), device="cuda", generator=g).to(torch.float16)
        table[lo:lo + chunk].copy_(part)
        if lo < c:
            cache[lo:lo + chunk] = -part                  # distinguishable from the host copy, bit-exactly invertible
    torch.cuda.synchronize()
    del part
    keys = torch.arange(c, device="cuda")
    h = capi.CUCOStaticHashmap(keys, keys, 0.8)
    assert h.capacity() == 50_000_000
    q = zipf_ranks(1 << 20, n, 1.1, seed=100)
    hit = q < c
    assert 0.97 < float(hit.float().mean()) < 0.99 and int((~hit).sum()) > 10_000
    out = capi.cache_fetch(table, cache, q, h)
    expect = torch.index_select(table, 0, q.cpu()).cuda()
    expect = torch.where(hit[:, None], -expect, expect)
    assert torch.equal(out.view(torch.int16), expect.view(torch.int16))
    assert torch.equal(capi.cache_fetch_with_mask(table, cache, q, h.query(q)).view(torch.int16), expect.view(torch.int16))
    del out, expect
    rows = torch.randperm(c, device="cuda", generator=g)[:262_144].contiguous()
    upd = torch.randn((262_144, d), device="cuda", generator=g).to(torch.float16)
    host_before = torch.index_select(table, 0, rows.cpu())
    capi.cache_set(table, cache, rows, upd, h)
    assert torch.equal(capi.cache_fetch(table, cache, rows, h).view(torch.int16), upd.view(torch.int16))
    assert torch.equal(torch.index_select(table, 0, rows.cpu()).view(torch.int16), host_before.view(torch.int16))
    capi.cache_set(table, cache, rows, upd, h, write_through=True)
    torch.cuda.synchronize()
    assert torch.equal(torch.index_select(table, 0, rows.cpu()).view(torch.int16), upd.cpu().view(torch.int16))


def test_large_skewed_fetch_scaled(capi):
    """The large fetch configuration at 1/25 scale: 4,000,000 x 128 fp16 rows pinned, the
    1,600,000 lowest ids cached, 1,048,576 Zipf(1.1) queries; then a set pass over 262,144
    cached rows. fp16 compared as raw 16-bit patterns."""
    from shmtensor_amd.synthetic import zipf_ranks
    n, c = 4_000_000, 1_600_000
    g = torch.Generator(device="cuda").manual_seed(2)
    table_d = torch.randn((n, 128), device="cuda", generator=g).to(torch.float16)
    table = torch.empty((n, 128), dtype=torch.float16).pin_memory()
    table.copy_(table_d)
    cache = table_d[:c].clone()
    del table_d
    keys = torch.arange(c, device="cuda")
    h = capi.CUCOStaticHashmap(keys, keys, 0.8)
    q = zipf_ranks(1 << 20, n, 1.1, seed=100)
    hits = float((q < c).float().mean())
    assert 0.9 < hits < 1.0 and int(q.max()) >= c          # a high hit rate with a miss tail
    out = capi.cache_fetch(table, cache, q, h)
    assert torch.equal(out.cpu().view(torch.int16), torch.index_select(table.view(torch.int16), 0, q.cpu()))
    rows = torch.randperm(c, device="cuda", generator=g)[:262_144].contiguous()
    upd = torch.randn((262_144, 128), device="cuda", generator=g).to(torch.float16)
    before = table.clone()
    capi.cache_set(table, cache, rows, upd, h)
    assert torch.equal(capi.cache_fetch(table, cache, rows, h).view(torch.int16), upd.view(torch.int16))
    torch.cuda.synchronize()
    assert torch.equal(table.view(torch.int16), before.view(torch.int16))      # hits never touch the host copy


@pytest.mark.parametrize("route", ["direct", "map", "mask"])
@pytest.mark.parametrize("count", [0, 1, 63, 64, 700, 5000, 9000])
def test_c_abi_fetch_with_the_row_count_in_device_memory(cabi, route, count):
    """shmt_fetch_counted moves min(max_rows, *count) rows, leaves the rest of
    the output alone and forwards the count to the host."""
    import ctypes
    lib = cabi.load()
    g = torch.Generator().manual_seed(count)
    table = torch.randn(4000, 48, generator=g)
    table_dev = table.cuda()
    ids = torch.randperm(4000, generator=g)[:1500]
    cache = (table[ids] + 1.0).cuda()                  # a hit is told from a miss by its content
    max_rows = 5000
    idx = torch.randint(0, 4000, (max(count, max_rows),), generator=g)
    slot_of = torch.full((4000,), -1, dtype=torch.int64)
    slot_of[ids] = torch.arange(1500)
    expect = torch.where((slot_of[idx] >= 0)[:, None], table[idx] + 1.0, table[idx]) if route != "direct" \
        else table[idx]
    idx_dev = idx.cuda()
    hnd, mask, keep = None, None, []
    if route == "map":
        keys, vals = ids.cuda(), torch.arange(1500).cuda()
        nbytes = lib.shmt_hashmap_table_bytes(1500, 0.8, 8, 8)
        keep.append(torch.empty(nbytes, dtype=torch.uint8).cuda())
        hnd = ctypes.c_void_p()
        cabi.check(lib.shmt_hashmap_create(ctypes.byref(hnd), keys.data_ptr(), vals.data_ptr(), 1500, 8, 8, 0.8,
                                           keep[0].data_ptr(), nbytes, cabi.current_stream()))
    elif route == "mask":
        mask = slot_of[idx].cuda()
    out = torch.full((max_rows, 48), -7.0).cuda()
    count_dev = torch.tensor([count]).cuda()
    seen = torch.full((1,), -1, dtype=torch.int64).pin_memory()
    seen_dev = ctypes.c_void_p()
    cabi.check(lib.shmt_host_devptr(seen.data_ptr(), ctypes.byref(seen_dev)))
    cabi.check(lib.shmt_fetch_counted(table_dev.data_ptr(), cache.data_ptr() if route != "direct" else None,
                                      idx_dev.data_ptr(), 8, hnd, mask.data_ptr() if mask is not None else None,
                                      8 if mask is not None else 0, out.data_ptr(), max_rows,
                                      count_dev.data_ptr(), seen_dev, 48 * 4,
                                      cabi.current_stream()))
    torch.cuda.synchronize()
    moved = min(count, max_rows)
    assert torch.equal(out[:moved].cpu(), expect[:moved])
    assert bool((out[moved:] == -7.0).all())
    assert seen.item() == count
    # without a host slot; and a null count is an argument error, not a launch
    out2 = torch.full((max_rows, 48), -7.0).cuda()
    cabi.check(lib.shmt_fetch_counted(table_dev.data_ptr(), cache.data_ptr() if route != "direct" else None,
                                      idx_dev.data_ptr(), 8, hnd, mask.data_ptr() if mask is not None else None,
                                      8 if mask is not None else 0, out2.data_ptr(), max_rows,
                                      count_dev.data_ptr(), None, 48 * 4, cabi.current_stream()))
    assert torch.equal(out2, out)
    assert lib.shmt_fetch_counted(table_dev.data_ptr(), None, idx_dev.data_ptr(), 8, None, None, 0,
                                  out2.data_ptr(), max_rows, None, None, 48 * 4, None) != 0
    if hnd is not None:
        torch.cuda.synchronize()
        lib.shmt_hashmap_destroy(hnd)


@pytest.mark.parametrize("route", ["map", "mask"])
@pytest.mark.parametrize("D", [4, 48, 256, 1000])
@pytest.mark.parametrize("count", [None, 0, 1, 700, 9000])
def test_c_abi_fetch_in_two_launches_equals_fetch(cabi, route, D, count):
    """shmt_fetch_cached_part (hits now, the misses marked in a bitmap) followed by shmt_fetch_missed_part on
    another stream gives what shmt_fetch / shmt_fetch_counted gives: every row once, hits from the cache
    (told apart by content), misses from the pinned host table, rows past the count untouched."""
    import ctypes
    lib = cabi.load()
    g = torch.Generator().manual_seed(D + (count or 3))
    n, c, max_rows = 6000, 2500, 5000
    table = torch.randn(n, D, generator=g).pin_memory()
    table_dev = ctypes.c_void_p()
    cabi.check(lib.shmt_host_devptr(table.data_ptr(), ctypes.byref(table_dev)))
    ids = torch.randperm(n, generator=g)[:c]
    cache = (table[ids] + 1.0).cuda()
    idx = torch.randint(0, n, (max_rows,), generator=g)
    slot_of = torch.full((n,), -1, dtype=torch.int64)
    slot_of[ids] = torch.arange(c)
    expect = torch.where((slot_of[idx] >= 0)[:, None], table[idx] + 1.0, table[idx])
    idx_dev = idx.cuda()
    hnd, mask, keep = None, None, []
    if route == "map":
        keys, vals = ids.cuda(), torch.arange(c).cuda()
        nbytes = lib.shmt_hashmap_table_bytes(c, 0.8, 8, 8)
        keep.append(torch.empty(nbytes, dtype=torch.uint8).cuda())
        hnd = ctypes.c_void_p()
        cabi.check(lib.shmt_hashmap_create(ctypes.byref(hnd), keys.data_ptr(), vals.data_ptr(), c, 8, 8, 0.8,
                                           keep[0].data_ptr(), nbytes, cabi.current_stream()))
    else:
        mask = slot_of[idx].cuda()
    out = torch.full((max_rows, D), -7.0).cuda()
    count_dev = torch.tensor([count if count is not None else 0]).cuda()
    words = (max_rows + 31) // 32
    marks = torch.full((words,), 0x5A5A5A5A, dtype=torch.int32).cuda()      # needs no clearing
    side = torch.cuda.Stream()
    cabi.check(lib.shmt_fetch_cached_part(table_dev, cache.data_ptr(), idx_dev.data_ptr(), 8, hnd,
                                          mask.data_ptr() if mask is not None else None,
                                          8 if mask is not None else 0, out.data_ptr(), max_rows,
                                          count_dev.data_ptr() if count is not None else None, D * 4,
                                          marks.data_ptr(), cabi.current_stream()))
    side.wait_stream(torch.cuda.current_stream())
    cabi.check(lib.shmt_fetch_missed_part(table_dev, idx_dev.data_ptr(), 8, marks.data_ptr(), out.data_ptr(),
                                          max_rows, count_dev.data_ptr() if count is not None else None, D * 4, 3,
                                          side.cuda_stream))
    side.synchronize()
    torch.cuda.synchronize()
    moved = max_rows if count is None else min(count, max_rows)
    miss_np = (slot_of[idx[:moved]] < 0).numpy()
    got = np.unpackbits(marks.cpu().numpy().view(np.uint8), bitorder="little")[:moved].astype(bool)
    assert np.array_equal(got, miss_np)                       # every existing row is marked or cleared
    assert torch.equal(out[:moved].cpu(), expect[:moved])
    assert bool((out[moved:] == -7.0).all())
    # the one-launch form on the same input
    whole = torch.full((max_rows, D), -7.0).cuda()
    if count is None:
        cabi.check(lib.shmt_fetch(table_dev, cache.data_ptr(), idx_dev.data_ptr(), 8, hnd,
                                  mask.data_ptr() if mask is not None else None, 8 if mask is not None else 0,
                                  whole.data_ptr(), max_rows, D * 4, cabi.current_stream()))
    else:
        cabi.check(lib.shmt_fetch_counted(table_dev, cache.data_ptr(), idx_dev.data_ptr(), 8, hnd,
                                          mask.data_ptr() if mask is not None else None,
                                          8 if mask is not None else 0, whole.data_ptr(), max_rows,
                                          count_dev.data_ptr(), None, D * 4, cabi.current_stream()))
    assert torch.equal(whole, out)
    # rows that do not allow 16-byte accesses are refused, not mis-read
    assert lib.shmt_fetch_cached_part(table_dev, cache.data_ptr(), idx_dev.data_ptr(), 8, hnd,
                                      mask.data_ptr() if mask is not None else None, 8 if mask is not None else 0,
                                      out.data_ptr(), max_rows, None, D * 4 - 4, marks.data_ptr(),
                                      cabi.current_stream()) != 0
    assert b"16-byte" in lib.shmt_last_error()
    if hnd is not None:
        torch.cuda.synchronize()
        lib.shmt_hashmap_destroy(hnd)


@pytest.mark.parametrize("D,dtype", [(32, torch.float32), (64, torch.float16), (7, torch.int8), (300, torch.float32)])
@pytest.mark.parametrize("slots", ["8-byte", "16-byte"])
def test_fetch_and_set_through_bucket_tables(capi, oracle, D, dtype, slots):
    """Key sets that are too sparse for a flat map keep the bucket table: with ids that fit 32 bits its
    8-byte slots (a small share of a large id universe is cached), with ids beyond 32 bits its 16-byte slots
    (there the queries are all hits: no host table has 2^33 rows). Routing stays observable because cache
    rows differ from host rows."""
    rng = np.random.default_rng(D + len(slots))
    n = 40_000
    raw = torch.from_numpy(rng.integers(-120, 120, size=(n, D)).astype(np.int8 if dtype == torch.int8 else np.float32))
    data = raw.to(dtype).pin_memory()
    view = torch.int16 if dtype == torch.float16 else dtype
    ids_np = rng.choice(n, size=n // 50, replace=False)                      # 1 id in 50 cached
    gpu_data = (data[torch.from_numpy(ids_np)].float() + 1).to(dtype).cuda()
    shift = 0 if slots == "8-byte" else 1 << 33
    h = capi.CUCOStaticHashmap(torch.from_numpy(ids_np + shift).cuda(), torch.arange(ids_np.size).cuda(), 0.8)
    assert h.layout() == "buckets" and h.memory_usage() == ids_np.size * 2 * (8 if shift == 0 else 16)
    if shift == 0:
        q_np = np.concatenate([rng.integers(0, n, size=3000), ids_np[rng.integers(0, ids_np.size, size=2001)]])
    else:
        q_np = ids_np[rng.integers(0, ids_np.size, size=5001)]
    ref_h = oracle.Hashmap(ids_np, np.arange(ids_np.size), 0.8)
    expect = oracle.fetch(data.view(view).numpy(), gpu_data.cpu().view(view).numpy(), q_np, hashmap=ref_h)
    got = capi.cache_fetch(data, gpu_data, torch.from_numpy(q_np + shift).cuda(), h)
    assert np.array_equal(got.cpu().view(view).numpy(), expect)
    # set through the same map: final state of both tables
    w_np = np.unique(q_np)
    upd = torch.from_numpy(rng.integers(-100, 100, size=(w_np.size, D)).astype(np.float32)).to(dtype)
    host_ref, gpu_ref = data.view(view).numpy().copy(), gpu_data.cpu().view(view).numpy().copy()
    oracle.set_rows(host_ref, gpu_ref, w_np, upd.view(view).numpy(), hashmap=ref_h)
    capi.cache_set(data, gpu_data, torch.from_numpy(w_np + shift).cuda(), upd.cuda(), h)
    torch.cuda.synchronize()
    assert np.array_equal(data.view(view).numpy(), host_ref) and np.array_equal(gpu_data.cpu().view(view).numpy(), gpu_ref)


@pytest.mark.parametrize("layout", ["buckets16", "buckets8", "direct"])
def test_fetch_and_set_through_tables_larger_than_the_caches(capi, layout):
    """Map tables beyond 64 MiB are read with the streaming cache policy (buffer loads) as long as a wave sees
    no repeated id, with plain loads afterwards: uniform queries (no repeats), skewed ones (repeats in nearly
    every tile) and a batch that is half and half must all give what indexing gives, for 16-byte and 8-byte
    bucket slots and for the direct table."""
    g = torch.Generator(device="cuda").manual_seed(41)
    n, D, c = 17_000_000, 8, 4_500_000
    table_d = torch.arange(n * D, dtype=torch.int32, device="cuda").view(n, D)
    table = table_d.cpu().pin_memory()
    ids = torch.randperm(n, device="cuda", generator=g)[:c].contiguous()
    cache = (table_d[ids] + 1).contiguous()                       # a hit is told from a miss by its content
    slots = torch.arange(c, device="cuda")
    if layout == "buckets16":
        h = capi.CUCOStaticHashmap(ids, slots, 0.5, layout="buckets")
        assert h.layout() == "buckets" and h.memory_usage() >= 64 << 20
    elif layout == "buckets8":
        h = capi.CUCOStaticHashmap(ids.int(), slots.int(), 0.5, layout="buckets")
        assert h.layout() == "buckets" and 64 << 20 <= h.memory_usage() < 100 << 20
    else:
        h = capi.CUCOStaticHashmap(ids, slots, 0.8)
        assert h.layout() == "direct" and h.memory_usage() >= 64 << 20
    slot_of = torch.full((n,), -1, dtype=torch.int64, device="cuda")
    slot_of[ids] = slots
    q_uniform = torch.randint(0, n, (150_000,), device="cuda", generator=g)
    hot = ids[:50]                                                  # fifty ids take nearly all requests
    q_skewed = torch.where(torch.rand(150_000, device="cuda", generator=g) < 0.9,
                           hot[torch.randint(0, 50, (150_000,), device="cuda", generator=g)], q_uniform)
    for q in (q_uniform, q_skewed, torch.cat([q_uniform[:70_001], q_skewed[:70_001]])):
        s = slot_of[q]
        expect = torch.where((s >= 0)[:, None], cache[s.clamp(min=0)], table_d[q])
        assert torch.equal(capi.cache_fetch(table, cache, q, h), expect)
        assert torch.equal(h.query(q).long(), s)
    # set through the same table: hits land in the cache, misses in the host table
    uq = torch.unique(q_uniform)[:50_000].contiguous()
    upd = torch.randint(-1000, 0, (uq.numel(), D), dtype=torch.int32, device="cuda", generator=g)
    capi.cache_set(table, cache, uq, upd, h)
    assert torch.equal(capi.cache_fetch(table, cache, uq, h), upd)
    torch.cuda.synchronize()
    s = slot_of[uq]
    assert torch.equal(cache[s[s >= 0]], upd[s >= 0])
    assert torch.equal(table[uq[s < 0].cpu()], upd[s < 0].cpu())
