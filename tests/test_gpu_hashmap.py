"""Static hashmap on the GPU against the CPU oracle and against closed forms.
Mirrors example/test_statichashmap.py (which only prints) with assertions."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TD = {np.int32: torch.int32, np.int64: torch.int64}


def _cuda(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("kd", [np.int32, np.int64])
@pytest.mark.parametrize("vd", [np.int32, np.int64])
@pytest.mark.parametrize("lf", [0.1, 0.5, 0.8, 0.99, 1.0])
def test_query_matches_oracle(capi, oracle, kd, vd, lf):
    rng = np.random.default_rng(hash((kd.__name__, vd.__name__, lf)) & 0xFFFF)
    keys = rng.choice(2_000_000, size=60_000, replace=False).astype(kd)
    vals = rng.integers(0, 2**31 - 1, size=keys.size).astype(vd)
    h = capi.CUCOStaticHashmap(_cuda(keys), _cuda(vals), lf)
    ref = oracle.Hashmap(keys, vals, lf)
    req = np.concatenate([keys[:20_000], rng.integers(0, 2_000_000, size=80_001), [-1]])
    for rd in (np.int32, np.int64):          # requests of either width are cast to the key width
        r = req.astype(rd)
        out = h.query(_cuda(r))
        assert out.dtype == TD[vd] and out.shape == (r.size,)
        assert np.array_equal(out.cpu().numpy(), ref.query(r))
    assert h.capacity() == ref.capacity() == int(np.ceil(keys.size / lf))
    assert h.memory_usage() >= keys.size * (8 if (kd, vd) == (np.int32, np.int32) else 16)


def test_reference_smoke_script_cases(capi):
    # example/test_statichashmap.py:6-41: values = keys + 1, query keys + 1
    torch.manual_seed(32)
    keys = torch.randint(0, 10000, (100,)).int().cuda().unique()
    values = keys + 1
    table = dict(zip(keys.tolist(), values.tolist()))
    expect = [table.get(k + 1, -1) for k in keys.tolist()]
    for kt in (torch.int32, torch.int64):
        for vt in (torch.int32, torch.int64):
            h = capi.CUCOStaticHashmap(keys.to(kt), values.to(vt), 0.5)
            out = h.query(keys.long() + 1)
            assert out.dtype == vt and out.tolist() == expect
            assert h.capacity() == int(np.ceil(keys.numel() / 0.5))


def test_narrowing_and_shapes(capi):
    keys = torch.tensor([7, 123456], dtype=torch.int32).cuda()
    h = capi.CUCOStaticHashmap(keys, torch.tensor([10, 20]).cuda(), 0.5)
    req = torch.tensor([[7, 7 + (1 << 32)], [123456 - (1 << 32), 8]]).cuda()
    out = h.query(req)
    assert out.shape == (2, 2) and out.tolist() == [[10, 10], [20, -1]]
    assert h.query(torch.tensor([-1, 7]).cuda()).tolist() == [-1, 10]
    assert h.query(torch.zeros(0, dtype=torch.int64).cuda()).numel() == 0


def test_single_key_full_table_and_empty_map(capi):
    h = capi.CUCOStaticHashmap(torch.tensor([42]).cuda(), torch.tensor([0]).cuda(), 1.0)
    assert h.query(torch.tensor([42, 41, 43]).cuda()).tolist() == [0, -1, -1]
    assert h.capacity() == 1
    h0 = capi.CUCOStaticHashmap(torch.zeros(0, dtype=torch.int64).cuda(),
                                torch.zeros(0, dtype=torch.int64).cuda(), 0.5)
    assert h0.query(torch.tensor([1, 2]).cuda()).tolist() == [-1, -1]


def test_duplicate_keys_one_winner(capi):
    keys = torch.tensor([5, 5, 5, 9]).cuda()
    h = capi.CUCOStaticHashmap(keys, torch.tensor([1, 2, 3, 4]).cuda(), 0.5)
    a, b = h.query(torch.tensor([5, 9]).cuda()).tolist()
    assert a in (1, 2, 3) and b == 4


def test_errors_are_exceptions(capi):
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        capi.CUCOStaticHashmap(torch.tensor([1]), torch.tensor([1]).cuda(), 0.5)
    with pytest.raises(RuntimeError, match="int32 or int64"):
        capi.CUCOStaticHashmap(torch.tensor([1.0]).cuda(), torch.tensor([1]).cuda(), 0.5)
    h = capi.CUCOStaticHashmap(torch.tensor([1]).cuda(), torch.tensor([1]).cuda(), 0.5)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        h.query(torch.tensor([1]))


def test_full_size_membership_property(capi):
    """Hashmap microbenchmark configuration at full size: 4,194,304 unique keys in [0, 2^40), LF 0.5,
    16,777,216 queries half members / half non-members. Checked through
    properties that need no CPU map: members return their insertion index,
    non-members return -1, and the sum of results is the closed form."""
    g = torch.Generator(device="cuda").manual_seed(2)
    n = 4_194_304
    keys = torch.unique(torch.randint(0, 1 << 40, (n + n // 8,), device="cuda", generator=g))
    keys = keys[torch.randperm(keys.numel(), device="cuda", generator=g)][:n].contiguous()
    assert keys.numel() == n
    vals = torch.arange(n, device="cuda")
    h = capi.CUCOStaticHashmap(keys, vals, 0.5)
    assert h.capacity() == 2 * n
    pick = torch.randint(0, n, (8_388_608,), device="cuda", generator=g)
    non = torch.randint(0, 1 << 40, (8_388_608,), device="cuda", generator=g) | (1 << 41)   # outside the key range
    req = torch.cat([keys[pick], non])
    perm = torch.randperm(req.numel(), device="cuda", generator=g)
    out = h.query(req[perm])
    expect = torch.cat([pick, torch.full_like(non, -1)])[perm]
    assert torch.equal(out, expect)


# ---- layouts chosen from the keys ------------------------------------------------------------------
# Whatever layout the constructor picks (bucket table with 16- or 8-byte slots, direct table, id range),
# query() must answer like a dict of the pairs (include/cuco_hashmap.cuh:81-87): the oracle is the judge.

def _probe_requests(rng, keys, lo, hi):
    """Members, near misses on both sides of the key range, far values, values beyond 32 bits, -1."""
    return np.concatenate([keys, rng.integers(lo - 50, hi + 50, size=5000), [lo - 1, hi + 1, -1, -2, 0],
                           rng.integers(-2**40, 2**40, size=1000), [2**31, 2**32, 2**32 + int(keys[0]), -2**31]])


_LAYOUT_CASES = ["range_identity", "range_offset", "range_shuffled", "range_from_zero_one_key", "range_with_repeat",
                 "range_negative_values", "direct_permuted", "direct_sparse", "direct_too_sparse", "negative_keys",
                 "values_beyond_32_bits", "rank_sorted_sparse", "rank_offset_values", "rank_values_beyond_32_bits",
                 "rank_one_id_in_100", "rank_too_sparse", "rank_block_edges", "rank_broken_by_one_value",
                 "rank_broken_by_order"]


@pytest.mark.parametrize("kd,vd,case", [(kd, vd, case) for kd in (np.int32, np.int64) for vd in (np.int32, np.int64)
                                        for case in _LAYOUT_CASES
                                        if not (case.endswith("values_beyond_32_bits") and vd is np.int32)])
def test_layouts_answer_like_a_dict(capi, oracle, kd, vd, case):
    rng = np.random.default_rng(len(case) * 7 + np.dtype(kd).itemsize + 3 * np.dtype(vd).itemsize)
    n = 30_000
    expect_layout = None
    if case == "range_identity":                     # a cache holding ids 0 .. n-1 in slot order
        keys = np.arange(n)
        vals = keys.copy()
        expect_layout = "range"
    elif case == "range_offset":                     # ids 1000 .. 1000+n-1 -> slots 7 ..
        keys = np.arange(1000, 1000 + n)
        vals = keys - 993
        expect_layout = "range"
    elif case == "range_shuffled":                   # the same pairs in any order
        keys = rng.permutation(np.arange(500, 500 + n))
        vals = keys - 500
        expect_layout = "range"
    elif case == "range_from_zero_one_key":
        keys, vals = np.array([0]), np.array([5])
        expect_layout = "range"
    elif case == "range_with_repeat":                # n pairs over n ids but one id twice, so one is missing
        keys = np.arange(n)
        keys[17] = 16
        vals = keys.copy()
        expect_layout = "direct"
    elif case == "range_negative_values":            # value = key - 20: key 19 maps to -1, i.e. reads as absent
        keys = np.arange(n)
        vals = keys - 20
        expect_layout = "range"
    elif case == "direct_permuted":                  # dense ids, slots in insertion (hotness) order
        keys = rng.permutation(n)
        vals = np.arange(n)
        expect_layout = "direct"
    elif case == "direct_sparse":                    # a third of an id universe
        keys = rng.choice(3 * n, size=n, replace=False) + 12345
        vals = np.arange(n)
        expect_layout = "direct"
    elif case == "direct_too_sparse":                # 1 id in 20: the bucket table is much smaller
        keys = rng.choice(20 * n, size=n, replace=False)
        vals = np.arange(n)
        expect_layout = "buckets"
    elif case == "negative_keys":                    # dense, but ids below zero: bucket table
        keys = rng.permutation(n) - 100
        keys = keys[keys != -1]                      # -1 is the empty key
        vals = np.arange(keys.size)
        expect_layout = "buckets"
    elif case == "values_beyond_32_bits":            # dense keys whose values need 64 bits
        keys = rng.permutation(n)
        vals = np.arange(n) + 2**33
        expect_layout = "buckets"
    elif case == "rank_sorted_sparse":               # a cache kept in id order: slot = rank of the id
        keys = np.sort(rng.choice(3 * n, size=n, replace=False)) + 12345
        vals = np.arange(n)
        expect_layout = "rank"
    elif case == "rank_offset_values":
        keys = np.sort(rng.choice(10 * n, size=n, replace=False))
        vals = np.arange(n) + 77
        expect_layout = "rank"
    elif case == "rank_values_beyond_32_bits":       # ranks are computed, so wide values cost nothing
        keys = np.sort(rng.choice(5 * n, size=n, replace=False))
        vals = np.arange(n) + 2**33
        expect_layout = "rank"
    elif case == "rank_one_id_in_100":               # most 96-id blocks hold no key or one
        keys = np.sort(rng.choice(100 * n, size=n, replace=False))
        vals = np.arange(n)
        expect_layout = "rank"
    elif case == "rank_too_sparse":                  # 1 id in 400: the bitmap would outgrow the bucket table
        keys = np.sort(rng.choice(400 * n, size=n, replace=False))
        vals = np.arange(n)
        expect_layout = "buckets"
    elif case == "rank_block_edges":                 # first / last id of the 96-id blocks and of their 32-bit words
        a = np.sort(rng.choice(4000, size=1500, replace=False))[:, None] * 96
        keys = np.unique((a + np.array([0, 31, 32, 63, 64, 95])[None, :]).ravel()) + 5
        vals = np.arange(keys.size)
        expect_layout = "rank"
    elif case == "rank_broken_by_one_value":         # ascending ids, but two slots swapped: a plain table again
        keys = np.sort(rng.choice(3 * n, size=n, replace=False))
        vals = np.arange(n)
        vals[[100, 20_000]] = vals[[20_000, 100]]
        expect_layout = "direct"
    else:                                            # consecutive values, but two ids out of order
        keys = np.sort(rng.choice(3 * n, size=n, replace=False))
        keys[[7, 8]] = keys[[8, 7]]
        vals = np.arange(n)
        expect_layout = "direct"
    keys, vals = keys.astype(kd), vals.astype(vd)
    h = capi.CUCOStaticHashmap(_cuda(keys), _cuda(vals), 0.8)
    assert h.layout() == expect_layout
    ref = oracle.Hashmap(keys, vals, 0.8)
    lo, hi = int(keys.min()), int(keys.max())
    req = _probe_requests(rng, keys.astype(np.int64), lo, hi)
    for rd in (np.int32, np.int64):
        r = req.astype(rd)                           # int32: two's-complement narrowing, like .to(int32)
        out = h.query(_cuda(r))
        assert out.dtype == TD[vd]
        if case == "range_with_repeat":
            # the repeated key has one winner among its two values; every other answer is determined
            want = ref.query(r)
            got = out.cpu().numpy()
            dup = r.astype(kd) == 16
            assert np.array_equal(got[~dup], want[~dup]) and set(got[dup].tolist()) <= {16}
            assert got[r.astype(kd) == 17].tolist() == [-1] * int((r.astype(kd) == 17).sum())
        else:
            assert np.array_equal(out.cpu().numpy(), ref.query(r))
    assert h.capacity() == int(np.ceil(keys.size / 0.8))
    if expect_layout == "range":
        assert h.memory_usage() == 0
    elif expect_layout == "direct":
        assert h.memory_usage() <= (hi - lo + 1) * 4 + 128
    elif expect_layout == "rank":
        assert h.memory_usage() <= (hi - lo + 1 + 95) // 96 * 16 + 128


def test_wide_dtypes_with_small_ids_use_narrow_slots(capi, oracle):
    """int64 keys and values that all fit 32 bits are stored in 8-byte slots; requests that do not fit
    32 bits are absent (not truncated: only int32-KEYED maps narrow their requests)."""
    rng = np.random.default_rng(3)
    keys = rng.choice(50_000_000, size=40_000, replace=False).astype(np.int64)
    vals = rng.integers(0, 2**31 - 1, size=keys.size).astype(np.int64)
    h = capi.CUCOStaticHashmap(_cuda(keys), _cuda(vals), 0.5)
    assert h.layout() == "buckets" and h.memory_usage() == 40_000 * 8 * 2
    req = np.concatenate([keys, keys + 2**32, keys - 2**32, rng.integers(0, 50_000_000, size=10_000)])
    assert np.array_equal(h.query(_cuda(req)).cpu().numpy(), oracle.Hashmap(keys, vals, 0.5).query(req))
    wide = capi.CUCOStaticHashmap(_cuda(keys + 2**32), _cuda(vals), 0.5)        # keys beyond 32 bits: 16-byte slots
    assert wide.memory_usage() == 40_000 * 16 * 2
    assert np.array_equal(wide.query(_cuda(req)).cpu().numpy(), oracle.Hashmap(keys + 2**32, vals, 0.5).query(req))


@pytest.mark.parametrize("layout", ["range", "direct", "rank"])
def test_flat_layouts_route_fetch_set_and_sampling(capi, oracle, layout):
    """cache_fetch / cache_set / csr_cache_sampling through a map in a flat layout against the oracle, with
    cache rows made different from the host rows so that routing shows."""
    rng = np.random.default_rng(8)
    n, c = 5000, 2000
    ids = np.arange(100, 100 + c) if layout == "range" else rng.choice(n, size=c, replace=False)
    if layout == "rank":
        ids = np.sort(ids)
    slots = ids - 100 if layout == "range" else np.arange(c)
    h = capi.CUCOStaticHashmap(_cuda(ids), _cuda(slots), 0.8)
    assert h.layout() == layout
    ref = oracle.Hashmap(ids, slots, 0.8)
    table = rng.standard_normal((n, 24)).astype(np.float32)
    host = torch.from_numpy(table.copy()).pin_memory()
    cache_np = np.empty((c, 24), np.float32)
    cache_np[slots] = table[ids] + 1000.0
    cache = _cuda(cache_np)
    q = rng.integers(0, n, size=7001)
    out = capi.cache_fetch(host, cache, _cuda(q), h)
    assert np.array_equal(out.cpu().numpy(), oracle.fetch(table, cache_np, q, hashmap=ref))
    w = rng.choice(n, size=1500, replace=False)
    upd = rng.standard_normal((1500, 24)).astype(np.float32)
    capi.cache_set(host, cache, _cuda(w), _cuda(upd), h)
    torch.cuda.synchronize()
    want_host, want_cache = table.copy(), cache_np.copy()
    oracle.set_rows(want_host, want_cache, w, upd, hashmap=ref)
    assert np.array_equal(host.numpy(), want_host) and np.array_equal(cache.cpu().numpy(), want_cache)
    # write-through: a hit also updates the host row
    upd2 = rng.standard_normal((1500, 24)).astype(np.float32)
    capi.cache_set(host, cache, _cuda(w), _cuda(upd2), h, write_through=True)
    torch.cuda.synchronize()
    want_host[w] = upd2
    hit = ref.query(w) >= 0
    want_cache[ref.query(w)[hit]] = upd2[hit]
    assert np.array_equal(host.numpy(), want_host) and np.array_equal(cache.cpu().numpy(), want_cache)
    # sampling: cached rows (a sub-CSR in map order) and cold rows give what the uncached sampler gives
    deg = rng.integers(0, 30, size=n)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    indices = rng.integers(0, n, size=int(indptr[-1])).astype(np.int32)
    ip, ix = torch.from_numpy(indptr).pin_memory(), torch.from_numpy(indices).pin_memory()
    order = np.empty(c, np.int64)
    order[slots] = ids
    gp, gi = capi.create_subcsr(ip, ix, _cuda(order))
    seeds = _cuda(rng.permutation(n)[:3000])
    a = capi.csr_cache_sampling(ip, ix, gp, gi, h, seeds, 7, False, seed=3)
    b = capi.csr_sampling(ip, ix, seeds, 7, False, seed=3)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    esp, esi = oracle.sample(indptr, indices, seeds.cpu().numpy(), 7, False, seed=3, algo="floyd")
    assert np.array_equal(a[0].cpu().numpy(), esp) and np.array_equal(a[1].cpu().numpy(), esi)


def test_planned_build_through_the_c_abi(cabi):
    """shmt_hashmap_plan / shmt_hashmap_create_planned with raw pointers: the layout struct, the sizes it
    asks for and the answers of the built map."""
    import ctypes
    lib = cabi.load()
    stream = cabi.current_stream()
    keys = torch.arange(10, 1034).cuda()
    vals = (keys - 10).contiguous()
    n = keys.numel()
    sb = lib.shmt_hashmap_plan_scratch_bytes(n)
    assert sb >= 256 + n
    scratch = torch.empty(sb, dtype=torch.uint8, device="cuda")
    lay = cabi.HashmapLayout()
    cabi.check(lib.shmt_hashmap_plan(keys.data_ptr(), vals.data_ptr(), n, 8, 8, 0.8, scratch.data_ptr(), sb,
                                     ctypes.byref(lay), stream))
    assert (lay.kind, lay.lo, lay.span, lay.delta) == (2, 10, 1024, -10)
    table = torch.empty(max(lay.table_bytes, 128), dtype=torch.uint8, device="cuda")
    handle = ctypes.c_void_p()
    cabi.check(lib.shmt_hashmap_create_planned(ctypes.byref(handle), ctypes.byref(lay), keys.data_ptr(),
                                               vals.data_ptr(), n, 8, 8, 0.8, table.data_ptr(), table.numel(), stream))
    assert lib.shmt_hashmap_kind(handle) == 2 and lib.shmt_hashmap_used_bytes(handle) == 0
    req = torch.tensor([9, 10, 500, 1033, 1034, -1]).cuda()
    out = torch.empty_like(req)
    cabi.check(lib.shmt_hashmap_query(handle, req.data_ptr(), 8, req.numel(), out.data_ptr(), stream))
    assert out.tolist() == [-1, 0, 490, 1023, -1, -1]
    lib.shmt_hashmap_destroy(handle)
    # scattered 64-bit keys: bucket table with 16-byte slots, sized like shmt_hashmap_table_bytes
    big = (torch.arange(n).cuda() * 1_000_003 + (1 << 35)).contiguous()
    cabi.check(lib.shmt_hashmap_plan(big.data_ptr(), vals.data_ptr(), n, 8, 8, 0.5, scratch.data_ptr(), sb,
                                     ctypes.byref(lay), stream))
    assert (lay.kind, lay.slot_bytes) == (0, 16) and lay.table_bytes == lib.shmt_hashmap_table_bytes(n, 0.5, 8, 8)
    small = torch.empty(1024, dtype=torch.uint8, device="cuda")
    assert lib.shmt_hashmap_plan(big.data_ptr(), vals.data_ptr(), n, 8, 8, 0.5, small.data_ptr(), 1024,
                                 ctypes.byref(lay), stream) == -4                     # scratch too small
