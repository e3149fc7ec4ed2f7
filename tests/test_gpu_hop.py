"""One fused hop (sample + relabel queued without a host wait between them)
against the two separate operators it replaces, and the device-side segment
length of shmt_relabel_segments against the oracle. Bit-exact throughout."""
import ctypes

import numpy as np
import pytest
import torch

from shmtensor_amd.synthetic import rmat_csr

pytestmark = pytest.mark.gpu


def _graph(scale=14, edge_factor=12, seed=3, ptr_dt=torch.int64, idx_dt=torch.int64):
    indptr, indices = rmat_csr(scale, edge_factor, seed)
    return indptr.to(ptr_dt), indices.to(idx_dt)


def _two_step(capi, indptr, indices, cache, seeds, k, replace, **kw):
    if cache is None:
        sp, si = capi.csr_sampling(indptr, indices, seeds, k, replace, **kw)
    else:
        gp, gi, h = cache
        sp, si = capi.csr_cache_sampling(indptr, indices, gp, gi, h, seeds, k, replace, **kw)
    uniq, (_, lab) = capi.tensor_relabel([seeds, si])
    return sp, si, uniq, lab


def _hop(capi, indptr, indices, cache, seeds, k, replace, **kw):
    gp, gi, h = cache if cache is not None else (None, None, None)
    return capi.sample_hop(indptr, indices, gp, gi, h, seeds, k, replace, **kw)


def _same(a, b):
    assert len(a) == len(b)
    for x, y in zip(a, b):
        assert x.dtype == y.dtype and x.shape == y.shape and x.device == y.device
        assert torch.equal(x, y)


@pytest.mark.parametrize("replace", [False, True])
@pytest.mark.parametrize("k", [1, 5, 25, 64, 100])
@pytest.mark.parametrize("seed_dt", [torch.int32, torch.int64])
def test_hop_equals_sampling_then_relabel_device_graph(capi, replace, k, seed_dt):
    indptr, indices = _graph()
    indptr, indices = indptr.cuda(), indices.cuda()
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(k)
    for S in (1, 7, 1024, 1025, 6000):
        seeds = torch.randint(0, n, (S,), generator=g).to(seed_dt).cuda()   # with repeats
        _same(_hop(capi, indptr, indices, None, seeds, k, replace),
              _two_step(capi, indptr, indices, None, seeds, k, replace))


@pytest.mark.parametrize("ptr_dt,idx_dt", [(torch.int64, torch.int32), (torch.int32, torch.int32),
                                           (torch.int64, torch.int64)])
def test_hop_cached_pinned_graph(capi, ptr_dt, idx_dt):
    indptr, indices = _graph(ptr_dt=ptr_dt, idx_dt=idx_dt)
    indptr, indices = indptr.cpu().pin_memory(), indices.cpu().pin_memory()
    n = indptr.numel() - 1
    hot = torch.randperm(n, generator=torch.Generator().manual_seed(1))[: n // 4].cuda()
    gp, gi = capi.create_subcsr(indptr, indices, hot)
    h = capi.CUCOStaticHashmap(hot.int(), torch.arange(hot.numel(), dtype=torch.int32).cuda(), 0.8)
    cache = (gp, gi, h)
    seeds = torch.randperm(n, generator=torch.Generator().manual_seed(2))[:3000].int().cuda()
    for replace in (False, True):
        for kw in ({}, {"seed": 99, "stream_id": 3}):
            got = _hop(capi, indptr, indices, cache, seeds, 10, replace, **kw)
            _same(got, _two_step(capi, indptr, indices, cache, seeds, 10, replace, **kw))
            _same(got, _hop(capi, indptr, indices, None, seeds, 10, replace, **kw))   # cache is transparent


def test_hop_degenerate_inputs(capi):
    # node 0: 3 neighbours, node 1: none, node 2: 1 neighbour
    indptr = torch.tensor([0, 3, 3, 4]).cuda()
    indices = torch.tensor([2, 1, 0, 2]).cuda()
    empty = torch.empty(0, dtype=torch.int64).cuda()
    sp, si, uniq, lab = capi.sample_hop(indptr, indices, None, None, None, empty, 5, False)
    assert sp.tolist() == [0] and si.numel() == 0 and uniq.numel() == 0 and lab.numel() == 0
    only_isolated = torch.tensor([1, 1]).cuda()
    sp, si, uniq, lab = capi.sample_hop(indptr, indices, None, None, None, only_isolated, 5, False)
    assert sp.tolist() == [0, 0, 0] and si.numel() == 0 and uniq.tolist() == [1] and lab.numel() == 0
    seeds = torch.tensor([2, 1, 0]).cuda()
    sp, si, uniq, lab = capi.sample_hop(indptr, indices, None, None, None, seeds, 5, False)
    assert sp.tolist() == [0, 1, 1, 4] and si[0].item() == 2 and sorted(si[1:].tolist()) == [0, 1, 2]
    assert uniq.tolist() == [2, 1, 0] and torch.equal(uniq[lab], si)
    sp0, si0, uniq0, lab0 = capi.sample_hop(indptr, indices, None, None, None, seeds, 0, False)
    assert sp0.tolist() == [0, 0, 0, 0] and si0.numel() == 0 and uniq0.tolist() == [2, 1, 0]
    with pytest.raises(RuntimeError):
        capi.sample_hop(indptr, indices, None, None, None, seeds.float(), 5, False)


def test_hop_chain_matches_dataloader_protocol(capi):
    """Three hops chained as the dataloader does (python/shmtensor/sampling.py:128-143):
    the unique ids of one hop seed the next; seeds stay a prefix of unique."""
    indptr, indices = _graph(scale=15)
    indptr, indices = indptr.cuda(), indices.cuda()
    seeds = torch.randperm(indptr.numel() - 1, generator=torch.Generator().manual_seed(5))[:1000].cuda()
    a = b = seeds
    for hop, k in enumerate([10, 10, 5]):
        got = _hop(capi, indptr, indices, None, a, k, False, seed=11, stream_id=hop)
        want = _two_step(capi, indptr, indices, None, b, k, False, seed=11, stream_id=hop)
        _same(got, want)
        assert torch.equal(got[2][: a.numel()], a)
        assert torch.equal(got[2][got[3]], got[1])
        a, b = got[2], want[2]


@pytest.mark.parametrize("len_bytes", [4, 8])
@pytest.mark.parametrize("true_len", [0, 1, 2047, 2048, 5000, 20000])
def test_relabel_segments_device_length(cabi, oracle, len_bytes, true_len):
    """The last segment's length read on the device: buffers and launches sized
    for the bound, results those of the true length."""
    lib = cabi.load()
    rng = np.random.default_rng(true_len + len_bytes)
    head = rng.integers(0, 3000, size=700).astype(np.int32)
    bound = 20000
    tail = rng.integers(0, 3000, size=bound).astype(np.int64)      # entries past true_len must be ignored
    exp_unique, exp_parts = oracle.relabel([head, tail[:true_len]])
    exp_labels = np.concatenate(exp_parts)
    d_head, d_tail = torch.from_numpy(head).cuda(), torch.from_numpy(tail).cuda()
    d_len = torch.tensor([true_len], dtype=torch.int32 if len_bytes == 4 else torch.int64).cuda()
    n_max = head.size + bound
    total = torch.empty(n_max, dtype=torch.int64).cuda()
    unique = torch.empty(n_max, dtype=torch.int64).cuda()
    labels = torch.empty(n_max, dtype=torch.int64).cuda()
    sbytes = lib.shmt_relabel_scratch_bytes(n_max)
    scratch = torch.empty(sbytes, dtype=torch.uint8).cuda()
    count = torch.full((1,), -5, dtype=torch.int64).cuda()
    vp = ctypes.c_void_p
    ptrs = (vp * 2)(d_head.data_ptr(), d_tail.data_ptr())
    lens = (ctypes.c_int64 * 2)(head.size, bound)
    widths = (ctypes.c_int * 2)(4, 8)
    cabi.check(lib.shmt_relabel_segments(ptrs, lens, widths, 2, d_len.data_ptr(), len_bytes, 8,
                                         total.data_ptr(), scratch.data_ptr(), sbytes, unique.data_ptr(),
                                         labels.data_ptr(), count.data_ptr(), cabi.current_stream()))
    torch.cuda.synchronize()
    n = head.size + true_len
    u = int(count.item())
    assert u == exp_unique.size
    assert np.array_equal(unique[:u].cpu().numpy(), exp_unique)
    assert np.array_equal(labels[:n].cpu().numpy(), exp_labels)
    assert np.array_equal(total[:n].cpu().numpy(), np.concatenate([head.astype(np.int64), tail[:true_len]]))


def test_relabel_segments_device_length_clamped_and_rejected(cabi):
    lib = cabi.load()
    head = torch.arange(10, dtype=torch.int64).cuda()
    tail = torch.arange(5, 15, dtype=torch.int64).cuda()
    too_long = torch.tensor([1000], dtype=torch.int64).cuda()       # beyond the bound: clamped to it
    total, unique, labels = (torch.empty(20, dtype=torch.int64).cuda() for _ in range(3))
    sbytes = lib.shmt_relabel_scratch_bytes(20)
    scratch = torch.empty(sbytes, dtype=torch.uint8).cuda()
    count = torch.zeros(1, dtype=torch.int64).cuda()
    vp = ctypes.c_void_p
    ptrs = (vp * 2)(head.data_ptr(), tail.data_ptr())
    lens = (ctypes.c_int64 * 2)(10, 10)
    widths = (ctypes.c_int * 2)(8, 8)
    args = (total.data_ptr(), scratch.data_ptr(), sbytes, unique.data_ptr(), labels.data_ptr(), count.data_ptr(),
            cabi.current_stream())
    cabi.check(lib.shmt_relabel_segments(ptrs, lens, widths, 2, too_long.data_ptr(), 8, 8, *args))
    torch.cuda.synchronize()
    assert count.item() == 15 and unique[:15].tolist() == list(range(15))
    assert labels.tolist() == list(range(10)) + list(range(5, 15))
    assert lib.shmt_relabel_segments(ptrs, lens, widths, 2, too_long.data_ptr(), 3, 8, *args) == -1
    assert b"last_len_bytes" in lib.shmt_last_error()


@pytest.mark.parametrize("in_flight", [1, 3, 8])
def test_sample_blocks_equals_hop_by_hop(capi, in_flight):
    """Several batches driven concurrently (host threads + side streams): the
    same results as one sample_hop call per hop and batch."""
    indptr, indices = _graph(scale=15)
    indptr_h, indices_h = indptr.cpu().pin_memory(), indices.cpu().pin_memory()
    n = indptr.numel() - 1
    hot = torch.randperm(n, generator=torch.Generator().manual_seed(1))[: n // 3].cuda()
    gp, gi = capi.create_subcsr(indptr_h, indices_h, hot)
    h = capi.CUCOStaticHashmap(hot, torch.arange(hot.numel()).cuda(), 0.8)
    g = torch.Generator().manual_seed(9)
    sizes = [1000, 1, 0, 257, 4000, 33, 1024, 2048, 5, 700, 1500]
    batches = [torch.randperm(n, generator=g)[:s].cuda() for s in sizes]
    rng = [100 + b for b in range(len(batches))]
    picks = [7, 12, 3]
    for repeat in range(3):              # also exercises reuse of the side streams' cached memory
        got = capi.sample_blocks(indptr_h, indices_h, gp, gi, h, batches, picks, False, seeds_rng=rng,
                                 max_in_flight=in_flight)
        assert len(got) == len(batches)
        for b, seeds in enumerate(batches):
            assert len(got[b]) == len(picks)
            for hop, k in enumerate(picks):
                want = capi.sample_hop(indptr_h, indices_h, gp, gi, h, seeds, k, False, seed=rng[b], stream_id=hop)
                _same(got[b][hop], want)
                seeds = want[2]
            # results are usable on the calling stream right away
            assert got[b][-1][2].sum().item() == seeds.sum().item()


def test_sample_blocks_arguments(capi):
    indptr = torch.tensor([0, 3, 3, 4]).cuda()
    indices = torch.tensor([2, 1, 0, 2]).cuda()
    assert capi.sample_blocks(indptr, indices, None, None, None, [], [5], False) == []
    seeds = [torch.tensor([0, 2]).cuda(), torch.tensor([1]).cuda()]
    a = capi.sample_blocks(indptr, indices, None, None, None, seeds, [5, 2], False)       # default RNG seed
    for b in range(2):
        first = capi.sample_hop(indptr, indices, None, None, None, seeds[b], 5, False)
        _same(a[b][0], first)
        _same(a[b][1], capi.sample_hop(indptr, indices, None, None, None, first[2], 2, False))
    assert capi.sample_blocks(indptr, indices, None, None, None, seeds, [], False) == [[], []]
    with pytest.raises(RuntimeError):
        capi.sample_blocks(indptr, indices, None, None, None, seeds, [5], False, seeds_rng=[1])
    with pytest.raises(RuntimeError):
        capi.sample_blocks(indptr, indices, None, None, None, seeds, [5], False, max_in_flight=0)
    with pytest.raises(RuntimeError):    # an error raised on a worker thread reaches the caller
        capi.sample_blocks(indptr.cpu(), indices, None, None, None, seeds, [5], False, max_in_flight=2)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):          # called with a non-default current stream
        b = capi.sample_blocks(indptr, indices, None, None, None, seeds, [5, 2], False, max_in_flight=2)
    side.synchronize()
    for x, y in zip(a, b):
        for hx, hy in zip(x, y):
            _same(hx, hy)


def test_hop_very_wide_fanout_and_hub(capi):
    """k beyond the LDS staging limit on a hub row (positions staged in the output segment)."""
    deg = 20000
    indptr = torch.tensor([0, deg, deg + 3, deg + 3]).cuda()
    indices = torch.cat([torch.arange(3, deg + 3), torch.tensor([0, 1, 2])]).cuda()
    seeds = torch.tensor([1, 0, 2, 0]).cuda()
    for k in (9000, 65):
        for replace in (False, True):
            got = capi.sample_hop(indptr, indices, None, None, None, seeds, k, replace, seed=3)
            _same(got, _two_step(capi, indptr, indices, None, seeds, k, replace, seed=3))
            if not replace:
                hub = got[1][got[0][1]:got[0][2]]
                assert hub.numel() == k and hub.unique().numel() == k


def test_sample_hop_c_abi_matches_separate_entry_points(cabi):
    """shmt_sample_hop against shmt_sample_plan + shmt_sample_pick + shmt_relabel_segments, raw pointers."""
    lib = cabi.load()
    indptr, indices = _graph(scale=13, ptr_dt=torch.int64, idx_dt=torch.int32)
    indptr, indices = indptr.cuda(), indices.cuda()
    n = indptr.numel() - 1
    vp, i64 = ctypes.c_void_p, ctypes.c_int64
    stream = cabi.current_stream()
    for S, k in ((300, 6), (3000, 20), (50, 70)):
        seeds = torch.randperm(n, generator=torch.Generator().manual_seed(S))[:S].cuda()      # int64
        n_max = S + S * k

        def buffers():
            return dict(sp=torch.empty(S + 1, dtype=torch.int64).cuda(), si=torch.empty(S * k, dtype=torch.int32).cuda(),
                        plan=torch.empty(lib.shmt_sample_plan_bytes(S), dtype=torch.uint8).cuda(),
                        total=torch.empty(n_max, dtype=torch.int64).cuda(), unique=torch.empty(n_max, dtype=torch.int64).cuda(),
                        labels=torch.empty(n_max, dtype=torch.int64).cuda(),
                        scratch=torch.empty(lib.shmt_relabel_scratch_bytes(n_max), dtype=torch.uint8).cuda(),
                        nnz=torch.zeros(1, dtype=torch.int64).cuda(), count=torch.zeros(1, dtype=torch.int64).cuda())
        a, b = buffers(), buffers()
        cabi.check(lib.shmt_sample_hop(indptr.data_ptr(), 8, indices.data_ptr(), 4, None, None, None, seeds.data_ptr(), 8,
                                       S, k, 0, 42, 1, a["sp"].data_ptr(), a["si"].data_ptr(), a["plan"].data_ptr(),
                                       a["plan"].numel(), 8, a["total"].data_ptr(), a["scratch"].data_ptr(),
                                       a["scratch"].numel(), a["unique"].data_ptr(), a["labels"].data_ptr(),
                                       a["nnz"].data_ptr(), a["count"].data_ptr(), stream))
        cabi.check(lib.shmt_sample_plan(indptr.data_ptr(), 8, None, None, seeds.data_ptr(), 8, S, k, 0, b["sp"].data_ptr(),
                                        b["plan"].data_ptr(), b["plan"].numel(), b["nnz"].data_ptr(), stream))
        cabi.check(lib.shmt_sample_pick(indices.data_ptr(), None, 4, seeds.data_ptr(), 8, S, k, 0, b["sp"].data_ptr(), 8,
                                        b["plan"].data_ptr(), b["si"].data_ptr(), 42, 1, stream))
        torch.cuda.synchronize()
        nnz = int(b["nnz"].item())
        ptrs = (vp * 2)(seeds.data_ptr(), b["si"].data_ptr())
        cabi.check(lib.shmt_relabel_segments(ptrs, (i64 * 2)(S, nnz), (ctypes.c_int * 2)(8, 4), 2, None, 0, 8,
                                             b["total"].data_ptr(), b["scratch"].data_ptr(), b["scratch"].numel(),
                                             b["unique"].data_ptr(), b["labels"].data_ptr(), b["count"].data_ptr(), stream))
        torch.cuda.synchronize()
        assert int(a["nnz"].item()) == nnz and int(a["count"].item()) == int(b["count"].item())
        u = int(b["count"].item())
        assert torch.equal(a["sp"], b["sp"]) and torch.equal(a["si"][:nnz], b["si"][:nnz])
        assert torch.equal(a["total"][:S + nnz], b["total"][:S + nnz])
        assert torch.equal(a["unique"][:u], b["unique"][:u]) and torch.equal(a["labels"][:S + nnz], b["labels"][:S + nnz])
    # argument checks
    assert lib.shmt_sample_hop(indptr.data_ptr(), 8, indices.data_ptr(), 4, None, None, None, seeds.data_ptr(), 8, 0, 5, 0,
                               1, 0, None, None, None, 0, 8, None, None, 0, None, None, None, None, stream) == -1
    assert b"must be >= 1" in lib.shmt_last_error()


@pytest.mark.parametrize("odd_ids", ["none", "beyond_32_bits", "negative", "uint32_max"])
def test_hop_relabel_table_format_follows_the_id_range(capi, oracle, odd_ids):
    """The hop's relabel uses packed 8-byte slots while every id fits 32 bits and falls
    back to 16-byte slots otherwise; both must give the oracle's labels. Heavy
    repetition of a few ids and dense id ranges stress slot take-overs in the packed table."""
    rng = np.random.default_rng(5)
    n, deg = 4000, 12
    indptr = np.arange(0, (n + 1) * deg, deg, dtype=np.int64)
    indices = rng.integers(0, 600, size=n * deg).astype(np.int64)          # few distinct ids, many repeats
    indices[::7] = rng.integers(0, 2**31, size=indices[::7].size)           # and some spread over 31 bits
    if odd_ids == "beyond_32_bits":
        indices[5::11] += 2**32
    elif odd_ids == "negative":
        indices[3::13] = -indices[3::13] - 2
    elif odd_ids == "uint32_max":
        indices[2::9] = 2**32 - 1
    seeds = rng.permutation(n)[:3000].astype(np.int64)
    ip, ix, sd = (torch.from_numpy(x).cuda() for x in (indptr, indices, seeds))
    for k in (12, 5):
        sp, si, uniq, lab = capi.sample_hop(ip, ix, None, None, None, sd, k, False, seed=1)
        exp_unique, (exp_seed_labels, exp_labels) = oracle.relabel([seeds, si.cpu().numpy()])
        assert np.array_equal(uniq.cpu().numpy(), exp_unique)
        assert np.array_equal(lab.cpu().numpy(), exp_labels)
        _same((sp, si, uniq, lab), _two_step(capi, ip, ix, None, sd, k, False, seed=1))


@pytest.mark.parametrize("max_rows", [None, 0, 600, 100000])
@pytest.mark.parametrize("in_flight", [1, 4])
@pytest.mark.parametrize("cached_rows", [True, False])
def test_sample_blocks_fetch_equals_sample_blocks_then_fetch(capi, max_rows, in_flight, cached_rows):
    """The feature fetch queued behind the last relabel (row count read on the
    device) returns what a separate fetch of the batch's input nodes returns,
    whether the speculative output is the bound, too small (600 rows: the
    count is then waited for), generous, or not used at all (0)."""
    indptr, indices = _graph(scale=13)
    indptr_h, indices_h = indptr.cpu().pin_memory(), indices.cpu().pin_memory()
    n = indptr.numel() - 1
    gen = torch.Generator().manual_seed(4)
    hot = torch.randperm(n, generator=gen)[: n // 3].cuda()
    gp, gi = capi.create_subcsr(indptr_h, indices_h, hot)
    h = capi.CUCOStaticHashmap(hot, torch.arange(hot.numel()).cuda(), 0.8)
    table = torch.randn(n, 24, generator=gen).pin_memory()
    rows_hot = torch.randperm(n, generator=gen)[: n // 4]
    gpu_rows = (table[rows_hot] + 1.0).cuda()          # a hit is told from a miss by its content
    rows_map = capi.CUCOStaticHashmap(rows_hot.cuda(), torch.arange(rows_hot.numel()).cuda(), 0.8)
    sizes = [300, 1, 0, 257, 1500, 33]
    batches = [torch.randperm(n, generator=gen)[:s].cuda() for s in sizes]
    rng = [50 + b for b in range(len(batches))]
    for picks in ([4, 6], [3], []):
        want_hops = capi.sample_blocks(indptr_h, indices_h, gp, gi, h, batches, picks, False, seeds_rng=rng)
        for repeat in range(2):
            got = capi.sample_blocks_fetch(indptr_h, indices_h, gp, gi, h, batches, picks, False, table,
                                           gpu_rows if cached_rows else None,
                                           rows_map if cached_rows else None, seeds_rng=rng,
                                           max_in_flight=in_flight, max_rows=max_rows)
            assert len(got) == len(batches)
            for b, (hops, rows) in enumerate(got):
                assert len(hops) == len(picks)
                for x, y in zip(hops, want_hops[b]):
                    _same(x, y)
                nodes = hops[-1][2] if picks else batches[b]
                if cached_rows:
                    want = capi.cache_fetch(table, gpu_rows, nodes, rows_map)
                else:
                    want = capi.uva_fetch(table, nodes)
                assert rows.shape == want.shape and torch.equal(rows, want)


def test_sample_blocks_fetch_arguments(capi):
    indptr = torch.tensor([0, 3, 3, 4]).cuda()
    indices = torch.tensor([2, 1, 0, 2]).cuda()
    table = torch.arange(12.0).reshape(3, 4).cuda()        # a device-resident table is accepted
    seeds = [torch.tensor([0, 2]).cuda(), torch.tensor([1]).cuda()]
    got = capi.sample_blocks_fetch(indptr, indices, None, None, None, seeds, [5], False, table, None, None)
    for hops, rows in got:
        assert torch.equal(rows, table[hops[-1][2]])
    one_d = torch.arange(3.0).cuda()                       # 1-D data gives 1-D rows, as cache_fetch does
    got = capi.sample_blocks_fetch(indptr, indices, None, None, None, seeds, [5], False, one_d, None, None)
    for hops, rows in got:
        assert rows.dim() == 1 and torch.equal(rows, one_d[hops[-1][2]])
    with pytest.raises(RuntimeError):                      # a hashmap without its cache rows
        capi.sample_blocks_fetch(indptr, indices, None, None, None, seeds, [5], False, table, None,
                                 capi.CUCOStaticHashmap(torch.arange(2).cuda(), torch.arange(2).cuda(), 0.5))
    with pytest.raises(RuntimeError):
        capi.sample_blocks_fetch(indptr, indices, None, None, None, seeds, [5], False, table, None, None,
                                 max_rows=-1)
    with pytest.raises(RuntimeError):                      # pageable host memory
        capi.sample_blocks_fetch(indptr, indices, None, None, None, seeds, [5], False, table.cpu(), None, None)


@pytest.mark.parametrize("cached", [False, True])
@pytest.mark.parametrize("S,picks,replace", [(200, (3, 4, 5), 0), (1500, (6, 3), 0), (40, (70, 2), 0),
                                             (300, (4, 4), 1)])
def test_c_abi_chained_hops_need_no_host_wait(cabi, cached, S, picks, replace):
    """shmt_sample_hop_chained: every hop takes its number of seeds from the device-side count of
    the hop before it and all hops are queued before anything is read back; results equal those
    of shmt_sample_hop called hop by hop with the host reading each count."""
    lib = cabi.load()
    indptr, indices = _graph(scale=13, ptr_dt=torch.int64, idx_dt=torch.int32)
    indptr, indices = indptr.cuda(), indices.cuda()
    n = indptr.numel() - 1
    stream = cabi.current_stream()
    gp = gi = hnd = None
    keep = []
    if cached:
        hot = torch.randperm(n, generator=torch.Generator().manual_seed(2))[: n // 2].cuda()
        deg = indptr[hot + 1] - indptr[hot]
        gp = torch.cat([torch.zeros(1, dtype=torch.int64).cuda(), torch.cumsum(deg, 0)])
        gi = torch.cat([indices[indptr[v]:indptr[v + 1]] for v in hot.tolist()])
        nbytes = lib.shmt_hashmap_table_bytes(hot.numel(), 0.8, 8, 8)
        keep.append(torch.empty(nbytes, dtype=torch.uint8).cuda())
        hnd = ctypes.c_void_p()
        cabi.check(lib.shmt_hashmap_create(ctypes.byref(hnd), hot.data_ptr(), torch.arange(hot.numel()).cuda().data_ptr(),
                                           hot.numel(), 8, 8, 0.8, keep[0].data_ptr(), nbytes, stream))
    seeds0 = torch.randperm(n, generator=torch.Generator().manual_seed(S))[:S].cuda()

    def buffers(s_max, k):
        n_max = s_max + s_max * k
        return dict(sp=torch.full((s_max + 1,), -1, dtype=torch.int64).cuda(),
                    si=torch.empty(s_max * k, dtype=torch.int32).cuda(),
                    plan=torch.empty(lib.shmt_sample_plan_bytes(s_max), dtype=torch.uint8).cuda(),
                    total=torch.empty(n_max, dtype=torch.int64).cuda(), unique=torch.empty(n_max, dtype=torch.int64).cuda(),
                    labels=torch.empty(n_max, dtype=torch.int64).cuda(),
                    scratch=torch.empty(lib.shmt_relabel_scratch_bytes(n_max), dtype=torch.uint8).cuda(),
                    nnz=torch.full((1,), -1, dtype=torch.int64).cuda(), count=torch.full((1,), -1, dtype=torch.int64).cuda(),
                    count_dev=torch.full((1,), -1, dtype=torch.int64).cuda())

    def graph_args():
        return (indptr.data_ptr(), 8, indices.data_ptr(), 4, gp.data_ptr() if cached else None,
                gi.data_ptr() if cached else None, hnd)

    # chained: nothing is read back until every hop is queued
    chained, seeds, s_max, s_len = [], seeds0, S, None
    for hop, k in enumerate(picks):
        b = buffers(s_max, k)
        cabi.check(lib.shmt_sample_hop_chained(*graph_args(), seeds.data_ptr(), 8, s_max, s_len, k, replace, 42, None, hop,
                                               b["sp"].data_ptr(), b["si"].data_ptr(), b["plan"].data_ptr(),
                                               b["plan"].numel(), 8, b["total"].data_ptr(), b["scratch"].data_ptr(),
                                               b["scratch"].numel(), b["unique"].data_ptr(), b["labels"].data_ptr(),
                                               b["nnz"].data_ptr(), b["count"].data_ptr(), b["count_dev"].data_ptr(),
                                               stream))
        chained.append(b)
        seeds, s_len, s_max = b["unique"], b["count_dev"].data_ptr(), s_max + s_max * k
    torch.cuda.synchronize()
    # hop by hop, the host reading each count
    seeds = seeds0
    for hop, k in enumerate(picks):
        s_now = seeds.numel()
        b = buffers(s_now, k)
        cabi.check(lib.shmt_sample_hop(*graph_args(), seeds.data_ptr(), 8, s_now, k, replace, 42, hop,
                                       b["sp"].data_ptr(), b["si"].data_ptr(), b["plan"].data_ptr(), b["plan"].numel(), 8,
                                       b["total"].data_ptr(), b["scratch"].data_ptr(), b["scratch"].numel(),
                                       b["unique"].data_ptr(), b["labels"].data_ptr(), b["nnz"].data_ptr(),
                                       b["count"].data_ptr(), stream))
        torch.cuda.synchronize()
        c = chained[hop]
        nnz, u = int(b["nnz"].item()), int(b["count"].item())
        assert (int(c["nnz"].item()), int(c["count"].item()), int(c["count_dev"].item())) == (nnz, u, u), hop
        assert torch.equal(c["sp"][:s_now + 1], b["sp"]) and torch.equal(c["si"][:nnz], b["si"][:nnz]), hop
        assert torch.equal(c["total"][:s_now + nnz], b["total"][:s_now + nnz]), hop
        assert torch.equal(c["unique"][:u], b["unique"][:u]), hop
        assert torch.equal(c["labels"][:s_now + nnz], b["labels"][:s_now + nnz]), hop
        seeds = b["unique"][:u].clone()
    if hnd is not None:
        lib.shmt_hashmap_destroy(hnd)


def _chains_equal(got, want):
    assert len(got) == len(want)
    for a, b in zip(got, want):
        assert len(a) == len(b)
        for x, y in zip(a, b):
            _same(x, y)


@pytest.mark.parametrize("seeded", [True, False])
@pytest.mark.parametrize("seed_dt", [torch.int64, torch.int32])
def test_batch_sampler_replays_a_recorded_batch(capi, seeded, seed_dt):
    """BatchSampler records the chained hops of one batch as a HIP graph and replays it per batch:
    same results as sample_blocks, for full, ragged and empty batches, with results of earlier
    calls still intact while later ones run, and lanes reused once results are dropped."""
    import gc
    indptr, indices = _graph(scale=14, idx_dt=torch.int32)
    indptr_h, indices_h = indptr.cpu().pin_memory(), indices.cpu().pin_memory()
    n = indptr.numel() - 1
    hot = torch.randperm(n, generator=torch.Generator().manual_seed(1))[: n // 3].cuda()
    gp, gi = capi.create_subcsr(indptr_h, indices_h, hot)
    h = capi.CUCOStaticHashmap(hot, torch.arange(hot.numel()).cuda(), 0.8)
    picks = [4, 6, 3]
    sampler = capi.BatchSampler(indptr_h, indices_h, gp, gi, h, 512, picks, False,
                                seed_bytes=torch.empty(0, dtype=seed_dt).element_size())
    g = torch.Generator().manual_seed(9)
    sizes = [512, 100, 512, 1, 0, 511, 512, 37, 512]
    batches = [torch.randperm(n, generator=g)[:s].to(seed_dt).cuda() for s in sizes]
    rng = [300 + b for b in range(len(batches))] if seeded else None
    want = capi.sample_blocks(indptr_h, indices_h, gp, gi, h, batches, picks, False, seeds_rng=rng)
    kept = []
    for repeat in range(3):
        got = sampler.sample(batches, seeds_rng=rng, max_in_flight=3)
        _chains_equal(got, want)
        kept.append(got)                       # earlier results stay alive ...
        for earlier in kept:
            _chains_equal(earlier, want)       # ... and intact
    lanes_held = sampler.lanes()
    assert lanes_held >= 3 * (len(sizes) - 1)  # every non-empty batch still held owns a lane
    del kept, got, earlier
    gc.collect()
    for repeat in range(3):                    # dropped results hand their lanes back: no new ones
        _chains_equal(sampler.sample(batches, seeds_rng=rng, max_in_flight=2), want)
        gc.collect()
    assert sampler.lanes() == lanes_held
    # the same through submit / collect, collected out of order
    tickets = [sampler.submit(b, rng[i] if seeded else None) for i, b in enumerate(batches[:4])]
    for i in (2, 0, 3, 1):
        _chains_equal([sampler.collect(tickets[i])], [want[i]])
    with pytest.raises(RuntimeError):
        sampler.collect(tickets[0])            # a ticket is good for one collect
    one = sampler.sample([batches[0]], seeds_rng=[300] if seeded else None)
    del sampler                                # results outlive the sampler object
    gc.collect()
    _chains_equal(one, [want[0]])


def test_batch_sampler_arguments(capi):
    indptr = torch.tensor([0, 3, 3, 4]).cuda()
    indices = torch.tensor([2, 1, 0, 2]).cuda()
    sampler = capi.BatchSampler(indptr, indices, None, None, None, 2, [5, 2], True)
    seeds = [torch.tensor([0, 2]).cuda(), torch.tensor([1]).cuda()]
    _chains_equal(sampler.sample(seeds), capi.sample_blocks(indptr, indices, None, None, None, seeds, [5, 2], True))
    assert sampler.sample([]) == []
    with pytest.raises(RuntimeError):          # more seeds than the recorded batch holds
        sampler.sample([torch.tensor([0, 1, 2]).cuda()])
    with pytest.raises(RuntimeError):          # other id width than the sampler was built for
        sampler.sample([torch.tensor([0], dtype=torch.int32).cuda()])
    with pytest.raises(RuntimeError):
        sampler.sample(seeds, seeds_rng=[1])
    with pytest.raises(RuntimeError):          # a hop without picks cannot be recorded
        capi.BatchSampler(indptr, indices, None, None, None, 2, [5, 0], False)
    with pytest.raises(RuntimeError):          # bounds beyond what a recorded batch may allocate
        capi.BatchSampler(indptr, indices, None, None, None, 4096, [25, 15, 10], False)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):              # called with a non-default current stream
        got = sampler.sample(seeds, seeds_rng=[4, 5])
    side.synchronize()
    _chains_equal(got, capi.sample_blocks(indptr, indices, None, None, None, seeds, [5, 2], True, seeds_rng=[4, 5]))


@pytest.mark.parametrize("S,k,replace", [(1, 3, 0), (256, 5, 0), (257, 5, 1), (3000, 20, 0), (50, 70, 0),
                                         (300000, 2, 0)])
def test_c_abi_sample_in_two_launches_matches_plan_then_pick(cabi, S, k, replace):
    """shmt_sample (bound-sized output, the pick kernel adds the tile offsets) against
    shmt_sample_plan + shmt_sample_pick with the total read by the host in between."""
    lib = cabi.load()
    indptr, indices = _graph(scale=13, ptr_dt=torch.int64, idx_dt=torch.int32)
    indptr, indices = indptr.cuda(), indices.cuda()
    n = indptr.numel() - 1
    stream = cabi.current_stream()
    seeds = torch.randint(0, n, (S,), generator=torch.Generator().manual_seed(S)).cuda()

    def buffers():
        return dict(sp=torch.full((S + 1,), -1, dtype=torch.int64).cuda(), si=torch.empty(S * k, dtype=torch.int32).cuda(),
                    plan=torch.empty(lib.shmt_sample_plan_bytes(S), dtype=torch.uint8).cuda(),
                    nnz=torch.full((1,), -1, dtype=torch.int64).cuda())
    a, b = buffers(), buffers()
    cabi.check(lib.shmt_sample(indptr.data_ptr(), 8, indices.data_ptr(), 4, None, None, None, seeds.data_ptr(), 8, S, k,
                               replace, 11, 3, a["sp"].data_ptr(), a["si"].data_ptr(), a["plan"].data_ptr(),
                               a["plan"].numel(), a["nnz"].data_ptr(), stream))
    cabi.check(lib.shmt_sample_plan(indptr.data_ptr(), 8, None, None, seeds.data_ptr(), 8, S, k, replace,
                                    b["sp"].data_ptr(), b["plan"].data_ptr(), b["plan"].numel(), b["nnz"].data_ptr(), stream))
    cabi.check(lib.shmt_sample_pick(indices.data_ptr(), None, 4, seeds.data_ptr(), 8, S, k, replace, b["sp"].data_ptr(), 8,
                                    b["plan"].data_ptr(), b["si"].data_ptr(), 11, 3, stream))
    torch.cuda.synchronize()
    nnz = int(b["nnz"].item())
    assert int(a["nnz"].item()) == nnz
    assert torch.equal(a["sp"], b["sp"]) and torch.equal(a["si"][:nnz], b["si"][:nnz])
    assert lib.shmt_sample(indptr.data_ptr(), 8, indices.data_ptr(), 4, None, None, None, seeds.data_ptr(), 8, 0, k,
                           replace, 11, 3, None, None, None, 0, None, stream) == -1


@pytest.mark.parametrize("cached", [False, True])
@pytest.mark.parametrize("sizes,picks", [([300, 300, 300], (4, 5)), ([1000, 1000, 1000, 1000, 1000], (6, 3, 2)),
                                         ([100, 1000, 200], (3, 3)), ([50] * 11, (8, 2)), ([40, 40], (70, 2))])
def test_c_abi_merged_jobs_equal_separate_chained_hops(cabi, cached, sizes, picks):
    """shmt_sample_hops_chained: the same hop of several batches in one call (launches merged when
    the jobs run the same kernels, issued one by one otherwise: unequal sizes, more than 8 jobs, a
    fan-out without merged form) gives what one shmt_sample_hop_chained call per batch gives."""
    lib = cabi.load()
    indptr, indices = _graph(scale=13, ptr_dt=torch.int64, idx_dt=torch.int32)
    indptr, indices = indptr.cuda(), indices.cuda()
    n = indptr.numel() - 1
    stream = cabi.current_stream()
    gp = gi = hnd = None
    keep = []
    if cached:
        hot = torch.randperm(n, generator=torch.Generator().manual_seed(2))[: n // 2].cuda()
        deg = indptr[hot + 1] - indptr[hot]
        gp = torch.cat([torch.zeros(1, dtype=torch.int64).cuda(), torch.cumsum(deg, 0)])
        gi = torch.cat([indices[indptr[v]:indptr[v + 1]] for v in hot.tolist()])
        nbytes = lib.shmt_hashmap_table_bytes(hot.numel(), 0.8, 8, 8)
        keep.append(torch.empty(nbytes, dtype=torch.uint8).cuda())
        hnd = ctypes.c_void_p()
        cabi.check(lib.shmt_hashmap_create(ctypes.byref(hnd), hot.data_ptr(), torch.arange(hot.numel()).cuda().data_ptr(),
                                           hot.numel(), 8, 8, 0.8, keep[0].data_ptr(), nbytes, stream))
    g = torch.Generator().manual_seed(len(sizes))
    seed_sets = [torch.randperm(n, generator=g)[:s].cuda() for s in sizes]

    def buffers(s_max, k):
        n_max = s_max + s_max * k
        return dict(s_max=s_max, k=k, sp=torch.full((s_max + 1,), -1, dtype=torch.int64).cuda(),
                    si=torch.empty(s_max * k, dtype=torch.int32).cuda(),
                    plan=torch.empty(lib.shmt_sample_plan_bytes(s_max), dtype=torch.uint8).cuda(),
                    total=torch.empty(n_max, dtype=torch.int64).cuda(), unique=torch.empty(n_max, dtype=torch.int64).cuda(),
                    labels=torch.empty(n_max, dtype=torch.int64).cuda(),
                    scratch=torch.empty(lib.shmt_relabel_scratch_bytes(n_max), dtype=torch.uint8).cuda(),
                    nnz=torch.full((1,), -1, dtype=torch.int64).cuda(), count=torch.full((1,), -1, dtype=torch.int64).cuda(),
                    count_dev=torch.full((1,), -1, dtype=torch.int64).cuda())

    def job(b, seeds_ptr, s_len, hop, rng):
        return cabi.HopJob(indptr.data_ptr(), 8, indices.data_ptr(), 4, gp.data_ptr() if cached else None,
                           gi.data_ptr() if cached else None, hnd, seeds_ptr, 8, b["s_max"], s_len, b["k"], 0, rng,
                           None, hop, b["sp"].data_ptr(), b["si"].data_ptr(), b["plan"].data_ptr(), b["plan"].numel(), 8,
                           b["total"].data_ptr(), b["scratch"].data_ptr(), b["scratch"].numel(), b["unique"].data_ptr(),
                           b["labels"].data_ptr(), b["nnz"].data_ptr(), b["count"].data_ptr(), b["count_dev"].data_ptr())

    def run(merged):
        chains = [[] for _ in sizes]
        src = [(s.data_ptr(), None, s.numel()) for s in seed_sets]
        for hop, k in enumerate(picks):
            jobs = []
            for j, (ptr, s_len, s_max) in enumerate(src):
                b = buffers(s_max, k)
                chains[j].append(b)
                jobs.append(job(b, ptr, s_len, hop, 90 + j))
                src[j] = (b["unique"].data_ptr(), b["count_dev"].data_ptr(), s_max + s_max * k)
            if merged:
                cabi.check(lib.shmt_sample_hops_chained((cabi.HopJob * len(jobs))(*jobs), len(jobs), stream))
            else:
                for one in jobs:
                    cabi.check(lib.shmt_sample_hops_chained(ctypes.byref(one), 1, stream))
        torch.cuda.synchronize()
        return chains

    got, want = run(True), run(False)
    for j in range(len(sizes)):
        s_now = sizes[j]
        for a, b in zip(got[j], want[j]):
            nnz, u = int(b["nnz"].item()), int(b["count"].item())
            assert (int(a["nnz"].item()), int(a["count"].item()), int(a["count_dev"].item())) == (nnz, u, u)
            assert torch.equal(a["sp"][:s_now + 1], b["sp"][:s_now + 1]) and torch.equal(a["si"][:nnz], b["si"][:nnz])
            assert torch.equal(a["unique"][:u], b["unique"][:u])
            assert torch.equal(a["labels"][:s_now + nnz], b["labels"][:s_now + nnz])
            s_now = u
    assert lib.shmt_sample_hops_chained(None, 0, stream) == 0 and lib.shmt_sample_hops_chained(None, 2, stream) == -1
    if hnd is not None:
        lib.shmt_hashmap_destroy(hnd)


@pytest.mark.parametrize("picks", [[10, 10, 30], [5, 0, 3], [40, 40], [3, 3, 3, 70]])
@pytest.mark.parametrize("in_flight", [1, 4])
def test_sample_blocks_with_hops_too_large_to_chain(capi, picks, in_flight):
    """Fan-outs whose bounds outgrow what a chained hop may allocate (the sizes are then read before
    that hop), a hop without picks in the middle, and a fan-out above 64 at the end: same results
    as one sample_hop call per hop and batch."""
    indptr, indices = _graph(scale=14)
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(17)
    sizes = [1000, 1000, 999, 1, 1000, 0, 1000]
    batches = [torch.randperm(n, generator=g)[:s].cuda() for s in sizes]
    rng = [7 + b for b in range(len(batches))]
    got = capi.sample_blocks(indptr, indices, None, None, None, batches, picks, False, seeds_rng=rng,
                             max_in_flight=in_flight)
    for b, seeds in enumerate(batches):
        assert len(got[b]) == len(picks)
        for hop, k in enumerate(picks):
            want = capi.sample_hop(indptr, indices, None, None, None, seeds, k, False, seed=rng[b], stream_id=hop)
            _same(got[b][hop], want)
            seeds = want[2]
