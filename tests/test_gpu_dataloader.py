"""GPUSamplingDataloader (python/shmtensor/sampling.py:30-237): hop order, relabel
argument order, returned triple, cache creation and presampling, checked
against the CPU oracle pipeline on a small graph; pin_memory behaviour."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def graph():
    rng = np.random.default_rng(3)
    n = 3000
    deg = rng.integers(0, 40, size=n)
    deg[:20] = 600
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    indices = rng.integers(0, n, size=int(indptr[-1])).astype(np.int64)
    return n, indptr, indices


def _loader(graph, **kw):
    import shmtensor
    n, indptr, indices = graph
    args = dict(batchsize=256, num_picks=[10, 5], shuffle=False)
    args.update(kw)
    return shmtensor.GPUSamplingDataloader(torch.from_numpy(indptr.copy()), torch.from_numpy(indices.copy()),
                                           torch.arange(0, 1000), **args)


def test_batches_follow_the_reference_pipeline(capi, oracle, graph):
    n, indptr, indices = graph
    dl = _loader(graph, rng_seed=11)
    assert len(dl) == 4 and dl.indptr.is_pinned() and dl.indices.is_pinned()
    seen = 0
    for b, (input_nodes, output_nodes, blocks) in enumerate(dl):
        seeds = np.arange(b * 256, min((b + 1) * 256, 1000))
        assert output_nodes.tolist() == seeds.tolist() and len(blocks) == 2
        ref_blocks = []
        cur = seeds
        for hop, k in enumerate(reversed([10, 5])):                  # last fanout first (sampling.py:128)
            # batch b draws from seed rng_seed + b, hop h from stream h
            sp, si = oracle.sample(indptr, indices, cur, k, False, seed=11 + b, stream=hop, algo="floyd")
            uniq, (_, rel) = oracle.relabel([cur, si])
            ref_blocks.insert(0, (sp, rel, uniq.size, cur.size))
            cur = uniq
        assert input_nodes.cpu().numpy().tolist() == cur.tolist()
        for blk, (sp, rel, nsrc, ndst) in zip(blocks, ref_blocks):
            assert blk.num_src == nsrc and blk.num_dst == ndst
            assert np.array_equal(blk.indptr.cpu().numpy(), sp) and np.array_equal(blk.indices.cpu().numpy(), rel)
        # destination nodes are a prefix of the source nodes of every block
        assert blocks[1].num_src == blocks[0].num_dst
        seen += 1
    assert seen == 4
    with pytest.raises(StopIteration):
        next(dl)


def test_cache_does_not_change_results(capi, graph):
    n, indptr, indices = graph
    plain = _loader(graph, rng_seed=3)
    cached = _loader(graph, rng_seed=3)
    sampling_hot, feature_hot = cached.presampling()
    assert sampling_hot.shape == (n,) and sampling_hot[:1000].min() >= 1 and feature_hot.sum() >= sampling_hot.sum()
    full = indptr.nbytes + indices.nbytes
    cached.create_cache(full // 3, sampling_hot)
    assert cached.has_cache and cached.gpu_indptr.is_cuda
    # the byte model of sampling.py:170-174: deg * 8 + 8 + 10 per cached node
    deg = np.diff(indptr)
    order = torch.sort(sampling_hot, descending=True)[1].numpy()    # the loader's own tie order
    cost = np.cumsum(deg[order] * 8 + 8 + 10.0)
    assert cached.gpu_indptr.numel() - 1 == np.searchsorted(cost, full // 3)
    cached_bytes = cached.gpu_indices.numel() * 8 + (cached.gpu_indptr.numel() - 1) * 18
    assert cached_bytes <= full // 3
    cached_gpu_indptr = cached.gpu_indptr
    for (a_in, a_out, a_blocks), (b_in, b_out, b_blocks) in zip(plain, cached):
        assert torch.equal(a_in, b_in) and torch.equal(a_out, b_out)
        for x, y in zip(a_blocks, b_blocks):
            assert torch.equal(x.indptr, y.indptr) and torch.equal(x.indices, y.indices)
    cached.clear_cache()
    assert not cached.has_cache and cached.hashmap is None
    split = _loader(graph, indptr_on_device=True, rng_seed=3)                   # offsets in HBM, adjacency pinned + cached
    assert split.indptr.is_cuda and split.indices.is_pinned()
    split.create_cache(full // 3, sampling_hot)
    assert split.has_cache and torch.equal(split.gpu_indptr, cached_gpu_indptr)
    # (a fresh plain loader: `plain` has an epoch behind it, and every epoch draws anew)
    for (a_in, _, a_blocks), (b_in, _, b_blocks) in zip(_loader(graph, rng_seed=3), split):
        assert torch.equal(a_in, b_in)
        for x, y in zip(a_blocks, b_blocks):
            assert torch.equal(x.indptr, y.indptr) and torch.equal(x.indices, y.indices)
    big = _loader(graph)
    big.create_cache(10 * full, sampling_hot)                       # everything fits: CSR moves to the GPU
    assert not big.has_cache and big.indptr.is_cuda and big.indices.is_cuda
    next(iter(big))


def test_shuffle_drop_last_and_rng_seed(capi, graph):
    dl = _loader(graph, shuffle=True, drop_last=True, batchsize=300, rng_seed=5)
    assert len(dl) == 3
    first = [out.clone() for _, out, _ in dl]
    order = torch.cat(first).tolist()
    assert len(set(order)) == 900 and order != sorted(order)                # a permutation, and not the identity
    assert all(o.numel() == 300 for o in first)
    # the 20 hub nodes (degree 600, ids 0..19) are seeds of the first batch: what they draw depends on
    # the RNG seed, on the hop (stream) and on the batch number, and repeats for a repeated seed
    def first_hop_of_first_batch(loader, epoch=0):
        it = iter(loader)
        for _ in range(epoch):
            for _ in it:
                pass
            it = iter(loader)
        _, _, blocks = next(it)
        return blocks[-1].indices[: int(blocks[-1].indptr[20])].clone()  # the seed layer's block: hubs 0..19
    a1 = first_hop_of_first_batch(_loader(graph, rng_seed=1))
    a2 = first_hop_of_first_batch(_loader(graph, rng_seed=1))
    b1 = first_hop_of_first_batch(_loader(graph, rng_seed=2))
    assert torch.equal(a1, a2) and not torch.equal(a1, b1)
    assert not torch.equal(a1, first_hop_of_first_batch(_loader(graph, rng_seed=1), epoch=1))   # second epoch
    torch.manual_seed(123)
    d1 = first_hop_of_first_batch(_loader(graph))                        # rng_seed=None: torch's global seed
    torch.manual_seed(123)
    d2 = first_hop_of_first_batch(_loader(graph))
    torch.manual_seed(124)
    d3 = first_hop_of_first_batch(_loader(graph))
    assert torch.equal(d1, d2) and not torch.equal(d1, d3)
    dl.update_params(seeds=torch.arange(100), batchsize=50)
    assert len(dl) == 2


def test_pin_memory_makes_a_plain_tensor_fetchable(capi):
    """capi.pin_memory(t) on an ordinary CPU tensor (example/test_cache_fetch.py:25-31):
    afterwards kernels can read it, the Python object is the same and its values are kept."""
    data = torch.arange(5000, dtype=torch.float32).reshape(1000, 5)
    keep = data
    expect = data.clone()
    capi.pin_memory(data)
    assert data is keep and torch.equal(data, expect)
    idx = torch.tensor([0, 999, 17]).cuda()
    assert torch.equal(capi.uva_fetch(data, idx).cpu(), expect[[0, 999, 17]])
    upd = torch.full((3, 5), -1.0).cuda()
    capi.uva_set(data, idx, upd)
    torch.cuda.synchronize()
    assert torch.equal(data[[0, 999, 17]], upd.cpu())               # GPU writes land in the same tensor
    capi.unpin_memory(data)
    capi.pin_memory(torch.zeros(0))                                  # empty tensors are a no-op


def _collect(dl):
    return [(i.clone(), o.clone(), [(b.indptr.clone(), b.indices.clone(), b.num_src, b.num_dst) for b in blocks])
            for i, o, blocks in dl]


def _same_epoch(a, b):
    assert len(a) == len(b)
    for (ai, ao, ab), (bi, bo, bb) in zip(a, b):
        assert torch.equal(ai, bi) and torch.equal(ao, bo) and len(ab) == len(bb)
        for (p, x, s, d), (q, y, t, e) in zip(ab, bb):
            assert torch.equal(p, q) and torch.equal(x, y) and (s, d) == (t, e)


@pytest.mark.parametrize("rng_seed", [None, 17])
def test_prefetch_and_background_give_the_same_batches(capi, graph, rng_seed):
    """Sampling several batches at once, or ahead on a background thread, changes
    neither the batches nor their order."""
    base_loader = _loader(graph, batchsize=100, num_picks=[6, 4, 3], rng_seed=rng_seed)
    base = _collect(base_loader)
    base2 = _collect(base_loader)                  # a second epoch draws new samples (the batch count goes on)
    assert len(base) == 10 and len(base2) == 10
    assert any(not torch.equal(a[2][-1][1], b[2][-1][1]) for a, b in zip(base, base2))
    for kw in (dict(prefetch=3), dict(prefetch=4, background=True), dict(prefetch=1, background=True),
               dict(prefetch=16), dict(indptr_on_device=True), dict(indptr_on_device=True, prefetch=2)):
        dl = _loader(graph, batchsize=100, num_picks=[6, 4, 3], rng_seed=rng_seed, **kw)
        _same_epoch(_collect(dl), base)
        _same_epoch(_collect(dl), base2)           # and so does a second epoch over the same loader
        assert dl._producer is None


@pytest.mark.parametrize("cached_rows", [True, False])
def test_features_option_adds_the_rows_of_the_input_nodes(capi, graph, cached_rows):
    """features=(table, cache rows, map): same batches, plus the feature rows of
    the input nodes exactly as a separate cache_fetch / uva_fetch returns them."""
    n = graph[0]
    gen = torch.Generator().manual_seed(8)
    table = torch.randn(n, 20, generator=gen).pin_memory()
    hot = torch.randperm(n, generator=gen)[: n // 3]
    rows = (table[hot] - 2.0).cuda()               # a hit is told from a miss by its content
    rows_map = capi.CUCOStaticHashmap(hot.cuda(), torch.arange(hot.numel()).cuda(), 0.8)
    feats = (table, rows, rows_map) if cached_rows else (table, None, None)
    base = _collect(_loader(graph, batchsize=100, num_picks=[6, 4, 3], rng_seed=5))
    for kw in (dict(), dict(prefetch=3), dict(prefetch=2, background=True)):
        dl = _loader(graph, batchsize=100, num_picks=[6, 4, 3], rng_seed=5, features=feats, **kw)
        got = [(i.clone(), o.clone(), [(b.indptr.clone(), b.indices.clone(), b.num_src, b.num_dst) for b in blocks], x)
               for i, o, blocks, x in dl]
        _same_epoch([g[:3] for g in got], base)
        for input_nodes, _, _, x in got:
            want = capi.cache_fetch(table, rows, input_nodes, rows_map) if cached_rows else \
                capi.uva_fetch(table, input_nodes)
            assert torch.equal(x, want)
        assert dl._feature_rows == max(g[0].numel() for g in got)
        dl.close()


def test_background_producer_stops_early_and_reports_errors(capi, graph):
    dl = _loader(graph, batchsize=50, prefetch=2, background=True)
    it = iter(dl)
    first = next(it)
    dl.close()                                     # mid-epoch: thread ends, prefetched batches dropped
    assert dl._producer is None and not dl._ready
    again = next(iter(dl))
    assert torch.equal(first[1], again[1])         # the epoch starts over: same seeds (a new draw around them)
    assert torch.equal(first[0][:50], again[0][:50]) and again[2][-1].num_dst == 50
    dl.close()
    bad = _loader(graph, batchsize=50, prefetch=2, background=True)
    bad.num_picks = [-1]                           # rejected by the operator on the producer thread
    with pytest.raises(RuntimeError):
        next(iter(bad))
    assert bad._producer is None


def test_end_to_end_batch_full_size(capi):
    """The end-to-end configuration at full size: R-MAT scale 24 (16.8 M nodes, 521 M edges), top 20 % of the
    adjacency cached, features 16,777,216 x 256 f32 (17.2 GB) pinned with the top-degree 25 % cached, batches of
    4,096 seeds with fanouts [25, 15, 10] through the dataloader, then the features of the input nodes.
    Checked by properties: block shapes chain, destination nodes are a prefix of source nodes, every block
    edge is an edge of the graph, fetched features equal index_select. Skipped when the features cannot be pinned."""
    import shmtensor
    from shmtensor_amd.synthetic import rmat_csr
    indptr_d, indices_d = rmat_csr(24, 16, seed=3)
    n, dim = indptr_d.numel() - 1, 256
    try:
        feats = torch.empty((n, dim), dtype=torch.float32, pin_memory=True)
    except RuntimeError as exc:
        pytest.skip("cannot pin 17.2 GB here: %s" % str(exc)[:80])
    g = torch.Generator(device="cuda").manual_seed(3)
    for lo in range(0, n, 2_000_000):
        hi = min(n, lo + 2_000_000)
        feats[lo:hi].copy_(torch.randn((hi - lo, dim), device="cuda", generator=g))
    torch.cuda.synchronize()
    deg = indptr_d[1:] - indptr_d[:-1]
    by_degree = torch.sort(deg, descending=True, stable=True).indices
    hot_feat = by_degree[: n // 4].contiguous()
    feat_cache = capi.uva_fetch(feats, hot_feat)
    feat_map = capi.CUCOStaticHashmap(hot_feat, torch.arange(hot_feat.numel(), device="cuda"), 0.8)
    seeds = torch.randperm(n, generator=torch.Generator().manual_seed(55))[: 3 * 4096]
    dl = shmtensor.GPUSamplingDataloader(indptr_d.cpu(), indices_d.cpu(), seeds, 4096, [25, 15, 10], shuffle=False,
                                         rng_seed=7, prefetch=3)
    hot_adj = by_degree[: n // 5].contiguous()
    dl.gpu_indptr, dl.gpu_indices = capi.create_subcsr(dl.indptr, dl.indices, hot_adj)
    dl.hashmap = capi.CUCOStaticHashmap(hot_adj, torch.arange(hot_adj.numel(), device="cuda"), 0.8)
    dl.has_cache = True
    batches = 0
    for input_nodes, output_nodes, blocks in dl:
        assert output_nodes.numel() == 4096 and len(blocks) == 3
        assert blocks[-1].num_dst == 4096 and blocks[0].num_src == input_nodes.numel()
        assert blocks[0].num_dst == blocks[1].num_src and blocks[1].num_dst == blocks[2].num_src
        assert torch.equal(input_nodes[:4096], output_nodes)                 # seeds stay first through every hop
        # the innermost block (fanout 25 on the widest frontier): every edge (dst -> src) is an edge of the graph
        blk = blocks[0]
        counts = blk.indptr[1:] - blk.indptr[:-1]
        dst = input_nodes[: blk.num_dst]
        assert torch.equal(counts, torch.clamp(deg[dst], max=25))
        owner = torch.repeat_interleave(dst, counts)
        nbr = input_nodes[blk.indices]
        first = indptr_d[owner]
        # neighbours are sorted within a row: locate each sampled one by bisection inside its row
        lo, hi = first.clone(), indptr_d[owner + 1].clone()
        for _ in range(32):
            mid = (lo + hi) // 2
            go_right = (indices_d[mid.clamp(max=indices_d.numel() - 1)].long() < nbr) & (lo < hi)
            lo = torch.where(go_right, mid + 1, lo)
            hi = torch.where(go_right, hi, mid)
        assert bool((indices_d[lo.clamp(max=indices_d.numel() - 1)].long() == nbr).all())
        x = capi.cache_fetch(feats, feat_cache, input_nodes, feat_map)
        assert torch.equal(x.cpu(), torch.index_select(feats, 0, input_nodes.cpu()))
        batches += 1
    assert batches == 3
