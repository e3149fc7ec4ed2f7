"""Neighbour sampling and the cached sub-CSR on the GPU: the reference's
known-answer cases (example/test_cache_sampling.py:23-126), the CPU oracle,
structural invariants, and chi-square tests of the uniform law."""
import numpy as np
import pytest
import torch
from scipy.stats import chi2 as chi2_dist

from conftest import load_golden

pytestmark = pytest.mark.gpu


def _kat_check(g, sp, si, replace):
    exp = g["replace_true" if replace else "replace_false"]
    assert sp.tolist() == exp["sub_indptr"]
    assert si.numel() == exp["sub_indptr"][-1]
    seg = lambda i: si[sp[i]:sp[i + 1]]
    if replace:
        for i, (lo, hi) in enumerate(exp["segment_ranges"]):
            assert bool(((seg(i) >= lo) & (seg(i) < hi)).all())
    else:
        for i, vals in exp["exact_segments"].items():
            assert seg(int(i)).tolist() == vals
        for i, (lo, hi) in exp["distinct_in_range"].items():
            s = seg(int(i))
            assert bool(((s >= lo) & (s < hi)).all()) and s.unique().numel() == g["num_picks"]


@pytest.mark.parametrize("replace", [True, False])
def test_csr_sampling_reference_kat(capi, replace):
    g = load_golden("csr_sampling_kat.json")
    indptr = torch.tensor(g["indptr"]).long().cuda()
    indices = torch.arange(g["num_indices"]).long().cuda()
    seeds = torch.tensor(g["seeds"]).int().cuda()
    sp, si = capi.csr_sampling(indptr, indices, seeds, g["num_picks"], replace)
    assert sp.dtype == torch.int64 and si.dtype == torch.int64 and sp.is_cuda and si.is_cuda
    _kat_check(g, sp, si, replace)
    again = capi.csr_sampling(indptr, indices, seeds, g["num_picks"], replace)
    assert torch.equal(again[1], si)          # fixed default seed: same call, same sample


def test_csr_cache_sampling_reference_kat(capi):
    g = load_golden("csr_sampling_kat.json")
    s = load_golden("subcsr_kat.json")
    indptr = torch.tensor(g["indptr"]).long().pin_memory()
    indices = torch.arange(g["num_indices"]).long().pin_memory()
    capi.pin_memory(indptr)
    capi.pin_memory(indices)
    cache_seeds = torch.tensor(g["cache_seeds"]).long().cuda()
    gp, gi = capi.create_subcsr(indptr, indices, cache_seeds)
    assert gp.tolist() == s["gpu_indptr"] and gi.tolist() == s["gpu_indices"]
    h = capi.CUCOStaticHashmap(cache_seeds, torch.arange(cache_seeds.numel()).cuda().long(), 0.8)
    seeds = torch.tensor(g["seeds"]).int().cuda()          # int32 seeds against int64 keys
    for replace in (True, False):
        sp, si = capi.csr_cache_sampling(indptr, indices, gp, gi, h, seeds, g["num_picks"], replace)
        _kat_check(g, sp, si, replace)
    capi.unpin_memory(indptr)
    capi.unpin_memory(indices)


def _random_csr(rng, n, max_deg, ptr_dt, idx_dt, hubs=()):
    deg = rng.integers(0, max_deg, size=n)
    deg[rng.integers(0, n, size=n // 10)] = 0
    for v, d in hubs:
        deg[v] = d
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(ptr_dt)
    indices = rng.integers(0, n, size=int(indptr[-1])).astype(idx_dt)
    return indptr, indices


@pytest.mark.parametrize("ptr_dt,idx_dt", [(np.int64, np.int64), (np.int32, np.int32), (np.int64, np.int32)])
@pytest.mark.parametrize("seed_dt", [np.int32, np.int64])
@pytest.mark.parametrize("k", [1, 5, 10, 15, 25, 64, 65, 200])
def test_sampling_matches_oracle_bit_exact(capi, oracle, ptr_dt, idx_dt, seed_dt, k):
    """Uncached and cached sampling against the oracle: sub_indptr and every
    deg <= k segment follow the reference rules; deg > k segments equal the
    oracle's restatement of the device selection rule (Floyd + Philox), which
    in turn is checked for uniformity in tests/test_oracle.py."""
    rng = np.random.default_rng(k * 131 + np.dtype(ptr_dt).itemsize + np.dtype(seed_dt).itemsize)
    n = 4000
    indptr, indices = _random_csr(rng, n, 40, ptr_dt, idx_dt, hubs=[(7, 5000), (8, k), (9, k + 1), (10, 300)])
    seeds = np.concatenate([[7, 8, 9, 10, 7], rng.integers(0, n, size=5001)]).astype(seed_dt)
    t = lambda a: torch.from_numpy(a)
    hp, hx = t(indptr).pin_memory(), t(indices).pin_memory()
    for replace in (False, True):
        esp, esi = oracle.sample(indptr, indices, seeds, k, replace, seed=7777, algo="floyd")
        sp, si = capi.csr_sampling(hp, hx, t(seeds).cuda(), k, replace)
        assert sp.dtype == t(indptr).dtype and si.dtype == t(indices).dtype
        assert np.array_equal(sp.cpu().numpy(), esp)
        assert np.array_equal(si.cpu().numpy(), esi)
        sp2, si2 = capi.csr_sampling(hp.cuda(), hx.cuda(), t(seeds).cuda(), k, replace)   # fully on the GPU
        assert torch.equal(sp2, sp) and torch.equal(si2, si)
    # cache the 30 % highest-degree rows; the result must not change
    order = np.argsort(-(indptr[1:] - indptr[:-1]), kind="stable")[: n * 3 // 10].astype(np.int64)
    gp, gi = capi.create_subcsr(hp, hx, t(order).cuda())
    egp, egi = oracle.create_subcsr(indptr, indices, order)
    assert np.array_equal(gp.cpu().numpy(), egp) and np.array_equal(gi.cpu().numpy(), egi)
    for key_dt in (torch.int32, torch.int64):
        h = capi.CUCOStaticHashmap(t(order).to(key_dt).cuda(), torch.arange(order.size, dtype=key_dt).cuda(), 0.8)
        sp3, si3 = capi.csr_cache_sampling(hp, hx, gp, gi, h, t(seeds).cuda(), k, False)
        esp, esi = oracle.sample(indptr, indices, seeds, k, False, seed=7777, algo="floyd")
        assert np.array_equal(sp3.cpu().numpy(), esp) and np.array_equal(si3.cpu().numpy(), esi)


def test_sampling_invariants_large_batch(capi, oracle):
    """S large enough for the multi-workgroup plan; every output is a true
    neighbour, no duplicates within a segment, exactly min(k, deg) per seed."""
    rng = np.random.default_rng(77)
    n, k = 200_000, 10
    indptr, indices_dup = _random_csr(rng, n, 60, np.int64, np.int32)
    # distinct neighbours per row so that "no duplicates" is meaningful
    indices = np.concatenate([rng.choice(n, size=d, replace=False) for d in np.diff(indptr[:2001])] +
                             [np.arange(indptr[2000], indptr[-1]) % n]).astype(np.int32)
    seeds = rng.permutation(n)[:150_000].astype(np.int64)
    hp, hx = torch.from_numpy(indptr).pin_memory(), torch.from_numpy(indices).pin_memory()
    sp, si = capi.csr_sampling(hp, hx, torch.from_numpy(seeds).cuda(), k, False, seed=123)
    deg = (indptr[1:] - indptr[:-1])[seeds]
    assert np.array_equal(np.diff(sp.cpu().numpy()), np.minimum(deg, k))
    esp, esi = oracle.sample(indptr, indices, seeds, k, False, seed=123, algo="floyd")
    assert np.array_equal(si.cpu().numpy(), esi)
    sp_n, si_n = sp.cpu().numpy(), si.cpu().numpy()
    for s in range(0, 150_000, 997):
        seg = si_n[sp_n[s]:sp_n[s + 1]]
        adj = indices[indptr[seeds[s]]:indptr[seeds[s] + 1]]
        assert np.isin(seg, adj).all()
        if seeds[s] < 2000:
            assert np.unique(seg).size == seg.size


@pytest.mark.parametrize("deg,k", [(6, 5), (12, 5), (100, 15), (1000, 25), (70, 65)])
def test_uniform_without_replacement_chi_square(capi, deg, k):
    """Per-edge selection frequency over many independent seeds: each of the deg
    neighbours must be chosen with probability k/deg (df = deg-1, level 1e-6)."""
    trials = 40_000
    indptr = torch.arange(0, (trials + 1) * deg, deg)
    indices = torch.arange(deg).repeat(trials).int()
    sp, si = capi.csr_sampling(indptr.cuda(), indices.cuda(), torch.arange(trials).cuda(), k, False, seed=2024)
    assert torch.equal(sp.cpu(), torch.arange(trials + 1) * k)
    picks = si.view(trials, k)
    assert bool((picks.sort(dim=1).values.diff(dim=1) > 0).all())        # distinct within every segment
    counts = torch.bincount(si.long(), minlength=deg).cpu().numpy()
    expected = trials * k / deg
    stat = ((counts - expected) ** 2 / expected).sum() / (1 - k / deg)
    assert stat < chi2_dist.ppf(1 - 1e-6, deg - 1), (stat, counts)
    # a different seed or stream id gives a different sample
    _, si2 = capi.csr_sampling(indptr.cuda(), indices.cuda(), torch.arange(trials).cuda(), k, False, seed=2025)
    _, si3 = capi.csr_sampling(indptr.cuda(), indices.cuda(), torch.arange(trials).cuda(), k, False, seed=2024,
                               stream_id=1)
    assert not torch.equal(si, si2) and not torch.equal(si, si3)


def test_uniform_with_replacement_chi_square(capi):
    deg, k, trials = 9, 4, 40_000
    indptr = torch.arange(0, (trials + 1) * deg, deg)
    indices = torch.arange(deg).repeat(trials)
    _, si = capi.csr_sampling(indptr.cuda(), indices.cuda(), torch.arange(trials).cuda(), k, True, seed=1)
    counts = torch.bincount(si, minlength=deg).cpu().numpy()
    expected = trials * k / deg
    assert ((counts - expected) ** 2 / expected).sum() < chi2_dist.ppf(1 - 1e-6, deg - 1)


def test_empty_and_degenerate(capi):
    indptr = torch.tensor([0, 0, 3]).cuda()
    indices = torch.tensor([5, 6, 7]).int().cuda()
    sp, si = capi.csr_sampling(indptr, indices, torch.zeros(0, dtype=torch.int64).cuda(), 5, False)
    assert sp.tolist() == [0] and si.numel() == 0 and si.dtype == torch.int32
    sp, si = capi.csr_sampling(indptr, indices, torch.tensor([0, 0]).cuda(), 5, False)
    assert sp.tolist() == [0, 0, 0] and si.numel() == 0
    sp, si = capi.csr_sampling(indptr, indices, torch.tensor([1, 1]).cuda(), 0, False)
    assert sp.tolist() == [0, 0, 0] and si.numel() == 0
    sp, si = capi.csr_sampling(indptr, indices, torch.tensor([1, 0, 1]).cuda(), 1 << 40, False)   # "take all"
    assert sp.tolist() == [0, 3, 3, 6] and si.tolist() == [5, 6, 7, 5, 6, 7]
    gp, gi = capi.create_subcsr(indptr, indices, torch.zeros(0, dtype=torch.int64).cuda())
    assert gp.tolist() == [0] and gi.numel() == 0


def test_rmat_three_hop_pipeline(capi, oracle):
    """Config-3 shape at reduced scale (R-MAT scale 16, edge factor 30): top 30 %
    of rows by degree cached, 1,024 seeds, fanouts [15, 10, 5] applied in the
    dataloader's order (python/shmtensor/sampling.py:128), relabel after each hop.
    Checked hop by hop against the oracle pipeline."""
    from shmtensor_amd.synthetic import rmat_csr
    indptr_d, indices_d = rmat_csr(16, 30, seed=1)
    n = indptr_d.numel() - 1
    indptr, indices = indptr_d.cpu().pin_memory(), indices_d.cpu().pin_memory()
    deg = indptr[1:] - indptr[:-1]
    hot = torch.sort(deg, descending=True, stable=True).indices[: n * 3 // 10].cuda()
    gp, gi = capi.create_subcsr(indptr, indices, hot)
    h = capi.CUCOStaticHashmap(hot, torch.arange(hot.numel()).cuda(), 0.8)
    ref_cache = (gp.cpu().numpy(), gi.cpu().numpy(), oracle.Hashmap(hot.cpu().numpy(), np.arange(hot.numel()), 0.8))
    g = torch.Generator().manual_seed(4)
    seeds = torch.randperm(n, generator=g)[:1024].cuda()
    ref_seeds = seeds.cpu().numpy()
    total_edges = 0
    for hop, k in enumerate(reversed([15, 10, 5])):
        sp, si = capi.csr_cache_sampling(indptr, indices, gp, gi, h, seeds, k, False, stream_id=hop)
        u, (ls, ln) = capi.tensor_relabel([seeds, si])
        esp, esi = oracle.sample(indptr.numpy(), indices.numpy(), ref_seeds, k, False, cache=ref_cache,
                                 seed=7777, stream=hop, algo="floyd")
        eu, (els, eln) = oracle.relabel([ref_seeds, esi])
        assert np.array_equal(sp.cpu().numpy(), esp) and np.array_equal(si.cpu().numpy(), esi)
        assert np.array_equal(u.cpu().numpy(), eu) and np.array_equal(ln.cpu().numpy(), eln)
        assert torch.equal(u[: seeds.numel()], seeds)
        total_edges += si.numel()
        seeds, ref_seeds = u, eu
    assert total_edges > 50_000


def test_config3_full_size_properties(capi):
    """Configuration 3 at full size (R-MAT scale 21, 116 M edges, top 30 % of rows cached, 1,024 seeds,
    fanouts [15, 10, 5] in the dataloader's order): properties that need no CPU pass over the graph.
    Counts are min(k, degree); every sampled id is a neighbour of its seed, without repeats; the cache is
    transparent; the fused hop equals the separate operators; relabel inverts and keeps the seeds first."""
    from shmtensor_amd.synthetic import rmat_csr
    indptr_d, indices_d = rmat_csr(21, 30, seed=1)
    n = indptr_d.numel() - 1
    indptr, indices = indptr_d.cpu().pin_memory(), indices_d.cpu().pin_memory()
    deg = indptr_d[1:] - indptr_d[:-1]
    hot = torch.sort(deg, descending=True, stable=True).indices[: n * 3 // 10].contiguous()
    gp, gi = capi.create_subcsr(indptr, indices, hot)
    h = capi.CUCOStaticHashmap(hot, torch.arange(hot.numel(), device="cuda"), 0.8)
    # every edge as one sorted key (rows ascending, neighbours sorted within a row)
    rows = torch.repeat_interleave(torch.arange(n, device="cuda"), deg)
    edge_keys = rows * n + indices_d.long()
    del rows
    seeds = torch.randperm(n, device="cuda", generator=torch.Generator(device="cuda").manual_seed(33))[:1024]
    for hop, k in enumerate([5, 10, 15]):
        sp, si = capi.csr_cache_sampling(indptr, indices, gp, gi, h, seeds, k, False, seed=7777, stream_id=hop)
        assert torch.equal(sp[1:] - sp[:-1], torch.clamp(deg[seeds], max=k))
        owner = torch.repeat_interleave(seeds, sp[1:] - sp[:-1])
        keys = owner * n + si.long()
        pos = torch.searchsorted(edge_keys, keys)
        assert bool((edge_keys[pos.clamp(max=edge_keys.numel() - 1)] == keys).all())      # real neighbours
        slot = torch.repeat_interleave(torch.arange(seeds.numel(), device="cuda"), sp[1:] - sp[:-1])
        assert torch.unique(slot * n + si.long()).numel() == si.numel()                    # no repeats in a row
        sp2, si2 = capi.csr_sampling(indptr, indices, seeds, k, False, seed=7777, stream_id=hop)
        assert torch.equal(sp, sp2) and torch.equal(si, si2)                               # cache is transparent
        u, (ls, ln) = capi.tensor_relabel([seeds, si])
        fsp, fsi, fu, fl = capi.sample_hop(indptr, indices, gp, gi, h, seeds, k, False, seed=7777, stream_id=hop)
        assert torch.equal(fsp, sp) and torch.equal(fsi, si) and torch.equal(fu, u) and torch.equal(fl, ln)
        assert torch.equal(u[: seeds.numel()], seeds) and torch.equal(u[ln], si.long())
        assert u.numel() == torch.unique(torch.cat([seeds, si.long()])).numel()
        seeds = u
    assert seeds.numel() > 100_000
