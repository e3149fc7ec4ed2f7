"""Randomised parity: shapes, dtypes, map layouts, cache fractions, fanouts, batch counts and pipeline depths
drawn from a seeded generator, every case checked bit for bit against numpy, the CPU oracle or the separate
operators. The fixed cases of the other files pin known edges; these catch what nobody thought of listing."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _keyset(rng, kind, n, universe):
    if kind == "range":
        lo = int(rng.integers(0, universe - n + 1))
        return np.arange(lo, lo + n)
    if kind == "rank":
        return np.sort(rng.choice(universe, size=n, replace=False))
    return rng.choice(universe, size=n, replace=False)


@pytest.mark.parametrize("seed", [11, 12])
def test_fetch_and_set_on_random_shapes(capi, cabi, seed):
    lib = cabi.load()
    rng = np.random.default_rng(seed)
    for case in range(60):
        rows = int(rng.integers(1000, 200000))
        width = int(rng.choice([1, 2, 3, 4, 8, 16, 24, 32, 64, 100, 128, 256]))
        dt = rng.choice([np.float32, np.float16, np.int64, np.uint8])
        ncache, Q = int(rng.integers(1, rows)), int(rng.integers(1, 300000))
        kind, layout = str(rng.choice(["range", "rank", "scatter"])), str(rng.choice(["auto", "buckets"]))
        idx_dt = rng.choice([np.int32, np.int64])
        print("case", case, rows, width, np.dtype(dt).name, ncache, Q, kind, layout, np.dtype(idx_dt).name, flush=True)
        host = torch.from_numpy(rng.integers(0, 200, size=(rows, width)).astype(dt)).pin_memory()
        keys = _keyset(rng, kind, ncache, rows)
        slots = np.arange(ncache) if kind != "scatter" else rng.permutation(ncache)
        gcache = torch.empty((ncache, width), dtype=host.dtype, device="cuda")
        gcache[torch.from_numpy(slots).cuda()] = torch.from_numpy((host.numpy()[keys] + 1).astype(dt)).cuda()
        m = capi.CUCOStaticHashmap(torch.from_numpy(keys).cuda(), torch.from_numpy(slots).cuda(), 0.8, layout=layout)
        q = (rng.zipf(1.3, size=Q) % rows if rng.random() < 0.5 else rng.integers(0, rows, size=Q)).astype(idx_dt)
        qg = torch.from_numpy(q).cuda()
        slot_of = np.full(rows, -1, dtype=np.int64)
        slot_of[keys] = slots
        s = slot_of[q]
        want = np.where((s >= 0)[:, None], gcache.cpu().numpy()[np.maximum(s, 0)], host.numpy()[q])
        assert np.array_equal(capi.cache_fetch(host, gcache, qg, m).cpu().numpy(), want)
        row_bytes = width * np.dtype(dt).itemsize
        if row_bytes % 16 == 0:                       # the same fetch in two launches, through the C ABI
            kd, vd = torch.from_numpy(keys).cuda(), torch.from_numpy(slots).cuda()
            nbytes = lib.shmt_hashmap_table_bytes(ncache, 0.8, 8, 8)
            table = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
            hnd, st = ctypes.c_void_p(), cabi.current_stream()
            cabi.check(lib.shmt_hashmap_create(ctypes.byref(hnd), kd.data_ptr(), vd.data_ptr(), ncache, 8, 8, 0.8,
                                               table.data_ptr(), nbytes, st))
            out = torch.empty((Q, width), dtype=host.dtype, device="cuda")
            bits = torch.empty((Q + 31) // 32, dtype=torch.int32, device="cuda")
            hostdev = ctypes.c_void_p()
            cabi.check(lib.shmt_host_devptr(host.data_ptr(), ctypes.byref(hostdev)))
            cabi.check(lib.shmt_fetch_cached_part(hostdev, gcache.data_ptr(), qg.data_ptr(), q.itemsize, hnd, None, 0,
                                                  out.data_ptr(), Q, None, row_bytes, bits.data_ptr(), st))
            cabi.check(lib.shmt_fetch_missed_part(hostdev, qg.data_ptr(), q.itemsize, bits.data_ptr(), out.data_ptr(),
                                                  Q, None, row_bytes, int(rng.choice([0, 1, 7, 48])), st))
            assert np.array_equal(out.cpu().numpy(), want)
            lib.shmt_hashmap_destroy(hnd)
        uq = np.unique(q)[: max(1, Q // 2)]               # set: every id once, so the result is defined
        upd = torch.from_numpy(rng.integers(0, 200, size=(uq.size, width)).astype(dt)).cuda()
        h0, c0 = host.numpy().copy(), gcache.cpu().numpy().copy()
        capi.cache_set(host, gcache, torch.from_numpy(uq.astype(idx_dt)).cuda(), upd, m)
        torch.cuda.synchronize()
        su, u = slot_of[uq], upd.cpu().numpy()
        c0[su[su >= 0]] = u[su >= 0]
        h0[uq[su < 0]] = u[su < 0]
        assert np.array_equal(gcache.cpu().numpy(), c0) and np.array_equal(host.numpy(), h0)


@pytest.mark.parametrize("seed", [21])
def test_scans_and_relabel_on_random_sizes(capi, cabi, oracle, seed):
    lib = cabi.load()
    rng = np.random.default_rng(seed)
    for case in range(40):
        n, off = int(rng.integers(1, 6_000_000)), int(rng.integers(0, 4))
        print("case", case, "scan", n, off, flush=True)
        a = rng.integers(0, 2**40, size=n + off)
        g = torch.from_numpy(a).cuda()[off:]              # not 16-byte aligned for off = 1, 3
        tmpb = lib.shmt_scan_tmp_bytes(n)
        tmp = torch.zeros(max(tmpb, 8), dtype=torch.uint8, device="cuda")
        cabi.check(lib.shmt_exclusive_scan_kept(g.data_ptr(), n, 8, tmp.data_ptr(), tmpb, cabi.current_stream()))
        assert np.array_equal(g.cpu().numpy(), oracle.exclusive_scan(a[off:]))
        assert int(tmp.sum()) == 0                        # left clean for the next scan
        b = rng.integers(0, 1000, size=n).astype(np.int32)
        gb = torch.from_numpy(b).cuda()
        capi.thrust_scan(gb)
        assert np.array_equal(gb.cpu().numpy(), oracle.inclusive_scan_i32(b))
        n1, n2 = int(rng.integers(1, 300000)), int(rng.integers(0, 600000))
        universe = int(rng.choice([50, 5000, 10**6, 2**33]))
        print("case", case, "relabel", n1, n2, universe, flush=True)
        t1, t2 = rng.integers(0, universe, size=n1), rng.integers(0, universe, size=n2)
        if universe < 2**31 and rng.random() < 0.5:
            t2 = t2.astype(np.int32)
        u, (l1, l2) = capi.tensor_relabel([torch.from_numpy(t1).cuda(), torch.from_numpy(t2).cuda()])
        ou, (o1, o2) = oracle.relabel([t1, t2.astype(np.int64)], algo="sweep")
        assert np.array_equal(u.cpu().numpy(), ou)
        assert np.array_equal(l1.cpu().numpy(), o1) and np.array_equal(l2.cpu().numpy(), o2)


@pytest.mark.parametrize("seed", [31, 32])
def test_sampling_on_random_graphs(capi, oracle, seed):
    """Cached sampling against the oracle's rule and the fused hop against sampling + relabel; degrees from 0 to
    five times the fanout's neighbourhood, so that every path of the duplicate resolution is met (rows shorter than
    the fanout, draws among the k largest positions, repeated draws, and both at once)."""
    rng = np.random.default_rng(seed)
    for case in range(40):
        n, maxdeg = int(rng.integers(100, 30000)), int(rng.choice([3, 30, 300, 3000]))
        k = int(rng.choice([1, 2, 5, 10, 15, 16, 17, 25, 31, 32, 33, 64, 70]))
        S, replace = int(rng.integers(1, 20000)), bool(rng.random() < 0.3)
        print("case", case, n, maxdeg, k, S, replace, flush=True)
        deg = rng.integers(0, maxdeg, size=n)
        deg[rng.integers(0, n, size=3)] = maxdeg * 5
        if rng.random() < 0.5:                            # many rows just above the fanout: large draws are common
            deg[rng.integers(0, n, size=n // 2)] = k + rng.integers(1, 4, size=n // 2)
        indptr = np.concatenate([np.zeros(1, dtype=np.int64), np.cumsum(deg)]).astype(np.int64)
        indices = rng.integers(0, n, size=int(indptr[-1])).astype(np.int32)
        ip, ix = torch.from_numpy(indptr).pin_memory(), torch.from_numpy(indices).pin_memory()
        hot = np.sort(rng.choice(n, size=n // 3, replace=False))
        gp, gi = capi.create_subcsr(ip, ix, torch.from_numpy(hot).cuda())
        m = capi.CUCOStaticHashmap(torch.from_numpy(hot).cuda(), torch.arange(hot.size, device="cuda"), 0.8)
        seeds = rng.integers(0, n, size=S)
        sg = torch.from_numpy(seeds).cuda()
        sp, si = capi.csr_cache_sampling(ip, ix, gp, gi, m, sg, k, replace, seed=99, stream_id=2)
        op, oi = oracle.sample(indptr, indices.astype(np.int64), seeds, k, replace, seed=99, stream=2, algo="floyd")
        assert np.array_equal(sp.cpu().numpy(), op) and np.array_equal(si.cpu().numpy().astype(np.int64), oi)
        sp2, si2, uq, rel = capi.sample_hop(ip, ix, gp, gi, m, sg, k, replace, seed=99, stream_id=2)
        assert torch.equal(sp2, sp) and torch.equal(si2, si)
        ou, (_, orel) = oracle.relabel([seeds, oi], algo="sweep")
        assert np.array_equal(uq.cpu().numpy(), ou) and np.array_equal(rel.cpu().numpy(), orel)


@pytest.mark.parametrize("seed", [41])
def test_pipelined_sampler_and_fetch_on_random_batches(capi, seed):
    """sample_blocks against the operators hop by hop, and sample_blocks_fetch (side streams, fetch in two launches,
    speculative row counts that fit, overflow or are switched off) against sample_blocks + cache_fetch."""
    rng = np.random.default_rng(seed)
    for case in range(60):
        n, maxdeg = int(rng.integers(200, 60000)), int(rng.choice([4, 40, 400]))
        D = int(rng.choice([4, 8, 32, 100, 128, 256]))
        fan = [int(x) for x in rng.choice([1, 2, 3, 5, 10, 15, 25], size=int(rng.integers(1, 4)))]
        S, B, depth = int(rng.integers(1, 3000)), int(rng.integers(1, 7)), int(rng.integers(1, 5))
        coo, dt = bool(rng.random() < 0.3), rng.choice([np.float32, np.float16])
        cached_adj, cached_feat, feat_dev = rng.random() < 0.8, rng.random() < 0.85, rng.random() < 0.15
        lim = str(rng.choice(["none", "zero", "small", "fit"]))
        print("case", case, n, maxdeg, D, fan, S, B, depth, coo, np.dtype(dt).name, cached_adj, cached_feat, feat_dev,
              lim, flush=True)
        deg = rng.integers(0, maxdeg, size=n)
        indptr = np.concatenate([np.zeros(1, dtype=np.int64), np.cumsum(deg)]).astype(np.int64)
        indices = rng.integers(0, n, size=int(indptr[-1])).astype(np.int32)
        ip, ix = torch.from_numpy(indptr).pin_memory(), torch.from_numpy(indices).pin_memory()
        gp = gi = m = None
        if cached_adj:
            hot = np.sort(rng.choice(n, size=max(1, n // 4), replace=False))
            gp, gi = capi.create_subcsr(ip, ix, torch.from_numpy(hot).cuda())
            m = capi.CUCOStaticHashmap(torch.from_numpy(hot).cuda(), torch.arange(hot.size, device="cuda"), 0.8)
        feats = torch.from_numpy(rng.integers(0, 100, size=(n, D)).astype(dt))
        feats = feats.cuda() if feat_dev else feats.pin_memory()
        fc = fm = None
        if cached_feat:
            hotf = rng.choice(n, size=max(1, n // 3), replace=False)
            if rng.random() < 0.5:
                hotf = np.sort(hotf)
            fc = (feats[torch.from_numpy(hotf).to(feats.device)].cuda() + 1).contiguous()   # told apart from host rows
            fm = capi.CUCOStaticHashmap(torch.from_numpy(hotf).cuda(), torch.arange(hotf.size, device="cuda"), 0.8,
                                        layout=str(rng.choice(["auto", "buckets"])))
        batches = [torch.from_numpy(rng.choice(n, size=min(S, n), replace=False)).cuda() for _ in range(B)]
        seeds_rng = [int(x) for x in rng.integers(0, 2**31, size=B)]
        ref = capi.sample_blocks(ip, ix, gp, gi, m, batches, fan, False, seeds_rng=seeds_rng, max_in_flight=depth,
                                 coo=coo)
        for b in range(B):
            seeds = batches[b]
            for h, k in enumerate(fan):
                if m is not None:
                    sp, si = capi.csr_cache_sampling(ip, ix, gp, gi, m, seeds, k, False, seed=seeds_rng[b], stream_id=h)
                else:
                    sp, si = capi.csr_sampling(ip, ix, seeds, k, False, seed=seeds_rng[b], stream_id=h)
                uq, (_, rel) = capi.tensor_relabel([seeds, si])
                r = ref[b][h]
                assert torch.equal(r[0], sp) and torch.equal(r[1], si) and torch.equal(r[2], uq) and torch.equal(r[3], rel)
                seeds = uq
        most = max(r[-1][2].numel() for r in ref)
        max_rows = {"none": None, "zero": 0, "small": 5, "fit": int(most * 1.25) + 1}[lim]
        got = capi.sample_blocks_fetch(ip, ix, gp, gi, m, batches, fan, False, feats, fc, fm, seeds_rng=seeds_rng,
                                       max_in_flight=depth, max_rows=max_rows, coo=coo)
        for b in range(B):
            hops, x = got[b]
            for h in range(len(fan)):
                for j in range(len(ref[b][h])):
                    assert torch.equal(hops[h][j], ref[b][h][j])
            inp = ref[b][-1][2]
            want = capi.cache_fetch(feats, fc, inp, fm) if fm is not None else capi.uva_fetch(feats, inp)
            assert x.shape == want.shape and torch.equal(x, want)
        del got, ref
