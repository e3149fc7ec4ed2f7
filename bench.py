#!/usr/bin/env python3
"""Benchmark of the GPU-cache hot path on one MI355X.

Headline ("step"): one cache_fetch call over one batch of benchmark configuration 4 —
100,000,000 x 128 fp16 feature table in pinned host memory, the 40,000,000
lowest ids cached in HBM, 1,048,576 int64 queries drawn from Zipf(1.1) over the
node rank. value = feature bytes delivered per second (Q * row_bytes / t), with
queries, cache and map resident in HBM when the timed region starts.

The same JSON line carries the roofline of the fetch kernel, the CPU baseline
(oracle gather on the host cores, bounded sample) and, under "extra", the
all-hit / all-miss fetch rates, the cache_set pass, the hashmap microbenchmark
(config 2), cached 3-hop sampling with relabel (config 3) beside its CPU
baseline, and the end-to-end mini-batch of config 5 (per stage and whole batch).

Benchmark configurations referred to by number in this file:
  1  small fetch: 200,000 x 128 f32 table in pinned host memory, 50,000 random ids cached,
     65,536 uniform queries (~25 % hits)
  2  static hashmap: 4,194,304 unique int64 keys in [0, 2^40) -> insertion index, load factor 0.5;
     16,777,216 queries, half members, half non-members
  3  cached sampling: R-MAT scale 21, edge factor 30 (a,b,c,d = .57,.19,.19,.05), symmetrised; int64
     indptr / int32 indices in pinned host memory, adjacency of the top 30 % of nodes by degree cached
     in HBM; batches of 1,024 seeds, fanouts [15,10,5], relabel after every hop
  4  large skewed fetch: the headline above, plus a cache_set pass over 262,144 cached rows
  5  end-to-end mini-batch: R-MAT scale 24, edge factor 16, top 20 % adjacency cached; 16,777,216 x 256
     f32 features in pinned host memory, top-degree 25 % cached; 4,096 seeds, fanouts [25,15,10],
     relabel, then fetch of all input nodes

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workloads fetch,hashmap,scan,harness,sampling,e2e]
"""
import argparse
import collections
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the config-4 fetch kernel come from two rocprofv3 --pmc runs (FETCH_SIZE,
# WRITE_SIZE); the summary of those runs states the scaled sum on a line of its own, which is read here.
CONFIG4_PMC_SUMMARY = os.path.join(ROOT, "profiles", "rows_kernel_fetch_config4_pmc.md")


def config4_traffic_bytes():
    """`roofline.traffic` per map layout: the figures the counter summary under profiles/ states on lines
    "traffic_bytes_per_launch[<layout>]: N"; an empty dict when the summary is absent."""
    found = {}
    try:
        with open(CONFIG4_PMC_SUMMARY) as f:
            for line in f:
                line = line.strip()
                if line.startswith("traffic_bytes_per_launch["):
                    layout = line[line.index("[") + 1:line.index("]")]
                    found[layout] = int(line.split(":")[1].split()[0].replace(",", ""))
    except OSError:
        pass
    return found


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def gpu_time_ms(fn, iters, warmup=3):
    """Median / mean / min of per-call durations measured with events on the
    current stream (the stream every operator launches on)."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(iters):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    times.sort()
    return {"median": times[len(times) // 2], "mean": sum(times) / len(times), "min": times[0]}


# ---------------------------------------------------------------------------
# config 4 (+ all-hit / all-miss / set): feature fetch

def build_feature_table(n_rows, dim, n_cached, seed):
    """fp16 N(0,1) table generated chunk-wise on the GPU and copied into pinned
    host memory; the first n_cached rows also stay in HBM as the cache."""
    import torch
    host = torch.empty((n_rows, dim), dtype=torch.float16, pin_memory=True)
    cache = torch.empty((n_cached, dim), dtype=torch.float16, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(seed)
    chunk = 4_000_000
    for lo in range(0, n_rows, chunk):
        hi = min(n_rows, lo + chunk)
        block = torch.randn((hi - lo, dim), device="cuda", generator=g).to(torch.float16)
        host[lo:hi].copy_(block, non_blocking=True)
        if lo < n_cached:
            c_hi = min(hi, n_cached)
            cache[lo:c_hi].copy_(block[: c_hi - lo])
        torch.cuda.synchronize()
    return host, cache


def bench_fetch(capi, args, result):
    import numpy as np
    import torch
    from shmtensor_amd.synthetic import zipf_ranks
    from oracle import oracle as orc

    N, D, Q = args.fetch_rows, 128, 1 << 20
    R = D * 2
    t0 = time.time()
    while True:     # if the box cannot pin the full table, halve it and say so in config.workload
        C = int(N * 0.4)
        try:
            host, cache = build_feature_table(N, D, C, seed=2)
            break
        except RuntimeError as exc:
            if N <= 1_000_000:
                raise
            log("[fetch] cannot allocate the %d-row table (%s): retrying with half" % (N, str(exc)[:80]))
            N //= 2
            torch.cuda.empty_cache()
    log("[fetch] table %d x %d fp16 (%.1f GB pinned), cache %d rows (%.2f GB HBM): %.1f s"
        % (N, D, N * R / 1e9, C, C * R / 1e9, time.time() - t0))
    keys = torch.arange(C, device="cuda")
    # The timed map is the general bucket table (int64 -> int64: 16-byte slots, one 128-byte bucket line per
    # probe), built whatever the keys look like, as the reference's cuco::static_map is. Left to itself the
    # constructor recognises this configuration's keys (ids 0 .. C-1 -> slot = id) as an id range and builds
    # no table at all; that form is timed beside it and reported as roofline_auto_layout.
    hmap = capi.CUCOStaticHashmap(keys, keys.clone(), 0.8, layout="buckets")
    hmap_auto = capi.CUCOStaticHashmap(keys, keys.clone(), 0.8)
    del keys
    nb = 8
    batches = [zipf_ranks(Q, N, 1.1, seed=100 + i) for i in range(nb)]
    hit_rate = float((batches[0] < C).float().mean())

    # correctness of the timed operator on the timed input (bit patterns)
    ref = torch.index_select(host.view(torch.int16), 0, batches[0].cpu())
    for m in (hmap, hmap_auto):
        out = capi.cache_fetch(host, cache, batches[0], m)
        assert torch.equal(out.cpu().view(torch.int16), ref), "cache_fetch differs from index_select"
        del out
    del ref

    W, K = args.warmup, args.steps
    algo_bytes = Q * (2 * R + 8)

    def timed_steps(m):
        for i in range(W):
            capi.cache_fetch(host, cache, batches[i % nb], m)
        torch.cuda.synchronize()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(K)]
        t0 = time.perf_counter()
        for i in range(K):
            ev[i][0].record()
            capi.cache_fetch(host, cache, batches[i % nb], m)
            ev[i][1].record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        kern_ms = sum(a.elapsed_time(b) for a, b in ev) / K
        return wall * 1e3 / K, kern_ms

    def roofline_of(m, kern_ms, traffic):
        achieved = algo_bytes / (kern_ms * 1e-3) / 1e9
        fmt = {"buckets": "map16" if m.memory_usage() >= 16 * 2 * C else "map8"}.get(m.layout(), "map_flat")
        return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                "kernel": "rows_kernel<u32x4, %s, fetch>" % fmt, "kernel_ms": round(kern_ms, 4),
                "bytes_per_launch": algo_bytes, "map_layout": m.layout(), "map_bytes": m.memory_usage()}

    traffic = config4_traffic_bytes() if N == 100_000_000 else {}
    if args.headline_only and args.headline_map == "auto":      # profiler runs of the id-range form only
        hmap = hmap_auto
    ms_per_step, kern_ms = timed_steps(hmap)
    value = Q * R / (ms_per_step * 1e-3) / 1e9
    result.update({"value": round(value, 2), "ms_per_step": round(ms_per_step, 4),
                   "roofline": roofline_of(hmap, kern_ms, traffic.get("range" if hmap is hmap_auto else "buckets"))})
    result["config"].update({"workload": "config 4: cache_fetch, %d x %d fp16 table pinned, %d rows cached, "
                             "Q=%d Zipf(1.1), general bucket hashmap" % (N, D, C, Q), "hit_rate": round(hit_rate, 4),
                             "row_bytes": R, "queries_per_step": Q, "map_layout": hmap.layout()})
    if not args.headline_only:
        ms_auto, kern_auto = timed_steps(hmap_auto)
        result["roofline_auto_layout"] = roofline_of(hmap_auto, kern_auto, traffic.get("range"))
        result["roofline_auto_layout"]["value_GBs"] = round(Q * R / (ms_auto * 1e-3) / 1e9, 2)
    extra = result["extra"]
    if args.headline_only:
        del host, cache, hmap
        return

    # what bounds the headline launch: its hits alone (the missed queries redirected to cached rows, same
    # locality) and its misses alone (only the missed queries, through the same kernel, over the host link)
    q0 = batches[0]
    missed = q0 >= C
    q_hits = torch.where(missed, q0 % C, q0)
    q_miss = q0[missed].contiguous()
    t_hits = gpu_time_ms(lambda: capi.cache_fetch(host, cache, q_hits, hmap), 30)
    t_miss = gpu_time_ms(lambda: capi.cache_fetch(host, cache, q_miss, hmap), 30)
    t_both = gpu_time_ms(lambda: capi.cache_fetch(host, cache, q0, hmap), 30)
    extra["config4_components"] = {
        "as_specified_ms": round(t_both["median"], 4), "hits_only_ms": round(t_hits["median"], 4),
        "misses_only_ms": round(t_miss["median"], 4), "missed_queries": int(q_miss.numel()),
        "misses_only_host_link_GBs": round(q_miss.numel() * R / (t_miss["median"] * 1e-3) / 1e9, 2)}
    del q_hits, q_miss, missed

    # pinned host -> device copy ceiling (DMA engine), the miss-path roofline
    nbytes = min(1 << 30, host.numel() * 2)
    rows = nbytes // R
    dst = torch.empty((rows, D), dtype=torch.float16, device="cuda")
    t = gpu_time_ms(lambda: dst.copy_(host[:rows], non_blocking=True), 10)
    h2d = nbytes / (t["median"] * 1e-3) / 1e9
    del dst
    extra["pinned_h2d_copy_GBs"] = round(h2d, 2)

    # device-to-device copy ceiling (read + write bytes), for scale next to the 8 TB/s peak
    src = cache[: (1 << 30) // R]
    dst = torch.empty_like(src)
    t = gpu_time_ms(lambda: dst.copy_(src), 20)
    extra["d2d_copy_GBs_read_plus_write"] = round(2 * src.numel() * 2 / t["median"] / 1e6, 1)
    del dst, src
    # streaming ceiling of the same kernel: sequential ids on the HBM table (a plain copy)
    qs = torch.arange(Q, device="cuda")
    t = gpu_time_ms(lambda: capi.uva_fetch(cache, qs), 30)
    extra["sequential_copy_same_kernel"] = {"ms": round(t["median"], 4), "ms_min": round(t["min"], 4),
                                            "algorithmic_GBs": round(algo_bytes / t["median"] / 1e6, 1)}
    # all-hit: uniform queries over the cached ids (no locality), HBM bound
    qh = torch.randint(0, C, (Q,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(7))
    t = gpu_time_ms(lambda: capi.cache_fetch(host, cache, qh, hmap_auto), 30)
    a = algo_bytes / (t["median"] * 1e-3) / 1e9
    extra["fetch_all_hit"] = {"ms": round(t["median"], 4), "ms_min": round(t["min"], 4), "algorithmic_GBs": round(a, 1),
                              "frac_hbm_peak": round(a / HBM_PEAK_GBS, 4), "payload_GBs": round(Q * R / t["median"] / 1e6, 1),
                              "map_layout": hmap_auto.layout(),
                              "note": "the configuration's own map: ids 0..C-1 -> slot = id, recognised as an id range"}
    tm = gpu_time_ms(lambda: capi.cache_fetch_with_mask(host, cache, qh, qh), 30)
    a = algo_bytes / (tm["median"] * 1e-3) / 1e9
    extra["fetch_all_hit_with_mask"] = {"ms": round(tm["median"], 4), "algorithmic_GBs": round(a, 1),
                                        "frac_hbm_peak": round(a / HBM_PEAK_GBS, 4)}
    # The same all-hit batch through maps that do need a table. A cache whose rows are kept in id order (39 % of
    # the ids 0 .. N-1, scattered; slot = rank of the id): bitmap with running counts, 16.7 MB, served from the
    # caches. Slots in arbitrary order over the ids 0 .. C-1: direct table, one 4-byte load per row. Scattered
    # ids with slots in arbitrary order: bucket table, one 128-byte bucket per probe. A random read from a table
    # that does not fit the caches costs a whole 128-byte line whatever its size, so the last two move
    # Q x (2R + 8 + 128) bytes for Q x (2R + 8) algorithmic ones: line_traffic_GBs is that real figure.
    gq = torch.Generator(device="cuda").manual_seed(17)
    by_table = {}
    kept = torch.nonzero(torch.rand(N, device="cuda", generator=gq) < 0.39).flatten()[:C].contiguous()
    m = capi.CUCOStaticHashmap(kept, torch.arange(kept.numel(), device="cuda"), 0.8)
    pos = torch.randint(0, kept.numel(), (Q,), device="cuda", generator=gq)
    req = kept[pos]
    assert torch.equal(capi.cache_fetch(host, cache, req[:4096], m), cache[pos[:4096]])
    tt = gpu_time_ms(lambda: capi.cache_fetch(host, cache, req, m), 30)
    a = algo_bytes / (tt["median"] * 1e-3) / 1e9
    by_table["rank_bitmap"] = {"ms": round(tt["median"], 4), "map_layout": m.layout(), "map_bytes": m.memory_usage(),
                               "keys": kept.numel(), "algorithmic_GBs": round(a, 1),
                               "frac_hbm_peak": round(a / HBM_PEAK_GBS, 4)}
    del m, kept, pos, req
    ids = torch.arange(C, device="cuda")
    slots = torch.randperm(C, device="cuda", generator=gq)
    for name, keys_t, req in (("direct_table", ids, qh), ("bucket_table_8B_slots", ids * 11 + 1, qh * 11 + 1),
                              ("bucket_table_16B_slots", ids * 37 + (1 << 33), qh * 37 + (1 << 33))):
        m = capi.CUCOStaticHashmap(keys_t, slots, 0.8)
        assert torch.equal(capi.cache_fetch(host, cache, req[:4096], m), cache[slots[qh[:4096]]])
        tt = gpu_time_ms(lambda: capi.cache_fetch(host, cache, req, m), 30)
        a = algo_bytes / (tt["median"] * 1e-3) / 1e9
        by_table[name] = {"ms": round(tt["median"], 4), "map_layout": m.layout(), "map_bytes": m.memory_usage(),
                          "algorithmic_GBs": round(a, 1), "frac_hbm_peak": round(a / HBM_PEAK_GBS, 4),
                          "line_traffic_GBs": round(Q * (2 * R + 8 + 128) / tt["median"] / 1e6, 1)}
        del m, keys_t, req
    extra["fetch_all_hit_by_map_layout"] = by_table
    del ids, slots
    # all-miss: uniform queries over the uncached ids, host-link bound
    qm = torch.randint(C, N, (Q,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(8))
    t = gpu_time_ms(lambda: capi.cache_fetch(host, cache, qm, hmap), 10)
    m = Q * R / (t["median"] * 1e-3) / 1e9
    extra["fetch_all_miss"] = {"ms": round(t["median"], 4), "ms_min": round(t["min"], 4), "host_link_GBs": round(m, 2),
                               "frac_of_pinned_copy": round(m / h2d, 4)}
    t = gpu_time_ms(lambda: capi.uva_fetch(host, qm), 10)
    m = Q * R / (t["median"] * 1e-3) / 1e9
    extra["uva_fetch"] = {"ms": round(t["median"], 4), "ms_min": round(t["min"], 4), "host_link_GBs": round(m, 2),
                          "frac_of_pinned_copy": round(m / h2d, 4)}

    # cache_set pass of config 4: 262,144 unique cached rows
    ns = 262_144
    sidx = torch.randperm(C, device="cuda", generator=torch.Generator(device="cuda").manual_seed(9))[:ns].contiguous()
    upd = torch.randn((ns, D), device="cuda").to(torch.float16)
    t = gpu_time_ms(lambda: capi.cache_set(host, cache, sidx, upd, hmap), 30)
    assert torch.equal(capi.cache_fetch(host, cache, sidx, hmap), upd)
    a = ns * (2 * R + 8) / (t["median"] * 1e-3) / 1e9
    # floor: the same bytes at the rate the 1,048,576-row all-hit fetch sustains (a launch four times shorter
    # spends a larger share of its time filling and draining the chip)
    t_auto = gpu_time_ms(lambda: capi.cache_set(host, cache, sidx, upd, hmap_auto), 30)
    extra["cache_set_262144"] = {"ms": round(t["median"], 4), "ms_min": round(t["min"], 4), "algorithmic_GBs": round(a, 1),
                                 "frac_hbm_peak": round(a / HBM_PEAK_GBS, 4), "map_layout": hmap.layout(),
                                 "ms_through_the_id_range_map": round(t_auto["median"], 4),
                                 "floor_ms_at_all_hit_fetch_rate": round(tm["median"] * ns / Q, 4),
                                 "floor_ms_at_hbm_peak": round(ns * (2 * R + 8) / HBM_PEAK_GBS / 1e6, 4)}

    # scatter to the host table over the link (all misses): 262,144 uncached rows
    sm = torch.randperm(N - C, device="cuda", generator=torch.Generator(device="cuda").manual_seed(10))[:ns] + C
    t = gpu_time_ms(lambda: capi.cache_set(host, cache, sm, upd, hmap), 10)
    torch.cuda.synchronize()
    assert torch.equal(host[sm[:64].cpu()].view(torch.int16), upd[:64].cpu().view(torch.int16))
    extra["cache_set_all_miss_262144"] = {"ms": round(t["median"], 4), "ms_min": round(t["min"], 4),
                                          "host_link_write_GBs": round(ns * R / t["median"] / 1e6, 2)}

    # CPU baseline: the reference's cpu_fetch idiom is data[query.cpu()] (example/test_cache_fetch.py:138);
    # timed here as the oracle's OpenMP gather and as torch.index_select on the same batch
    if not args.no_cpu:
        q_cpu = batches[0].cpu().numpy()
        host_np = host.view(torch.int16).numpy()
        threads = orc.num_threads()
        orc.fetch(host_np, None, q_cpu)
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < args.cpu_seconds:
            orc.fetch(host_np, None, q_cpu)
            reps += 1
        cpu_t = (time.perf_counter() - t0) / reps
        qt = batches[0].cpu()
        torch.index_select(host, 0, qt)
        t1 = time.perf_counter()
        for _ in range(5):
            torch.index_select(host, 0, qt)
        torch_t = (time.perf_counter() - t1) / 5
        result["cpu_baseline"] = {
            "value": round(Q * R / cpu_t / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "%d passes of one 1,048,576-query Zipf batch over the same host table (oracle gather, "
                      "OpenMP); torch.index_select with %d threads on the same batch: %.2f GB/s"
                      % (reps, torch.get_num_threads(), Q * R / torch_t / 1e9)}
        # CPU set: the reference's cpu_data[idx] = update idiom (example/test_cache_set.py:183-184)
        sidx_cpu, upd_cpu = sidx.cpu(), upd.cpu()
        host[sidx_cpu] = upd_cpu
        t1 = time.perf_counter()
        for _ in range(5):
            host[sidx_cpu] = upd_cpu
        set_t = (time.perf_counter() - t1) / 5
        extra["cache_set_262144"]["cpu_index_put_ms"] = round(set_t * 1e3, 3)
        extra["cache_set_262144"]["cpu_threads"] = torch.get_num_threads()
    del host, cache, hmap, hmap_auto


# ---------------------------------------------------------------------------
# config 1: small fetch, as specified (~25 % hits) plus all-hit and all-miss variants

def bench_fetch_small(capi, args, result):
    import torch
    torch.manual_seed(0)
    N, D, C, Q = 200_000, 128, 50_000, 65_536
    R = D * 4
    table = torch.randn(N, D).pin_memory()
    ids = torch.randperm(N)[:C]
    cache = table[ids].cuda()
    ids = ids.cuda()
    hmap = capi.CUCOStaticHashmap(ids, torch.arange(C, device="cuda"), 0.8)
    q = torch.randint(0, N, (Q,)).cuda()
    out = capi.cache_fetch(table, cache, q, hmap)
    assert torch.equal(out.cpu(), torch.index_select(table, 0, q.cpu()))
    hit = float((hmap.query(q) >= 0).float().mean())
    q_hit = ids[torch.randint(0, C, (Q,), device="cuda")]
    cached = torch.zeros(N, dtype=torch.bool, device="cuda")
    cached[ids] = True
    cold = torch.nonzero(~cached).flatten()
    q_miss = cold[torch.randint(0, cold.numel(), (Q,), device="cuda")]
    res = {"hit_rate": round(hit, 4)}
    for name, qq in (("as_specified", q), ("all_hit", q_hit), ("all_miss", q_miss)):
        t = gpu_time_ms(lambda: capi.cache_fetch(table, cache, qq, hmap), 30)
        res[name] = {"ms": round(t["median"], 4), "ms_min": round(t["min"], 4), "payload_GBs": round(Q * R / t["median"] / 1e6, 2),
                     "algorithmic_GBs": round(Q * (2 * R + 8) / t["median"] / 1e6, 1)}
    if not args.no_cpu:
        qc = q.cpu()
        torch.index_select(table, 0, qc)
        t0 = time.perf_counter()
        for _ in range(20):
            torch.index_select(table, 0, qc)
        res["cpu_index_select_GBs"] = round(Q * R * 20 / (time.perf_counter() - t0) / 1e9, 2)
        res["cpu_threads"] = torch.get_num_threads()
    result["extra"]["fetch_config1"] = res


# ---------------------------------------------------------------------------
# config 2: static hashmap

def bench_hashmap(capi, args, result):
    import torch
    n, nq = 4_194_304, 16_777_216
    g = torch.Generator(device="cuda").manual_seed(22)
    keys = torch.unique(torch.randint(0, 1 << 40, (n + n // 8,), device="cuda", generator=g))
    keys = keys[torch.randperm(keys.numel(), device="cuda", generator=g)][:n].contiguous()
    vals = torch.arange(n, device="cuda")
    pick = torch.randint(0, n, (nq // 2,), device="cuda", generator=g)
    non = torch.randint(0, 1 << 40, (nq // 2,), device="cuda", generator=g) | (1 << 41)
    perm = torch.randperm(nq, device="cuda", generator=g)
    req = torch.cat([keys[pick], non])[perm].contiguous()
    expect = torch.cat([pick, torch.full_like(non, -1)])[perm]
    del non, perm, pick
    tb = gpu_time_ms(lambda: capi.CUCOStaticHashmap(keys, vals, 0.5), 10)
    h = capi.CUCOStaticHashmap(keys, vals, 0.5)
    assert torch.equal(h.query(req), expect)
    tq = gpu_time_ms(lambda: h.query(req), 30)
    result["extra"]["hashmap_config2"] = {
        "build_ms": round(tb["median"], 4), "build_Mkeys_s": round(n / tb["median"] / 1e3, 1),
        "query_ms": round(tq["median"], 4), "query_Mkeys_s": round(nq / tq["median"] / 1e3, 1),
        "query_algorithmic_GBs": round(nq * 32 / tq["median"] / 1e6, 1),
        "query_frac_hbm_peak": round(nq * 32 / tq["median"] / 1e6 / HBM_PEAK_GBS, 4),
        # what the memory system moves: a probe reads one whole 128-byte bucket line (FETCH_SIZE per launch in
        # profiles/hashmap_sampling_kernels_pmc.md: 2,291 MB = nq x (128 + 8)), next to 8 B request + 8 B result
        "query_line_traffic_GBs": round(nq * 144 / tq["median"] / 1e6, 1),
        "query_line_traffic_frac_hbm_peak": round(nq * 144 / tq["median"] / 1e6 / HBM_PEAK_GBS, 4),
        "table_bytes": h.memory_usage(), "map_layout": h.layout()}
    if not args.no_cpu:
        from oracle import oracle as orc
        k_np, v_np, r_np = keys.cpu().numpy(), vals.cpu().numpy(), req[: nq // 4].cpu().numpy()
        t0 = time.perf_counter()
        m = orc.Hashmap(k_np, v_np, 0.5)
        tbuild = time.perf_counter() - t0
        t0 = time.perf_counter()
        m.query(r_np)
        tquery = time.perf_counter() - t0
        result["extra"]["hashmap_config2"]["cpu_oracle"] = {
            "build_Mkeys_s": round(n / tbuild / 1e6, 2), "query_Mkeys_s": round(r_np.size / tquery / 1e6, 2),
            "cores": orc.num_threads(), "sample": "build 4,194,304 keys (1 thread); query 4,194,304 requests (OpenMP)"}


def bench_hashmap_sweep(capi, args, result):
    """Bulk query rate against the size of the bucket table (int64 keys, 16-byte slots, load factor 0.5):
    where the probes are served from (the 4 MB L2 of each of the 8 XCDs, the 256 MB memory-side cache, HBM)."""
    import torch
    nq = 1 << 24
    g = torch.Generator(device="cuda").manual_seed(1)
    rows = []
    for lg in range(14, 27):
        n = 1 << lg
        keys = (torch.randperm(1 << 27, device="cuda", generator=g)[:n] * 8191 + (1 << 34)).contiguous()
        h = capi.CUCOStaticHashmap(keys, torch.arange(n, device="cuda"), 0.5)
        req = keys[torch.randint(0, n, (nq,), device="cuda", generator=g)]
        t = gpu_time_ms(lambda: h.query(req), 10)
        rows.append({"keys": n, "table_MiB": round(h.memory_usage() / 2**20, 1), "query_ms": round(t["median"], 4),
                     "Gkeys_s": round(nq / t["median"] / 1e6, 1),
                     "line_traffic_GBs": round(nq * 144 / t["median"] / 1e6, 1)})
        del h, req, keys
    result["extra"]["hashmap_query_by_table_size"] = rows


# ---------------------------------------------------------------------------
# scans (cub_exclusiveSum / thrust_scan of the reference): 2 * n * element bytes against the HBM peak

def bench_scan(capi, args, result):
    import torch
    from shmtensor_amd import cabi
    lib = cabi.load()
    n = 1 << 24
    res = {}
    a64 = torch.randint(0, 1000, (n,), device="cuda", dtype=torch.int64)
    work = a64.clone()
    tmp_bytes = lib.shmt_scan_tmp_bytes(n)
    tmp = torch.empty(max(tmp_bytes, 1), dtype=torch.uint8, device="cuda")
    stream = cabi.current_stream()
    cabi.check(lib.shmt_exclusive_scan(work.data_ptr(), n, 8, tmp.data_ptr(), tmp_bytes, stream))
    expect = torch.cumsum(a64, 0) - a64
    assert torch.equal(work, expect), "exclusive scan differs from cumsum"
    del expect

    def ex64():     # in place: rescanning the scanned values costs the same
        cabi.check(lib.shmt_exclusive_scan(work.data_ptr(), n, 8, tmp.data_ptr(), tmp_bytes, stream))

    def ex64_kept():    # the workspace is kept clean by the scans themselves: no clearing launch
        cabi.check(lib.shmt_exclusive_scan_kept(work.data_ptr(), n, 8, tmp.data_ptr(), tmp_bytes, stream))
    t_any = gpu_time_ms(ex64, 30)
    cabi.check(lib.shmt_scan_workspace_clear(tmp.data_ptr(), tmp_bytes, stream))
    t = gpu_time_ms(ex64_kept, 30)
    res["exclusive_int64_16777216"] = {"ms": round(t["median"], 4), "algorithmic_GBs": round(2 * n * 8 / t["median"] / 1e6, 1),
                                       "frac_hbm_peak": round(2 * n * 8 / t["median"] / 1e6 / HBM_PEAK_GBS, 4),
                                       "workspace": "kept clean (shmt_exclusive_scan_kept)",
                                       "ms_with_a_workspace_cleared_per_call": round(t_any["median"], 4)}
    a32 = torch.randint(0, 100, (n,), device="cuda", dtype=torch.int32)
    t = gpu_time_ms(lambda: capi.thrust_scan(a32), 30)
    res["thrust_scan_int32_16777216"] = {"ms": round(t["median"], 4), "algorithmic_GBs": round(2 * n * 4 / t["median"] / 1e6, 1),
                                         "frac_hbm_peak": round(2 * n * 4 / t["median"] / 1e6 / HBM_PEAK_GBS, 4)}
    tt = gpu_time_ms(lambda: torch.cumsum(a64, 0), 10)
    res["torch_cumsum_int64_ms"] = round(tt["median"], 4)
    if not args.no_cpu:
        import numpy as np
        from oracle import oracle as orc
        a_np = a64.cpu().numpy()
        t0 = time.perf_counter()
        orc.exclusive_scan(a_np)
        res["cpu_baseline"] = {"ms": round((time.perf_counter() - t0) * 1e3, 2), "cores": 1, "kind": "port",
                               "sample": "one exclusive scan of the same 16,777,216 int64 (oracle, sequential, incl. a copy)"}
    result["extra"]["scan"] = res


# ---------------------------------------------------------------------------
# config 3: cached 3-hop sampling + relabel

def bench_sampling(capi, args, result):
    import numpy as np
    import torch
    from shmtensor_amd.synthetic import rmat_csr
    t0 = time.time()
    indptr_d, indices_d = rmat_csr(args.sampling_scale, 30, seed=1)
    n = indptr_d.numel() - 1
    indptr = indptr_d.cpu().pin_memory()
    indices = indices_d.cpu().pin_memory()
    deg = indptr_d[1:] - indptr_d[:-1]
    # the cached rows are kept in id order (slot = rank of the id): the map is then a bitmap with running counts
    hot = torch.sort(torch.sort(deg, descending=True, stable=True).indices[: n * 3 // 10]).values.contiguous()
    del indptr_d, indices_d
    gp, gi = capi.create_subcsr(indptr, indices, hot)
    hmap = capi.CUCOStaticHashmap(hot, torch.arange(hot.numel(), device="cuda"), 0.8)
    log("[sampling] R-MAT scale %d: %d nodes, %d edges, cache %d rows / %d edges (%.0f %% of edges): %.1f s"
        % (args.sampling_scale, n, indices.numel(), hot.numel(), gi.numel(),
           100.0 * gi.numel() / indices.numel(), time.time() - t0))
    fanouts, S, nbatch = [15, 10, 5], 1024, args.sampling_batches
    g = torch.Generator(device="cuda").manual_seed(33)
    seed_batches = [torch.randperm(n, device="cuda", generator=g)[:S].contiguous() for _ in range(nbatch)]

    indptr_hbm = indptr.cuda()      # 8 bytes per node: small next to the adjacency, which stays split

    def run_batch(seeds, b, fused=False, ptr=None):
        edges = 0
        for hop, k in enumerate(reversed(fanouts)):       # python/shmtensor/sampling.py:128
            if fused:     # the same two operators queued as one call (one host wait per hop)
                sp, si, uniq, rel = capi.sample_hop(indptr if ptr is None else ptr, indices, gp, gi, hmap, seeds, k,
                                                    False, seed=7777 + b, stream_id=hop)
            else:
                sp, si = capi.csr_cache_sampling(indptr, indices, gp, gi, hmap, seeds, k, False, seed=7777 + b,
                                                 stream_id=hop)
                uniq, (_, rel) = capi.tensor_relabel([seeds, si])
            edges += si.numel()
            seeds = uniq
        return edges

    def timed(fused, ptr=None):
        for b in range(3):
            run_batch(seed_batches[b], b, fused, ptr)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        edges = sum(run_batch(seed_batches[b], b, fused, ptr) for b in range(nbatch))
        torch.cuda.synchronize()
        return edges, time.perf_counter() - t0

    picks = list(reversed(fanouts))

    def timed_in_flight(in_flight, row_offsets=indptr):
        """All batches through sample_blocks (hops chained on the device): up to `in_flight` of them
        advance concurrently."""
        rng = [7777 + b for b in range(nbatch)]
        for _ in range(2):
            capi.sample_blocks(row_offsets, indices, gp, gi, hmap, seed_batches, picks, False, seeds_rng=rng,
                               max_in_flight=in_flight)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        res = capi.sample_blocks(row_offsets, indices, gp, gi, hmap, seed_batches, picks, False, seeds_rng=rng,
                                 max_in_flight=in_flight)
        torch.cuda.synchronize()
        t = time.perf_counter() - t0
        return sum(hop[1].numel() for chain in res for hop in chain), t

    edges, gpu_t = timed(False)
    edges_fused, gpu_t_fused = timed(True)
    assert edges_fused == edges, "fused hop sampled a different number of edges"
    # the caller's choice, not part of the configuration: the whole indptr in HBM (cold rows then cost one
    # host-link round trip per hop instead of two)
    edges_hbm, gpu_t_hbm = timed(True, indptr_hbm)
    assert edges_hbm == edges, "indptr placement changed the sample"
    overlapped = {}
    for in_flight in (1, 2, 4, 8, 16):
        e, t = timed_in_flight(in_flight)
        assert e == edges, "batched hops sampled a different number of edges"
        overlapped["%d_batches_in_flight" % in_flight] = {"ms_per_batch": round(t * 1e3 / nbatch, 4),
                                                          "sampled_edges_per_s": round(e / t, 1)}
    e, t_chain_hbm = timed_in_flight(1, indptr_hbm)
    assert e == edges, "indptr placement changed the sample"
    # the batch recorded once as a HIP graph and replayed per batch (one staging kernel + one graph launch)
    sampler = capi.BatchSampler(indptr, indices, gp, gi, hmap, S, picks, False)
    replayed = {}

    def replay_all(in_flight):
        """Every batch through submit / collect with `in_flight` batches queued ahead; a batch's results are
        dropped as soon as they are counted (as a training loop consumes them), so lanes are reused."""
        e, tickets, nxt = 0, collections.deque(), 0
        while nxt < nbatch or tickets:
            while nxt < nbatch and len(tickets) < in_flight:
                tickets.append(sampler.submit(seed_batches[nxt], 7777 + nxt))
                nxt += 1
            chain = sampler.collect(tickets.popleft())
            e += sum(hop[1].numel() for hop in chain)
            del chain
        return e

    for in_flight in (1, 2, 4, 8):
        for _ in range(2):
            replay_all(in_flight)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e = replay_all(in_flight)
        torch.cuda.synchronize()
        t = time.perf_counter() - t0
        assert e == edges, "replayed batches sampled a different number of edges"
        replayed["%d_batches_in_flight" % in_flight] = {"ms_per_batch": round(t * 1e3 / nbatch, 4),
                                                        "sampled_edges_per_s": round(e / t, 1),
                                                        "lanes": sampler.lanes()}
    del sampler
    res = {"graph": "R-MAT scale %d ef 30 symmetrised: %d nodes, %d edges; top 30 %% by degree cached"
                    % (args.sampling_scale, n, indices.numel()),
           "map_layout": hmap.layout(),
           "seeds_per_batch": S, "fanouts_in_call_order": list(reversed(fanouts)), "batches": nbatch,
           "edges_per_batch": edges // nbatch, "ms_per_batch": round(gpu_t * 1e3 / nbatch, 4),
           "sampled_edges_per_s": round(edges / gpu_t, 1),
           "fused_hop_ms_per_batch": round(gpu_t_fused * 1e3 / nbatch, 4),
           "fused_hop_sampled_edges_per_s": round(edges / gpu_t_fused, 1),
           "fused_hop_indptr_in_hbm_ms_per_batch": round(gpu_t_hbm * 1e3 / nbatch, 4),
           "chained_hops_ms_per_batch": overlapped["1_batches_in_flight"]["ms_per_batch"],
           "chained_hops_indptr_in_hbm_ms_per_batch": round(t_chain_hbm * 1e3 / nbatch, 4),
           "sample_blocks_batches_in_flight": overlapped,
           "batch_sampler_graph_replay": replayed}
    if not args.no_cpu:
        from oracle import oracle as orc
        ip, ix = indptr.numpy(), indices.numpy().astype(np.int64)
        nb_cpu = min(nbatch, 20)

        def cpu_pipeline(sampler, relabeler):
            """(edges, seconds in the sampler, seconds in the relabel) over nb_cpu batches."""
            total, t_samp, t_rel = 0, 0.0, 0.0
            for b in range(nb_cpu):
                seeds = seed_batches[b].cpu().numpy()
                for hop, k in enumerate(reversed(fanouts)):
                    t0 = time.perf_counter()
                    sp, si = orc.sample(ip, ix, seeds, k, False, seed=7777 + b, stream=hop, algo=sampler)
                    t1 = time.perf_counter()
                    uniq, _ = orc.relabel([seeds, si], algo=relabeler)
                    t2 = time.perf_counter()
                    t_samp += t1 - t0
                    t_rel += t2 - t1
                    total += si.size
                    seeds = uniq
            return total, t_samp, t_rel

        # (a) the reference's algorithms on host cores: Algorithm R (O(degree) draws per seed) and the four-pass
        #     relabel over its low-bit hash table; (b) what a CPU programmer would write for the same contract,
        #     on all cores: Floyd's O(k) subset selection (OpenMP over seeds) and a multi-core relabel (ids dealt
        #     to one partition per thread by their mixed hash, in index order; every thread sweeps its own
        #     partition with a private table; first occurrences ranked by a prefix sum; tables kept between
        #     calls; inputs below 16,384 ids take the sequential sweep); (c) as (b) with the relabel as ONE
        #     sequential sweep whatever the size. The speed-ups are quoted
        #     against the fastest of the three.
        def entry(e, ts, tr, what):
            return {"sampled_edges_per_s": round(e / (ts + tr), 1), "cores": orc.num_threads(), "kind": "port",
                    "sample_ms_per_batch": round(ts * 1e3 / nb_cpu, 3), "relabel_ms_per_batch": round(tr * 1e3 / nb_cpu, 3),
                    "sample": "%d batches, %s (oracle)" % (nb_cpu, what)}
        e_ref, ts_ref, tr_ref = cpu_pipeline("reservoir", "passes")
        e_par, ts_par, tr_par = cpu_pipeline("floyd", "parallel")
        e_swp, ts_swp, tr_swp = cpu_pipeline("floyd", "sweep")
        res["cpu_baseline_reference_algorithms"] = entry(
            e_ref, ts_ref, tr_ref, "Algorithm-R sampler + four-pass low-bit-hash relabel, both OpenMP")
        res["cpu_baseline"] = entry(
            e_par, ts_par, tr_par, "Floyd O(k) sampler (OpenMP over seeds) + multi-core relabel (OpenMP, hash-"
                                   "partitioned, private tables kept between calls)")
        res["cpu_baseline_sequential_relabel"] = entry(
            e_swp, ts_swp, tr_swp, "Floyd O(k) sampler (OpenMP over seeds) + one-sweep mixed-hash relabel (one thread)")
        rates = {"reference_algorithms": e_ref / (ts_ref + tr_ref), "multi_core_relabel": e_par / (ts_par + tr_par),
                 "sequential_relabel": e_swp / (ts_swp + tr_swp)}
        best = max(rates.values())
        res["cpu_baseline_fastest"] = max(rates, key=rates.get)
        # quoted for the reference's operators called one after the other, one batch at a time (the slowest way
        # to drive the GPU path); the merged-launch form of the same batches is given beside it
        res["speedup_vs_cpu"] = round((edges / gpu_t) / best, 2)
        res["speedup_vs_cpu_reference_algorithms"] = round((edges / gpu_t) / rates["reference_algorithms"], 2)
        res["speedup_vs_cpu_chained_hops"] = round(overlapped["1_batches_in_flight"]["sampled_edges_per_s"] / best, 2)
        gpu_best = max(v["sampled_edges_per_s"] for v in overlapped.values())
        res["speedup_vs_cpu_batches_sharing_launches"] = round(gpu_best / best, 2)
    result["extra"]["sampling_config3"] = res


# ---------------------------------------------------------------------------
# config 5: end-to-end mini-batch (sample 3 hops + relabel, then fetch the input nodes' features)

def bench_e2e(capi, args, result):
    import torch
    from shmtensor_amd.synthetic import rmat_csr
    t0 = time.time()
    indptr_d, indices_d = rmat_csr(args.e2e_scale, 16, seed=3)
    n = indptr_d.numel() - 1
    indptr, indices = indptr_d.cpu().pin_memory(), indices_d.cpu().pin_memory()
    deg = indptr_d[1:] - indptr_d[:-1]
    by_degree = torch.sort(deg, descending=True, stable=True).indices
    del indptr_d, indices_d, deg
    hot_adj = torch.sort(by_degree[: n // 5]).values.contiguous()       # cache rows in id order, as above
    gp, gi = capi.create_subcsr(indptr, indices, hot_adj)
    adj_map = capi.CUCOStaticHashmap(hot_adj, torch.arange(hot_adj.numel(), device="cuda"), 0.8)
    D = 256
    feats = torch.empty((n, D), dtype=torch.float32, pin_memory=True)
    g = torch.Generator(device="cuda").manual_seed(3)
    for lo in range(0, n, 2_000_000):
        hi = min(n, lo + 2_000_000)
        feats[lo:hi].copy_(torch.randn((hi - lo, D), device="cuda", generator=g))
    torch.cuda.synchronize()
    hot_feat = torch.sort(by_degree[: n // 4]).values.contiguous()
    feat_cache = capi.uva_fetch(feats, hot_feat)
    feat_map = capi.CUCOStaticHashmap(hot_feat, torch.arange(hot_feat.numel(), device="cuda"), 0.8)
    log("[e2e] R-MAT scale %d ef 16: %d nodes, %d edges; adjacency cache %d rows / %d edges; features %.1f GB "
        "pinned, %.1f GB cached: %.1f s" % (args.e2e_scale, n, indices.numel(), hot_adj.numel(), gi.numel(),
                                            feats.numel() * 4 / 1e9, feat_cache.numel() * 4 / 1e9, time.time() - t0))
    fanouts, S, nbatch = [25, 15, 10], 4096, args.e2e_batches
    gs = torch.Generator(device="cuda").manual_seed(55)
    batches = [torch.randperm(n, device="cuda", generator=gs)[:S].contiguous() for _ in range(nbatch + 1)]

    def one(seeds, b, ev=None, fused=False):
        edges = 0
        if ev: ev[0].record()
        for hop, k in enumerate(reversed(fanouts)):
            if fused:
                sp, si, uniq, rel = capi.sample_hop(indptr, indices, gp, gi, adj_map, seeds, k, False, seed=7777 + b,
                                                    stream_id=hop)
            else:
                sp, si = capi.csr_cache_sampling(indptr, indices, gp, gi, adj_map, seeds, k, False, seed=7777 + b,
                                                 stream_id=hop)
                uniq, (_, rel) = capi.tensor_relabel([seeds, si])
            edges += si.numel()
            seeds = uniq
        if ev: ev[1].record()
        x = capi.cache_fetch(feats, feat_cache, seeds, feat_map)
        if ev: ev[2].record()
        return edges, seeds, x

    edges, inp, x = one(batches[nbatch], nbatch)          # warm-up + check
    assert torch.equal(x.cpu(), torch.index_select(feats, 0, inp.cpu())), "e2e features differ from index_select"
    hit = float((feat_map.query(inp) >= 0).float().mean())
    del x
    tot_edges = tot_nodes = 0
    t_s = t_f = 0.0
    torch.cuda.synchronize()
    w0 = time.perf_counter()
    for b in range(nbatch):
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        e, inp, x = one(batches[b], b, ev)
        ev[2].synchronize()
        t_s += ev[0].elapsed_time(ev[1])
        t_f += ev[1].elapsed_time(ev[2])
        tot_edges += e
        tot_nodes += inp.numel()
        del x
    wall = time.perf_counter() - w0
    # (--e2e-operators-only: the reference's operator sequence alone, the form a profile of single kernels wants)
    wall_fused = wall_pipe = None
    fetched_ms, in_flight_ms = {}, {}
    if not args.e2e_operators_only:
        # the same batches with each hop issued as one fused call
        _, inp_f, x = one(batches[nbatch], nbatch, fused=True)
        del x
        torch.cuda.synchronize()
        w0 = time.perf_counter()
        for b in range(nbatch):
            _, inp_f, x = one(batches[b], b, fused=True)
            del x
        torch.cuda.synchronize()
        wall_fused = time.perf_counter() - w0
        assert torch.equal(inp_f, inp), "fused hops gave different input nodes"
        # the same again with the feature fetch queued behind the last relabel (row count read on the device)
        rng = [7777 + b for b in range(nbatch)]
        picks = list(reversed(fanouts))
        cap = int(1.25 * inp.numel())
        fetched_ms = {}
        for k_in_flight in (1, 2, 4):
            # (the warm-up's results are dropped before the timed call, as a training loop drops each batch: the
            # caching allocator then hands their blocks out again instead of asking the driver for new memory)
            capi.sample_blocks_fetch(indptr, indices, gp, gi, adj_map, batches[:nbatch], picks, False, feats, feat_cache,
                                     feat_map, seeds_rng=rng, max_in_flight=k_in_flight, max_rows=cap)
            torch.cuda.synchronize()
            w0 = time.perf_counter()
            got = capi.sample_blocks_fetch(indptr, indices, gp, gi, adj_map, batches[:nbatch], picks, False, feats,
                                           feat_cache, feat_map, seeds_rng=rng, max_in_flight=k_in_flight, max_rows=cap)
            torch.cuda.synchronize()
            fetched_ms[str(k_in_flight)] = round((time.perf_counter() - w0) * 1e3 / nbatch, 3)
            hops_l, x_l = got[nbatch - 1]
            assert torch.equal(hops_l[-1][2], inp), "sample_blocks_fetch gave different input nodes"
            assert torch.equal(x_l, capi.cache_fetch(feats, feat_cache, inp, feat_map)), "sample_blocks_fetch rows differ"
            del got, hops_l, x_l
        # sampling + relabel only, several batches advancing concurrently
        in_flight_ms = {}
        for k_in_flight in (1, 4, 8):
            rng = [7777 + b for b in range(nbatch)]
            capi.sample_blocks(indptr, indices, gp, gi, adj_map, batches[:nbatch], list(reversed(fanouts)), False,
                               seeds_rng=rng, max_in_flight=k_in_flight)
            torch.cuda.synchronize()
            w0 = time.perf_counter()
            chains = capi.sample_blocks(indptr, indices, gp, gi, adj_map, batches[:nbatch], list(reversed(fanouts)), False,
                                        seeds_rng=rng, max_in_flight=k_in_flight)
            torch.cuda.synchronize()
            in_flight_ms[str(k_in_flight)] = round((time.perf_counter() - w0) * 1e3 / nbatch, 3)
            assert torch.equal(chains[nbatch - 1][-1][2], inp), "sample_blocks gave different input nodes"
            del chains
        # the dataloader sampling ahead on a background thread (4 batches in flight) while this thread fetches
        import shmtensor
        dl = shmtensor.GPUSamplingDataloader(indptr, indices, torch.cat(batches[:nbatch]), S, fanouts, shuffle=False,
                                             rng_seed=7777, prefetch=4, background=True)
        dl.gpu_indptr, dl.gpu_indices, dl.hashmap, dl.has_cache = gp, gi, adj_map, True

        def epoch():
            last = None
            for input_nodes, _, _ in dl:
                x = capi.cache_fetch(feats, feat_cache, input_nodes, feat_map)
                last = input_nodes
                del x
            torch.cuda.synchronize()
            return last

        # first epoch: batch b draws from seed 7777 + b like the loops above (later epochs continue the count)
        assert torch.equal(epoch(), inp), "prefetching dataloader gave different input nodes"
        w0 = time.perf_counter()
        epoch()
        wall_pipe = time.perf_counter() - w0
        dl.close()          # the producer thread has ended with its epoch; this only makes that explicit
    cpu = None
    if not args.no_cpu:
        import numpy as np
        from oracle import oracle as orc
        ip, ix = indptr.numpy(), indices.numpy().astype(np.int64)
        feats_np = feats.numpy()
        nb_cpu = min(nbatch, 2)
        t_samp = t_fetch = 0.0
        c_edges = c_nodes = 0
        for b in range(nb_cpu):
            seeds = batches[b].cpu().numpy()
            t0 = time.perf_counter()
            for hop, k in enumerate(reversed(fanouts)):
                sp, si = orc.sample(ip, ix, seeds, k, False, seed=7777 + b, stream=hop, algo="floyd")
                uniq, _ = orc.relabel([seeds, si], algo="parallel")
                c_edges += si.size
                seeds = uniq
            t1 = time.perf_counter()
            rows = orc.fetch(feats_np, None, seeds)
            t2 = time.perf_counter()
            t_samp += t1 - t0
            t_fetch += t2 - t1
            c_nodes += seeds.size
            del rows
        idx_t = torch.from_numpy(seeds)
        t0 = time.perf_counter()
        torch.index_select(feats, 0, idx_t)
        t_torch = time.perf_counter() - t0
        cpu = {"cores": orc.num_threads(), "kind": "port",
               "sample": "%d batches: Floyd sampler (OpenMP) + multi-core relabel (OpenMP), then an OpenMP gather of the "
                         "input nodes' rows from the same host table (oracle)" % nb_cpu,
               "sample_relabel_ms": round(t_samp * 1e3 / nb_cpu, 2), "fetch_ms": round(t_fetch * 1e3 / nb_cpu, 2),
               "batch_ms": round((t_samp + t_fetch) * 1e3 / nb_cpu, 2),
               "sampled_edges_per_s": round(c_edges / t_samp, 1),
               "fetch_payload_GBs": round(c_nodes * D * 4 / t_fetch / 1e9, 2),
               "torch_index_select_ms": round(t_torch * 1e3, 2), "torch_threads": torch.get_num_threads()}
    result["extra"]["e2e_config5"] = {
        "cpu_baseline": cpu,
        "graph": "R-MAT scale %d ef 16 symmetrised: %d nodes, %d edges; top 20 %% adjacency cached; features %d x %d "
                 "f32 pinned, top-degree 25 %% cached" % (args.e2e_scale, n, indices.numel(), n, D),
        "map_layouts": {"adjacency": adj_map.layout(), "features": feat_map.layout()},
        "seeds_per_batch": S, "fanouts_in_call_order": list(reversed(fanouts)), "batches": nbatch,
        "edges_per_batch": tot_edges // nbatch, "input_nodes_per_batch": tot_nodes // nbatch,
        "feature_hit_rate": round(hit, 4),
        "sample_relabel_ms": round(t_s / nbatch, 3), "fetch_ms": round(t_f / nbatch, 3),
        "batch_ms_wall": round(wall * 1e3 / nbatch, 3), "batches_per_s": round(nbatch / wall, 2),
        "fused_hop_batch_ms_wall": wall_fused and round(wall_fused * 1e3 / nbatch, 3),
        "background_prefetch_batch_ms_wall": wall_pipe and round(wall_pipe * 1e3 / nbatch, 3),
        "sample_blocks_fetch_batch_ms_wall_by_batches_in_flight": fetched_ms,
        "sample_blocks_ms_per_batch_by_batches_in_flight": in_flight_ms,
        "sampled_edges_per_s": round(tot_edges / (t_s * 1e-3), 1),
        "fetch_payload_GBs": round(tot_nodes * D * 4 / (t_f * 1e-3) / 1e9, 2)}


# ---------------------------------------------------------------------------
# the reference's own benchmark harnesses, shape for shape (they only print): per-call latency by the wall
# clock, synchronised on both sides as time_recorder does there (example/test_cache_fetch.py:9-22)

def wall_us(fn, reps):
    """Median wall-clock microseconds of fn(), device idle before and after each call."""
    import torch
    fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        ts.append((time.perf_counter() - t0) * 1e6)
    ts.sort()
    return round(ts[len(ts) // 2], 1)


def bench_ref_harness(capi, args, result):
    import torch
    res = {}
    g = torch.Generator().manual_seed(123)
    sizes = [10, 100, 1000, 10_000, 100_000, 300_000, 1_000_000]

    def reps_for(n):
        return 200 if n <= 10_000 else 30

    # example/test_cache_fetch.py:108-154: 1,000,000 x 128 f32, 90 % of the ids cached in random order
    N, D = 1_000_000, 128
    data = torch.randn(N, D, generator=g).pin_memory()
    full_gpu = data.cuda()
    ids = torch.randperm(N, generator=g)[: int(N * 0.9)].cuda()
    cache = full_gpu[ids].contiguous()
    hmap = capi.CUCOStaticHashmap(ids, torch.arange(ids.numel(), device="cuda"), 0.8)
    fetch = {"map_layout": hmap.layout(), "by_queries": {}}
    for n in sizes:
        q = torch.randint(0, N, (n,), generator=g).cuda()
        q_cpu = q.cpu()
        a = capi.cache_fetch(data, cache, q, hmap)
        assert torch.equal(a, full_gpu[q]) and torch.equal(a, capi.uva_fetch(data, q))
        r = reps_for(n)
        row = {"cache_fetch_us": wall_us(lambda: capi.cache_fetch(data, cache, q, hmap), r),
               "uva_fetch_us": wall_us(lambda: capi.uva_fetch(data, q), r),
               "mask_fetch_us": wall_us(lambda: capi.cache_fetch_with_mask(data, cache, q, hmap.query(q)), r),
               "gpu_index_us": wall_us(lambda: full_gpu[q], r),
               "gpu_index_select_us": wall_us(lambda: torch.index_select(full_gpu, 0, q), r)}
        if not args.no_cpu:
            row["cpu_fetch_us"] = wall_us(lambda: data[q_cpu].cuda(), 5 if n >= 100_000 else 30)
        fetch["by_queries"][str(n)] = row
    res["fetch_1M_x_128_f32_90pct_cached"] = fetch

    # what a call costs the host (queued back to back, no synchronisation): the floor of the small-n rows
    # above is one launch plus the synchronisation, and the operator's own share of it is this
    def host_us(fn, n=2000):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        t = (time.perf_counter() - t0) / n * 1e6
        torch.cuda.synchronize()
        return round(t, 2)
    q10 = torch.randint(0, N, (10,), generator=g).cuda()
    res["host_cost_per_call_us_10_queries"] = {
        "cache_fetch_pinned_table": host_us(lambda: capi.cache_fetch(data, cache, q10, hmap)),
        "cache_fetch_device_table": host_us(lambda: capi.cache_fetch(full_gpu, cache, q10, hmap)),
        "uva_fetch_pinned_table": host_us(lambda: capi.uva_fetch(data, q10)),
        "hashmap_query": host_us(lambda: hmap.query(q10)),
        "torch_index": host_us(lambda: full_gpu[q10]),
        "torch_index_select": host_us(lambda: torch.index_select(full_gpu, 0, q10)),
        "torch_empty_output_only": host_us(lambda: torch.empty((10, D), device="cuda"))}
    del cache, hmap, ids

    # example/test_cache_set.py:150-194: the same table, every id cached in random order
    ids = torch.randperm(N, generator=g).cuda()
    cache = full_gpu[ids].contiguous()
    hmap = capi.CUCOStaticHashmap(ids, torch.arange(N, device="cuda"), 0.8)
    sets = {"map_layout": hmap.layout(), "by_updates": {}}
    for n in sizes:
        idx = torch.randint(0, N, (n,), generator=g).cuda().unique()
        upd = torch.randn(idx.numel(), D, generator=g).cuda()
        r = reps_for(n)
        row = {"rows": idx.numel(),
               "cache_set_us": wall_us(lambda: capi.cache_set(data, cache, idx, upd, hmap), r),
               "uva_set_us": wall_us(lambda: capi.uva_set(data, idx, upd), r),
               "mask_set_us": wall_us(lambda: capi.cache_set_with_mask(data, cache, idx, upd, hmap.query(idx)), r),
               "gpu_index_put_us": wall_us(lambda: full_gpu.index_put_((idx,), upd), r)}
        assert torch.equal(capi.cache_fetch(data, cache, idx, hmap), upd)
        sets["by_updates"][str(n)] = row
    res["set_1M_x_128_f32_all_cached"] = sets
    del cache, hmap, ids, full_gpu, data

    # example/simple_bench.py:6-34: ~950,000 distinct int32 keys below 10,000,000, 1,000,000 int32 requests
    keys = torch.randint(0, 10_000_000, (1_000_000,), generator=g).int().unique().cuda()
    vals = torch.arange(keys.numel(), dtype=torch.int32, device="cuda")
    req = torch.randint(0, 10_000_000, (1_000_000,), generator=g).int().cuda()
    by_lf = {}
    for lf in (0.1, 0.2, 0.3, 0.4, 0.5, 0.6, 0.7, 0.8, 0.9, 0.99, 1.0):
        # (sorted keys with consecutive values would make the constructor choose its rank bitmap: the general
        # table is timed beside the layout it picks)
        row = {}
        for layout in ("auto", "buckets"):
            m = capi.CUCOStaticHashmap(keys, vals, lf, layout=layout)
            row[layout] = {"layout": m.layout(), "query_us": wall_us(lambda: m.query(req), 50),
                           "table_bytes": m.memory_usage()}
            del m
        by_lf[str(lf)] = row
    res["hashmap_query_1M_int32_by_load_factor"] = by_lf
    del keys, vals, req

    # example/test_cache_sampling.py:167-221: 2,000,000 rows of degree U[0, 1000), int64 CSR, the top 30 % by
    # degree cached, 5 picks without replacement; the reference times 50 calls per entry, here one call
    if not args.harness_skip_sampling:
        deg = torch.randint(0, 1000, (2_000_000,), generator=g)
        indptr = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(deg, 0)])
        nnz = int(indptr[-1])
        indices = torch.empty(nnz, dtype=torch.int64, pin_memory=True)
        torch.arange(nnz, out=indices)
        indptr = indptr.pin_memory()
        gpu_full_p, gpu_full_i = indptr.cuda(), indices.cuda()
        hot = torch.sort(deg, descending=True).indices[: int(2_000_000 * 0.3)].cuda()
        gp, gi = capi.create_subcsr(indptr, indices, hot)
        hmap = capi.CUCOStaticHashmap(hot, torch.arange(hot.numel(), device="cuda"), 0.8)
        samp = {"map_layout": hmap.layout(), "edges": nnz, "by_seeds": {}}
        for n in [10, 100, 1000, 10_000, 100_000, 300_000, 500_000]:
            seeds = torch.randperm(2_000_000, generator=g)[:n].cuda()
            r = reps_for(n)
            samp["by_seeds"][str(n)] = {
                "gpu_us": wall_us(lambda: capi.csr_sampling(gpu_full_p, gpu_full_i, seeds, 5, False), r),
                "uva_us": wall_us(lambda: capi.csr_sampling(indptr, indices, seeds, 5, False), r),
                "cache_us": wall_us(lambda: capi.csr_cache_sampling(indptr, indices, gp, gi, hmap, seeds, 5, False), r)}
        res["sampling_2M_rows_deg_u1000_k5_30pct_cached"] = samp
    result["extra"]["ref_harness"] = res


def probe_granularity(capi, args, result):
    """Random rows of 16/32/64/128 bytes from a 4 GiB HBM table: run under
    rocprofv3 --pmc FETCH_SIZE to see how many bytes one small random read costs."""
    import torch
    q_n = 1 << 22
    res = {}
    for rb in (16, 32, 64, 128):
        n = (1 << 32) // rb
        tab = torch.empty((n, rb), device="cuda", dtype=torch.uint8)
        q = torch.randint(0, n, (q_n,), device="cuda")
        t = gpu_time_ms(lambda: capi.uva_fetch(tab, q), 3, warmup=1)
        res["row_bytes_%d" % rb] = {"rows": q_n, "ms": round(t["median"], 4)}
        del tab
    result["extra"]["granularity_probe"] = res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workloads", default="fetch,hashmap,scan,harness,sampling,e2e")
    ap.add_argument("--harness-skip-sampling", action="store_true",
                    help="harness workload: leave out the 8 GB sampling graph of example/test_cache_sampling.py")
    ap.add_argument("--fetch-rows", type=int, default=100_000_000)
    ap.add_argument("--sampling-scale", type=int, default=21)
    ap.add_argument("--sampling-batches", type=int, default=50)
    ap.add_argument("--e2e-scale", type=int, default=24)
    ap.add_argument("--e2e-batches", type=int, default=24)
    ap.add_argument("--e2e-operators-only", action="store_true",
                    help="e2e workload: only the batches issued operator by operator (no fused, pipelined or "
                         "prefetching forms)")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--headline-map", default="buckets", choices=["buckets", "auto"],
                    help="with --headline-only: which map's launches to run (for profiler runs)")
    ap.add_argument("--headline-only", action="store_true",
                    help="fetch workload: only the timed config-4 steps (used for profiler runs, so that "
                         "every launch of the fetch kernel in the trace belongs to the headline workload)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import torch
    import shmtensor_amd
    capi = shmtensor_amd.install_aliases()        # raises if the HIP extension is missing
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    torch.cuda.set_device(0)

    result = {"metric": "cache-fetch GB/s + sampled edges/sec on 1 MI355X; % of HBM / host-link roofline",
              "value": None, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
              "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
              "dtype": "u8", "data": "synthetic", "config": {"workload": None},
              "roofline": None, "cpu_baseline": None,
              "extra": {"host_threads": {"os_cpu_count": os.cpu_count(), "torch": torch.get_num_threads(),
                                         "OMP_NUM_THREADS": os.environ.get("OMP_NUM_THREADS")}}}
    todo = args.workloads.split(",")
    if "fetch" in todo:
        bench_fetch(capi, args, result)
        torch.cuda.empty_cache()
    if "fetch" in todo and not args.headline_only:
        bench_fetch_small(capi, args, result)
    if "hashmap" in todo:
        bench_hashmap(capi, args, result)
        torch.cuda.empty_cache()
    if "hashmap_sweep" in todo:
        bench_hashmap_sweep(capi, args, result)
    if "scan" in todo:
        bench_scan(capi, args, result)
    if "granularity" in todo:
        probe_granularity(capi, args, result)
    if "harness" in todo:
        bench_ref_harness(capi, args, result)
        torch.cuda.empty_cache()
    if "sampling" in todo:
        bench_sampling(capi, args, result)
        s = result["extra"]["sampling_config3"]
        # config 3 through the reference's operators, one batch at a time; and through sample_blocks with
        # batches sharing their launches (what the dataloader's prefetch= uses)
        result["sampled_edges_per_s"] = s["sampled_edges_per_s"]
        result["sampled_edges_per_s_batches_sharing_launches"] = max(
            v["sampled_edges_per_s"] for v in s["sample_blocks_batches_in_flight"].values())
    if "e2e" in todo:
        torch.cuda.empty_cache()
        bench_e2e(capi, args, result)
    # the figures a reader wants without digging through `extra`, and `extra` last
    extra = result.pop("extra")
    summary = {}
    by_map = extra.get("fetch_all_hit_by_map_layout")
    if by_map:
        summary["fetch_all_hit_frac_hbm_peak_by_map_layout"] = dict(
            {k: v["frac_hbm_peak"] for k, v in by_map.items()},
            id_range=extra["fetch_all_hit"]["frac_hbm_peak"], mask=extra["fetch_all_hit_with_mask"]["frac_hbm_peak"])
    if "scan" in extra:
        summary["scan_frac_hbm_peak"] = {"exclusive_int64": extra["scan"]["exclusive_int64_16777216"]["frac_hbm_peak"],
                                         "inclusive_int32": extra["scan"]["thrust_scan_int32_16777216"]["frac_hbm_peak"]}
    if "hashmap_config2" in extra:
        summary["hashmap_query_line_traffic_frac_hbm_peak"] = extra["hashmap_config2"]["query_line_traffic_frac_hbm_peak"]
    if "sampling_config3" in extra:
        s3 = extra["sampling_config3"]
        summary["config3_ms_per_batch"] = {"operators": s3["ms_per_batch"], "fused_hop": s3["fused_hop_ms_per_batch"],
                                           "chained_hops": s3["chained_hops_ms_per_batch"],
                                           "batches_sharing_launches": min(
                                               v["ms_per_batch"] for v in s3["sample_blocks_batches_in_flight"].values())}
        speedups = {k: s3[k] for k in ("speedup_vs_cpu", "speedup_vs_cpu_chained_hops",
                                       "speedup_vs_cpu_batches_sharing_launches") if k in s3}
        if speedups:
            summary["config3_speedup_vs_fastest_cpu_baseline"] = speedups
    if "e2e_config5" in extra:
        e5 = extra["e2e_config5"]
        summary["config5_ms_per_batch"] = {"operators": e5["batch_ms_wall"], "sample_relabel": e5["sample_relabel_ms"],
                                           "fetch": e5["fetch_ms"]}
        if e5["sample_blocks_fetch_batch_ms_wall_by_batches_in_flight"]:
            summary["config5_ms_per_batch"]["sampler_and_fetch_pipelined"] = min(
                e5["sample_blocks_fetch_batch_ms_wall_by_batches_in_flight"].values())
    if summary:
        result["summary"] = summary
    result["extra"] = extra
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
