"""Operators follow torch's current stream, and the ones without a
data-dependent output size can be captured into a HIP graph and replayed."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cache(capi):
    torch.manual_seed(0)
    data = torch.randn(20000, 128).pin_memory()
    ids = torch.randperm(20000)[:5000].cuda()
    gpu = data[ids.cpu()].cuda()
    h = capi.CUCOStaticHashmap(ids, torch.arange(5000).cuda(), 0.8)
    return data, gpu, ids, h


def test_operators_run_on_the_current_stream(capi, cache):
    data, gpu, ids, h = cache
    q = torch.randint(0, 20000, (4096,)).cuda()
    indptr = torch.arange(0, 20001 * 4, 4).cuda()
    indices = torch.arange(20000 * 4).int().cuda()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        out = capi.cache_fetch(data, gpu, q, h)
        uniq, (labels,) = capi.tensor_relabel([q])
        sp, si = capi.csr_sampling(indptr, indices, q, 3, False)
        slots = h.query(q)
    side.synchronize()
    assert torch.equal(out, data[q.cpu()].cuda())
    assert torch.equal(uniq[labels], q)
    assert torch.equal(sp, torch.arange(4097).cuda() * 3) and si.numel() == 4096 * 3
    expect = torch.full((20000,), -1).cuda()
    expect[ids] = torch.arange(5000).cuda()
    assert torch.equal(slots, expect[q])


def test_fetch_query_and_set_replay_in_a_hip_graph(capi, cache):
    data, gpu, ids, h = cache
    gpu = gpu.clone()
    static_q = torch.randint(0, 20000, (4096,)).cuda()
    static_upd = torch.zeros(128, 128).cuda()
    static_rows = ids[:128].clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        capi.cache_set(data, gpu, static_rows, static_upd, h)
        static_out = capi.cache_fetch(data, gpu, static_q, h)
        static_slots = h.query(static_q)
    lut = torch.full((20000,), -1).cuda()
    lut[ids] = torch.arange(5000).cuda()
    for it in range(4):          # replays with eager work and synchronisations in between
        q = torch.randint(0, 20000, (4096,)).cuda()
        upd = torch.randn(128, 128).cuda()
        static_q.copy_(q)
        static_upd.copy_(upd)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        expect_cache = data[ids.cpu()].cuda()
        expect_cache[:128] = upd
        slot = lut[q]
        expect = torch.where((slot >= 0).unsqueeze(1), expect_cache[slot.clamp(min=0)], data[q.cpu()].cuda())
        assert torch.equal(static_out, expect), it
        assert torch.equal(static_slots, slot), it
        assert float(static_out.abs().sum()) > 0


def test_one_pass_scans_replay_in_a_hip_graph(capi, cabi):
    """thrust_scan (workspace from the shim), shmt_exclusive_scan with a caller's workspace and the form
    without a workspace, each over several tiles, recorded once and replayed on new data: the kernels clear
    the published sums they use with a kernel of their own, so every replay starts clean."""
    lib = cabi.load()
    n = 3_000_017
    static_a = torch.zeros(n, dtype=torch.int32).cuda()
    static_b = torch.zeros(n, dtype=torch.int64).cuda()
    static_c = torch.zeros(n, dtype=torch.int64).cuda()
    tmp = torch.empty(lib.shmt_scan_tmp_bytes(n), dtype=torch.uint8).cuda()
    cabi.check(lib.shmt_exclusive_scan_noalloc(None, 0, 8, cabi.current_stream()))     # set-up call outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        capi.thrust_scan(static_a)
        cabi.check(lib.shmt_exclusive_scan(static_b.data_ptr(), n, 8, tmp.data_ptr(), tmp.numel(), cabi.current_stream()))
        cabi.check(lib.shmt_exclusive_scan_noalloc(static_c.data_ptr(), n, 8, cabi.current_stream()))
    g = torch.Generator(device="cuda").manual_seed(3)
    for it in range(4):
        a = torch.randint(-1000, 1000, (n,), device="cuda", generator=g, dtype=torch.int32)
        b = torch.randint(0, 2**40, (n,), device="cuda", generator=g)
        static_a.copy_(a)
        static_b.copy_(b)
        static_c.copy_(b)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_a, torch.cumsum(a, 0, dtype=torch.int32)), it
        assert torch.equal(static_b, torch.cumsum(b, 0) - b), it
        assert torch.equal(static_c, static_b), it
        torch.zeros(1000, device="cuda").sum()       # eager work between the replays


def test_fused_hop_replays_in_a_hip_graph(capi, cabi):
    """shmt_sample_hop never waits for the host (sizes go to device memory here), so the whole hop can be
    captured once and replayed on new seeds: every replay is compared with the eager operator, with eager
    work and synchronisations in between. One replay feeds ids beyond 32 bits (the relabel then switches
    table format inside the captured kernels) and the next goes back."""
    from shmtensor_amd.synthetic import rmat_csr
    lib = cabi.load()
    indptr, indices = rmat_csr(13, 12, seed=3)
    indices = indices.long()
    n = indptr.numel() - 1
    S, k = 3000, 8
    n_max = S + S * k
    seeds = torch.zeros(S, dtype=torch.int64, device="cuda")
    graph_indices = indices.clone()
    buf = dict(sp=torch.empty(S + 1, dtype=torch.int64, device="cuda"), si=torch.empty(S * k, dtype=torch.int64, device="cuda"),
               plan=torch.empty(lib.shmt_sample_plan_bytes(S), dtype=torch.uint8, device="cuda"),
               total=torch.empty(n_max, dtype=torch.int64, device="cuda"), unique=torch.empty(n_max, dtype=torch.int64, device="cuda"),
               labels=torch.empty(n_max, dtype=torch.int64, device="cuda"),
               scratch=torch.empty(lib.shmt_relabel_scratch_bytes(n_max), dtype=torch.uint8, device="cuda"),
               nnz=torch.zeros(1, dtype=torch.int64, device="cuda"), count=torch.zeros(1, dtype=torch.int64, device="cuda"))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cabi.check(lib.shmt_sample_hop(indptr.data_ptr(), 8, graph_indices.data_ptr(), 8, None, None, None, seeds.data_ptr(), 8,
                                       S, k, 0, 5, 2, buf["sp"].data_ptr(), buf["si"].data_ptr(), buf["plan"].data_ptr(),
                                       buf["plan"].numel(), 8, buf["total"].data_ptr(), buf["scratch"].data_ptr(),
                                       buf["scratch"].numel(), buf["unique"].data_ptr(), buf["labels"].data_ptr(),
                                       buf["nnz"].data_ptr(), buf["count"].data_ptr(), cabi.current_stream()))
    g = torch.Generator().manual_seed(12)
    for it in range(5):
        seeds.copy_(torch.randperm(n, generator=g)[:S])
        graph_indices.copy_(indices)
        if it == 2:
            graph_indices[::3] += 1 << 33          # ids that need the 16-byte table format
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = capi.sample_hop(indptr, graph_indices, None, None, None, seeds, k, False, seed=5, stream_id=2)
        nnz, u = int(buf["nnz"].item()), int(buf["count"].item())
        assert nnz == want[1].numel() and u == want[2].numel(), it
        assert torch.equal(buf["sp"], want[0]) and torch.equal(buf["si"][:nnz], want[1]), it
        assert torch.equal(buf["unique"][:u], want[2]) and torch.equal(buf["labels"][S:S + nnz], want[3]), it


def test_a_whole_batch_of_chained_hops_replays_in_a_hip_graph(capi, cabi):
    """Three hops chained on the device (each takes its seeds and their number from the hop before) are
    captured as ONE graph and replayed on new seed batches; every replay equals sample_blocks run eagerly."""
    from shmtensor_amd.synthetic import rmat_csr
    lib = cabi.load()
    indptr, indices = rmat_csr(13, 12, seed=5)
    n = indptr.numel() - 1
    S, picks = 500, (3, 4, 6)
    seeds = torch.zeros(S, dtype=torch.int64, device="cuda")
    hops, s_max = [], S
    for k in picks:
        n_max = s_max + s_max * k
        hops.append(dict(s_max=s_max, k=k,
                         sp=torch.empty(s_max + 1, dtype=torch.int64, device="cuda"),
                         si=torch.empty(s_max * k, dtype=indices.dtype, device="cuda"),
                         plan=torch.empty(lib.shmt_sample_plan_bytes(s_max), dtype=torch.uint8, device="cuda"),
                         total=torch.empty(n_max, dtype=torch.int64, device="cuda"),
                         unique=torch.empty(n_max, dtype=torch.int64, device="cuda"),
                         labels=torch.empty(n_max, dtype=torch.int64, device="cuda"),
                         scratch=torch.empty(lib.shmt_relabel_scratch_bytes(n_max), dtype=torch.uint8, device="cuda"),
                         nnz=torch.zeros(1, dtype=torch.int64, device="cuda"), count=torch.zeros(1, dtype=torch.int64, device="cuda"),
                         count_dev=torch.zeros(1, dtype=torch.int64, device="cuda")))
        s_max = n_max
    ib = indices.element_size()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        src, src_len = seeds, None
        for hop, b in enumerate(hops):
            cabi.check(lib.shmt_sample_hop_chained(
                indptr.data_ptr(), 8, indices.data_ptr(), ib, None, None, None, src.data_ptr(), 8, b["s_max"], src_len,
                b["k"], 0, 77, None, hop, b["sp"].data_ptr(), b["si"].data_ptr(), b["plan"].data_ptr(), b["plan"].numel(), 8,
                b["total"].data_ptr(), b["scratch"].data_ptr(), b["scratch"].numel(), b["unique"].data_ptr(),
                b["labels"].data_ptr(), b["nnz"].data_ptr(), b["count"].data_ptr(), b["count_dev"].data_ptr(),
                cabi.current_stream()))
            src, src_len = b["unique"], b["count_dev"].data_ptr()
    g = torch.Generator().manual_seed(3)
    for it in range(4):
        seeds.copy_(torch.randperm(n, generator=g)[:S])
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = capi.sample_blocks(indptr, indices, None, None, None, [seeds], list(picks), False, seeds_rng=[77])[0]
        s_now = S
        for b, (sp, si, uniq, rel) in zip(hops, want):
            nnz, u = int(b["nnz"].item()), int(b["count"].item())
            assert (nnz, u) == (si.numel(), uniq.numel()), it
            assert torch.equal(b["sp"][:s_now + 1], sp) and torch.equal(b["si"][:nnz], si), it
            assert torch.equal(b["unique"][:u], uniq) and torch.equal(b["labels"][s_now:s_now + nnz], rel), it
            s_now = u
