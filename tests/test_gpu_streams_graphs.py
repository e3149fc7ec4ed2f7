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
