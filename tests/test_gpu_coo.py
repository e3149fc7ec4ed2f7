"""Blocks in coordinate form (create_block_from_coo, python/shmtensor/sampling.py:21-27):
with coo=True a hop also returns, per sampled id, the position of the seed it was sampled
for. (row, col) = (relabel_indices, coo_dst) must be the edge list of the block whose CSC
form is (sub_indptr, relabel_indices): col == repeat_interleave(arange(S), diff(sub_indptr)).
Checked through sample_hop, sample_blocks (merged launches, host threads, chained and
unchained hops), sample_blocks_fetch, the dataloader and the raw C ABI, and against the
CPU oracle's pipeline."""
import numpy as np
import pytest
import torch

from shmtensor_amd.synthetic import rmat_csr

pytestmark = pytest.mark.gpu


def _expand(sub_indptr, dtype):
    s = sub_indptr.numel() - 1
    return torch.repeat_interleave(torch.arange(s, device=sub_indptr.device), sub_indptr.diff()).to(dtype)


def _check_hop(hop5, hop4):
    assert len(hop5) == 5 and len(hop4) == 4
    for a, b in zip(hop5[:4], hop4):
        assert a.dtype == b.dtype and torch.equal(a, b)              # asking for COO changes nothing else
    sp, _, uniq, row, col = hop5
    assert col.dtype == row.dtype and col.shape == row.shape and col.is_cuda
    assert torch.equal(col, _expand(sp, row.dtype))
    if row.numel():
        assert int(row.max()) < uniq.numel() and int(col.max()) < sp.numel() - 1


@pytest.fixture(scope="module")
def graph():
    indptr, indices = rmat_csr(15, 12, seed=9)
    return indptr, indices


def _cache(capi, indptr, indices, frac=4):
    n = indptr.numel() - 1
    hot = torch.randperm(n, generator=torch.Generator().manual_seed(1))[: n // frac].cuda()
    gp, gi = capi.create_subcsr(indptr, indices, hot)
    h = capi.CUCOStaticHashmap(hot.int(), torch.arange(hot.numel(), dtype=torch.int32).cuda(), 0.8)
    return gp, gi, h


@pytest.mark.parametrize("replace", [False, True])
@pytest.mark.parametrize("k", [1, 5, 25, 64, 100])
@pytest.mark.parametrize("seed_dt", [torch.int32, torch.int64])
def test_sample_hop_coo(capi, oracle, graph, replace, k, seed_dt):
    indptr, indices = graph
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(k)
    for S in (1, 7, 300, 1025, 6000):                                # one-workgroup and tiled plans, small relabel
        seeds = torch.randint(0, n, (S,), generator=g).to(seed_dt).cuda()
        plain = capi.sample_hop(indptr, indices, None, None, None, seeds, k, replace, seed=5, stream_id=2)
        coo = capi.sample_hop(indptr, indices, None, None, None, seeds, k, replace, seed=5, stream_id=2, coo=True)
        _check_hop(coo, plain)
    # against the oracle's pipeline: sample, relabel, expand
    sp, si = oracle.sample(indptr.cpu().numpy(), indices.cpu().numpy(), seeds.cpu().numpy(), k, replace, seed=5,
                           stream=2, algo="floyd")
    _, (_, lab) = oracle.relabel([seeds.cpu().numpy().astype(np.int64), si.astype(np.int64)])
    assert np.array_equal(coo[3].cpu().numpy(), lab.astype(coo[3].cpu().numpy().dtype))
    assert np.array_equal(coo[4].cpu().numpy(), np.repeat(np.arange(S), np.diff(sp)))


def test_sample_hop_coo_degenerate(capi):
    indptr = torch.tensor([0, 3, 3, 4]).cuda()                       # node 1 has no neighbours
    indices = torch.tensor([2, 1, 0, 2]).cuda()
    empty = torch.empty(0, dtype=torch.int64).cuda()
    out = capi.sample_hop(indptr, indices, None, None, None, empty, 5, False, coo=True)
    assert len(out) == 5 and out[4].numel() == 0
    out = capi.sample_hop(indptr, indices, None, None, None, torch.tensor([1, 1, 0, 2]).cuda(), 2, False, coo=True)
    assert out[0].tolist() == [0, 0, 0, 2, 3] and out[4].tolist() == [2, 2, 3]
    out = capi.sample_hop(indptr, indices, None, None, None, torch.tensor([0, 2]).cuda(), 0, False, coo=True)
    assert len(out) == 5 and out[4].numel() == 0                     # no picks: the two separate operators ran


@pytest.mark.parametrize("cached", [False, True])
@pytest.mark.parametrize("picks", [[5, 10, 15], [10, 25], [3, 3, 3, 3]])
def test_sample_blocks_coo(capi, graph, cached, picks):
    indptr, indices = graph
    indptr, indices = indptr.cpu().pin_memory(), indices.cpu().pin_memory()
    n = indptr.numel() - 1
    gp, gi, h = _cache(capi, indptr, indices) if cached else (None, None, None)
    gen = torch.Generator().manual_seed(4)
    batches = [torch.randperm(n, generator=gen)[:256 + 64 * b].cuda() for b in range(9)]
    rng = list(range(50, 59))
    plain = capi.sample_blocks(indptr, indices, gp, gi, h, batches, picks, False, seeds_rng=rng, max_in_flight=1)
    for in_flight in (1, 4, 8):                                     # one by one, merged launches of 4 and of 8 (+1)
        got = capi.sample_blocks(indptr, indices, gp, gi, h, batches, picks, False, seeds_rng=rng,
                                 max_in_flight=in_flight, coo=True)
        assert len(got) == len(batches)
        for hops5, hops4 in zip(got, plain):
            assert len(hops5) == len(picks)
            for a, b in zip(hops5, hops4):
                _check_hop(a, b)


def test_sample_blocks_coo_when_the_last_hop_does_not_chain(capi, graph):
    """4,096 seeds with fanouts [10, 15, 25]: the bound of the third hop (4,096 x 11 x 16 x 26 ids) is
    beyond what is queued ahead of its seed count, so batches run hop by hop on host threads."""
    indptr, indices = graph
    n = indptr.numel() - 1
    gen = torch.Generator().manual_seed(6)
    batches = [torch.randperm(n, generator=gen)[:4096].cuda() for _ in range(3)]
    plain = capi.sample_blocks(indptr, indices, None, None, None, batches, [10, 15, 25], False, max_in_flight=2)
    got = capi.sample_blocks(indptr, indices, None, None, None, batches, [10, 15, 25], False, max_in_flight=2,
                             coo=True)
    for hops5, hops4 in zip(got, plain):
        for a, b in zip(hops5, hops4):
            _check_hop(a, b)


def test_sample_blocks_fetch_coo(capi, graph):
    indptr, indices = graph
    n = indptr.numel() - 1
    table = torch.randn(n, 12, generator=torch.Generator().manual_seed(3)).pin_memory()
    batches = [torch.arange(b * 200, b * 200 + 200).cuda() for b in range(4)]
    plain = capi.sample_blocks_fetch(indptr, indices, None, None, None, batches, [4, 6], False, table, None, None)
    got = capi.sample_blocks_fetch(indptr, indices, None, None, None, batches, [4, 6], False, table, None, None,
                                   coo=True)
    for (hops5, x5), (hops4, x4) in zip(got, plain):
        assert torch.equal(x5, x4)
        for a, b in zip(hops5, hops4):
            _check_hop(a, b)


@pytest.mark.parametrize("ptr_bytes,out_bytes", [(8, 8), (8, 4), (4, 4), (4, 8)])
def test_csr_rows_c_abi(cabi, ptr_bytes, out_bytes):
    """shmt_csr_rows: the row of every element of a CSR structure, with empty rows, one very long row
    and chunk boundaries (2,048 elements per workgroup pass) inside and between rows."""
    lib = cabi.load()
    rng = np.random.default_rng(ptr_bytes * 10 + out_bytes)
    for lens in ([0, 0, 5, 0, 1, 0], [3], [0], [2047, 1, 2048, 0, 0, 4097], [100_000] + [0] * 50 + [1],
                 rng.integers(0, 40, size=30_000).tolist()):
        offsets = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32 if ptr_bytes == 4 else np.int64)
        nnz, S = int(offsets[-1]), len(lens)
        o = torch.from_numpy(offsets).cuda()
        out = torch.full((max(nnz, 1),), -7, dtype=torch.int32 if out_bytes == 4 else torch.int64).cuda()
        cabi.check(lib.shmt_csr_rows(o.data_ptr(), ptr_bytes, S, nnz, out.data_ptr(), out_bytes,
                                     cabi.current_stream()))
        assert np.array_equal(out.cpu().numpy()[:nnz], np.repeat(np.arange(S), lens))
        if nnz == 0:
            assert int(out[0]) == -7
    assert lib.shmt_csr_rows(None, 3, 1, 1, None, 8, None) == -1


def test_dataloader_coo_blocks(capi, graph):
    import shmtensor
    indptr, indices = graph
    seeds = torch.arange(0, 2000)
    kw = dict(batchsize=512, num_picks=[15, 10, 5], shuffle=False, rng_seed=21)
    csc = shmtensor.GPUSamplingDataloader(indptr.cpu(), indices.cpu(), seeds, **kw)
    coo = shmtensor.GPUSamplingDataloader(indptr.cpu(), indices.cpu(), seeds, block_format="coo", prefetch=4, **kw)
    n = 0
    for (a_in, a_out, a_blocks), (b_in, b_out, b_blocks) in zip(csc, coo):
        assert torch.equal(a_in, b_in) and torch.equal(a_out, b_out) and len(a_blocks) == len(b_blocks) == 3
        for x, y in zip(a_blocks, b_blocks):
            assert isinstance(y, shmtensor.sampling.COOBlock)
            assert (y.num_src, y.num_dst) == (x.num_src, x.num_dst)
            assert torch.equal(y.row, x.indices)                    # source of every edge: its label
            assert torch.equal(y.col, _expand(x.indptr, y.row.dtype))
        n += 1
    assert n == 4
    with pytest.raises(ValueError):
        shmtensor.GPUSamplingDataloader(indptr.cpu(), indices.cpu(), seeds, block_format="csr", **kw)
