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
