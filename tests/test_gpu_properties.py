"""Property tests (hypothesis) on the GPU: random shapes, widths, load factors
and hit rates for the hashmap, fetch/set, relabel and scan operators, each
compared with the CPU oracle."""
import numpy as np
import pytest
import torch
from hypothesis import HealthCheck, given, settings, strategies as st

pytestmark = pytest.mark.gpu

SETTINGS = dict(max_examples=40, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
TORCH = {np.int32: torch.int32, np.int64: torch.int64}
np_ints = st.sampled_from([np.int32, np.int64])


def _cuda(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@settings(**SETTINGS)
@given(n=st.integers(0, 5000), nq=st.integers(0, 7000), kd=np_ints, vd=np_ints, rd=np_ints,
       lf=st.floats(0.05, 1.0), seed=st.integers(0, 2**31))
def test_hashmap_random(capi, oracle, n, nq, kd, vd, rd, lf, seed):
    rng = np.random.default_rng(seed)
    keys = rng.choice(50_000, size=n, replace=False).astype(kd)
    vals = rng.integers(0, 2**31 - 1, size=n).astype(vd)
    req = rng.integers(-1, 50_000, size=nq).astype(rd)
    h = capi.CUCOStaticHashmap(_cuda(keys), _cuda(vals), lf)
    ref = oracle.Hashmap(keys, vals, lf)
    out = h.query(_cuda(req))
    assert out.dtype == TORCH[vd]
    assert np.array_equal(out.cpu().numpy(), ref.query(req))
    assert h.capacity() == ref.capacity()


@settings(**SETTINGS)
@given(rows=st.integers(1, 3000), dims=st.lists(st.integers(1, 9), min_size=0, max_size=3),
       dtype=st.sampled_from([torch.float32, torch.float16, torch.float64, torch.int8, torch.int16, torch.int64]),
       idt=np_ints, mdt=np_ints, q=st.integers(0, 4000), frac=st.floats(0.0, 1.0), seed=st.integers(0, 2**31))
def test_fetch_and_set_random(capi, oracle, rows, dims, dtype, idt, mdt, q, frac, seed):
    rng = np.random.default_rng(seed)
    shape = (rows, *dims)
    host = torch.from_numpy(rng.integers(-100, 100, size=shape)).to(dtype).pin_memory()
    ncache = int(rows * frac)
    ids = rng.choice(rows, size=ncache, replace=False)
    gpu = (host[torch.from_numpy(ids)].to(torch.float64) + 1).to(dtype).cuda() if ncache else \
        torch.zeros((0, *dims), dtype=dtype).cuda()
    h = capi.CUCOStaticHashmap(_cuda(ids), torch.arange(ncache).cuda(), 0.7)
    ref_h = oracle.Hashmap(ids, np.arange(ncache), 0.7)
    query = rng.integers(0, rows, size=q).astype(idt)
    view = torch.int16 if dtype == torch.float16 else dtype
    expect = oracle.fetch(host.view(view).numpy(), gpu.cpu().view(view).numpy(), query, hashmap=ref_h)
    got = capi.cache_fetch(host, gpu, _cuda(query), h)
    assert got.shape == (q, *dims) and got.dtype == dtype
    assert np.array_equal(got.cpu().view(view).numpy(), expect)
    mask = h.query(_cuda(query)).to(TORCH[mdt])
    assert np.array_equal(capi.cache_fetch_with_mask(host, gpu, _cuda(query), mask).cpu().view(view).numpy(), expect)
    # set with unique indices, then the final state of both tables must match the oracle's
    uq = np.unique(query)
    upd = torch.from_numpy(rng.integers(-100, 100, size=(uq.size, *dims))).to(dtype)
    host_ref, gpu_ref = host.view(view).numpy().copy(), gpu.cpu().view(view).numpy().copy()
    oracle.set_rows(host_ref, gpu_ref, uq, upd.view(view).numpy(), hashmap=ref_h)
    capi.cache_set(host, gpu, _cuda(uq), upd.cuda(), h)
    torch.cuda.synchronize()
    assert np.array_equal(host.view(view).numpy(), host_ref)
    assert np.array_equal(gpu.cpu().view(view).numpy(), gpu_ref)


@settings(**SETTINGS)
@given(sizes=st.lists(st.integers(0, 3000), min_size=1, max_size=5), dts=st.lists(np_ints, min_size=5, max_size=5),
       span=st.integers(1, 4000), seed=st.integers(0, 2**31))
def test_relabel_random(capi, oracle, sizes, dts, span, seed):
    rng = np.random.default_rng(seed)
    arrays = [rng.integers(0, span, size=n).astype(dt) for n, dt in zip(sizes, dts)]
    uniq, labels = capi.tensor_relabel([_cuda(a) for a in arrays])
    eu, el = oracle.relabel(arrays)
    assert uniq.dtype == TORCH[eu.dtype.type]
    assert np.array_equal(uniq.cpu().numpy(), eu)
    assert len(labels) == len(arrays)
    for l, e in zip(labels, el):
        assert np.array_equal(l.cpu().numpy(), e)


@settings(**SETTINGS)
@given(n=st.integers(0, 200_000), seed=st.integers(0, 2**31))
def test_thrust_scan_random(capi, n, seed):
    a = np.random.default_rng(seed).integers(-2**31, 2**31 - 1, size=n).astype(np.int32)
    t = _cuda(a.copy())
    capi.thrust_scan(t)
    assert np.array_equal(t.cpu().numpy(), np.cumsum(a, dtype=np.int32))
