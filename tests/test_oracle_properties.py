"""Property tests (hypothesis) of the CPU oracle against closed forms: random
sizes, dtypes, load factors and duplicates rather than hand-picked cases."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

pytest.importorskip("hypothesis")

SETTINGS = dict(max_examples=60, deadline=None)
int_dtypes = st.sampled_from([np.int32, np.int64])


@settings(**SETTINGS)
@given(keys=st.lists(st.integers(0, 2**31 - 2), min_size=0, max_size=300, unique=True),
       extra=st.lists(st.integers(-1, 2**31 - 2), min_size=0, max_size=100),
       kd=int_dtypes, vd=int_dtypes, lf=st.floats(0.05, 1.0))
def test_hashmap_is_a_dict(oracle, keys, extra, kd, vd, lf):
    k = np.array(keys, dtype=kd)
    v = np.arange(k.size, dtype=vd) * 3 + 1
    h = oracle.Hashmap(k, v, lf)
    table = dict(zip(k.tolist(), v.tolist()))
    req = np.array(keys[::2] + extra, dtype=np.int64)
    assert h.query(req).tolist() == [table.get(int(r), -1) for r in req]
    assert h.capacity() == int(np.ceil(k.size / lf))


@settings(**SETTINGS)
@given(parts=st.lists(st.lists(st.integers(0, 40), max_size=60), min_size=1, max_size=4), dt=int_dtypes,
       offset=st.sampled_from([0, 2**31, 2**40]))
def test_relabel_is_first_occurrence_order(oracle, parts, dt, offset):
    if dt == np.int32:
        offset = 0
    arrays = [np.array(p, dtype=dt) + offset for p in parts]
    uniq, labels = oracle.relabel(arrays)
    total = np.concatenate(arrays).tolist()
    first = {}
    for x in total:
        first.setdefault(x, len(first))
    assert uniq.tolist() == list(first.keys())
    assert np.concatenate(labels).tolist() == [first[x] for x in total]
    assert [l.size for l in labels] == [a.size for a in arrays]


@settings(**SETTINGS)
@given(vals=st.lists(st.integers(-2**31, 2**31 - 1), max_size=300), dt=int_dtypes)
def test_scans_wrap_like_numpy(oracle, vals, dt):
    a = np.array(vals, dtype=dt)
    expect = np.concatenate([[0], np.cumsum(a, dtype=dt)])[: a.size].astype(dt)
    assert np.array_equal(oracle.exclusive_scan(a), expect)
    a32 = a.astype(np.int32)
    assert np.array_equal(oracle.inclusive_scan_i32(a32), np.cumsum(a32, dtype=np.int32))


@settings(**SETTINGS)
@given(degs=st.lists(st.integers(0, 30), min_size=1, max_size=40), k=st.integers(0, 35), replace=st.booleans(),
       seed=st.integers(0, 2**32), algo=st.sampled_from(["reservoir", "floyd"]), data=st.data())
def test_sampling_contract(oracle, degs, k, replace, seed, algo, data):
    """sub_indptr = exclusive scan of the per-seed counts; deg <= k segments are the
    adjacency in CSR order; otherwise k distinct neighbours (no replacement) or k
    neighbours (replacement); the cached and the uncached call agree under the device rule."""
    n = len(degs)
    indptr = np.concatenate([[0], np.cumsum(degs)]).astype(np.int64)
    indices = np.arange(indptr[-1], dtype=np.int64) * 7 % 1000003          # distinct within a row
    seeds = np.array(data.draw(st.lists(st.integers(0, n - 1), min_size=0, max_size=50)), dtype=np.int64)
    sp, si = oracle.sample(indptr, indices, seeds, k, replace, seed=seed, algo=algo)
    deg = np.array(degs)[seeds] if seeds.size else np.zeros(0, int)
    cnt = np.where(deg > 0, k, 0) if replace else np.minimum(deg, k)
    assert sp.tolist() == np.concatenate([[0], np.cumsum(cnt)]).tolist()
    for s, v in enumerate(seeds):
        seg = si[sp[s]:sp[s + 1]]
        adj = indices[indptr[v]:indptr[v + 1]]
        assert np.isin(seg, adj).all()
        if not replace:
            if adj.size <= k:
                assert seg.tolist() == adj.tolist()
            else:
                assert np.unique(seg).size == k
    if algo == "floyd" and n >= 2:
        rows = np.arange(0, n, 2)
        gp, gi = oracle.create_subcsr(indptr, indices, rows)
        cache = (gp, gi, oracle.Hashmap(rows, np.arange(rows.size), 0.8))
        sp2, si2 = oracle.sample(indptr, indices, seeds, k, replace, cache=cache, seed=seed, algo=algo)
        assert np.array_equal(sp, sp2) and np.array_equal(si, si2)


def test_zipf_generator_follows_the_exact_law():
    """The benchmark's query stream: ranks must follow P(r) ~ (r + 1)^-s exactly at the head (where almost
    all of the mass and all of the repetition is) and within sampling noise in the tail. Chi-square over the
    first 30 ranks one by one plus geometric buckets up to the last rank, against pmf values summed directly."""
    import torch
    from shmtensor_amd.synthetic import zipf_ranks
    for num_items, s, head in ((200_000, 1.1, 1 << 20), (200_000, 1.1, 1000), (50_000, 0.8, 64)):
        n = 2_000_000
        r = zipf_ranks(n, num_items, s, seed=3, device="cpu", head=head).numpy()
        assert r.min() >= 0 and r.max() < num_items
        pmf = np.arange(1, num_items + 1, dtype=np.float64) ** -s
        pmf /= pmf.sum()
        edges = list(range(0, 31)) + [int(x) for x in np.unique(np.geomspace(31, num_items, 40).astype(np.int64))]
        edges[-1] = num_items
        observed = np.histogram(r, bins=edges)[0]
        expected = np.add.reduceat(pmf, edges[:-1]) * n
        chi2 = ((observed - expected) ** 2 / expected).sum()
        dof = len(edges) - 2
        assert chi2 < dof + 6 * np.sqrt(2 * dof), (num_items, s, head, chi2, dof)
        # rank 0 alone: the continuous approximation that the exact head replaces is off by +11 % here
        assert abs(observed[0] / n - pmf[0]) < 4 * np.sqrt(pmf[0] / n)
